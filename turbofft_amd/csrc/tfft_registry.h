// Kernel registry entry emitted by the generator: the role of the reference's
// TurboFFT_Kernel_Entry<T, ft, err, arch>::turboFFTArr[logN][launch] function
// pointer table (include/TurboFFT.h:22-25, 118-526), keyed by tile shape
// instead of by logN.
#pragma once
#include "../../include/turbofft_kargs.h"

typedef struct tfft_kernel_entry {
    const char* name;
    const void* func;    // host-side kernel handle for hipLaunchKernel
    int datatype;        // 0 = float2, 1 = double2
    int kind;            // 0 = row1, 1 = col, 2 = rowT
    int logNi, BS, n;
    int ft;              // 0 plain, 1 fused checksums (recompute correction), 2 fused checksums with delayed batch correction
    int split;           // 1: re and im are exchanged through LDS in two rounds
    int pf;              // 1: the block prefetches its next tile (wants a persistent grid)
    int xl;              // 1: the last small-radix pass runs across lanes (DPP / ds_swizzle)
    int wv;              // > 0: compiled for this many wavefronts per SIMD
    int nt;              // bit 0: non-temporal tile loads, bit 1: non-temporal tile stores, bit 2: raised wave priority for the tile loads
    int inv;             // 1: component-swapping flavour for the first / last launch of an inverse plan
    int ck;              // > 0: reads the compact (cotangent) checksum table; 1 words kept in registers, 2 read per tile, 3 parked in LDS
    int threads;         // block size
    int lds_bytes;       // dynamic LDS
} tfft_kernel_entry;

// A fused pair: the column launch and the row launch of a two-launch plan as one kernel
// (arguments: in, out, twiddles, the two launches' tfft_kargs, tfft_fuse_args).
typedef struct tfft_pair_entry {
    const char* name;
    const void* func;
    int datatype;
    int logN1, BS1, n1, split1, nt1;    // the column launch (nt1: bit 0 only, its loads)
    int logN2, BS2, n2, split2, nt2;    // the row launch (nt2: bit 1 only, its stores)
    int threads;                        // block size (the larger of the two halves)
    int lds_bytes;                      // dynamic LDS (the larger of the two halves)
} tfft_pair_entry;

#ifdef __cplusplus
extern "C" {
#endif
const tfft_kernel_entry* tfft_kernel_table(int* count);
const tfft_pair_entry* tfft_pair_table(int* count);
#ifdef __cplusplus
}
#endif
