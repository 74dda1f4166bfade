// Device-side helpers shared by every generated kernel.
//
// The generated code is written once and compiled two ways:
//   * hipcc --offload-arch=gfx950          -> the product kernels;
//   * g++ -DTFFT_SIM (tests only)          -> a lock-step CPU execution of the
//     same phase list with bounds-checked global / LDS accessors, used to
//     catch index and barrier-placement mistakes without a GPU.
// Complex arithmetic mirrors the reference's 2-op add/sub and 4-op multiply
// (include/turbofft/macro_ops.h:14-18).
#pragma once
#include "../../include/turbofft_kargs.h"

#ifndef TFFT_SIM
#include <hip/hip_runtime.h>
#define TFFT_DEV __device__ __forceinline__
// Global memory goes through buffer instructions: the resource holds a wave-uniform base
// (tensor pointer + tile base, SGPRs), a second uniform offset rides in an SGPR and the lane
// part is ONE 32-bit VGPR shared by every access of a tile -- no per-access vector address
// arithmetic and no 64-bit address registers.  (p, ub): uniform element base; uo: uniform
// element offset; off / i: per-lane element offset.  All offsets within a tile or table are
// below 2^32 bytes.
typedef unsigned tfft_u2 __attribute__((ext_vector_type(2)));
typedef unsigned tfft_u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tfft_rsrc(const void* p) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, -1, 0x00020000);
}
// AUX is the cache-policy immediate of the instruction: 0 = default, 2 = non-temporal (nt)
template <int AUX = 0>
__device__ __forceinline__ float2 tfft_bld(const float2* p, unsigned voff, unsigned soff) {
    const tfft_u2 t = __builtin_amdgcn_raw_buffer_load_b64(tfft_rsrc(p), voff, soff, AUX);
    float2 r; r.x = __uint_as_float(t.x); r.y = __uint_as_float(t.y); return r;
}
template <int AUX = 0>
__device__ __forceinline__ double2 tfft_bld(const double2* p, unsigned voff, unsigned soff) {
    const tfft_u4 t = __builtin_amdgcn_raw_buffer_load_b128(tfft_rsrc(p), voff, soff, AUX);
    double2 r; r.x = __hiloint2double((int)t.y, (int)t.x); r.y = __hiloint2double((int)t.w, (int)t.z); return r;
}
template <int AUX = 0>
__device__ __forceinline__ void tfft_bst(float2* p, unsigned voff, unsigned soff, float2 v) {
    tfft_u2 t; t.x = __float_as_uint(v.x); t.y = __float_as_uint(v.y);
    __builtin_amdgcn_raw_buffer_store_b64(t, tfft_rsrc(p), voff, soff, AUX);
}
template <int AUX = 0>
__device__ __forceinline__ void tfft_bst(double2* p, unsigned voff, unsigned soff, double2 v) {
    tfft_u4 t;
    t.x = (unsigned)__double2loint(v.x); t.y = (unsigned)__double2hiint(v.x);
    t.z = (unsigned)__double2loint(v.y); t.w = (unsigned)__double2hiint(v.y);
    __builtin_amdgcn_raw_buffer_store_b128(t, tfft_rsrc(p), voff, soff, AUX);
}
// Two adjacent fp32 elements in one 128-bit access: for kernels whose threads hold whole
// transforms, so that a lane's elements are contiguous.  The byte address must be a multiple
// of 16: the kernels test the tensor pointer and use the one-element accesses otherwise.
template <int AUX = 0>
__device__ __forceinline__ void tfft_bld2(const float2* p, unsigned voff, unsigned soff, float2& a, float2& b) {
    const tfft_u4 t = __builtin_amdgcn_raw_buffer_load_b128(tfft_rsrc(p), voff, soff, AUX);
    a.x = __uint_as_float(t.x); a.y = __uint_as_float(t.y); b.x = __uint_as_float(t.z); b.y = __uint_as_float(t.w);
}
template <int AUX = 0>
__device__ __forceinline__ void tfft_bst2(float2* p, unsigned voff, unsigned soff, float2 a, float2 b) {
    tfft_u4 t; t.x = __float_as_uint(a.x); t.y = __float_as_uint(a.y); t.z = __float_as_uint(b.x); t.w = __float_as_uint(b.y);
    __builtin_amdgcn_raw_buffer_store_b128(t, tfft_rsrc(p), voff, soff, AUX);
}
// priority of the calling wave for instruction issue on its SIMD (0 lowest, 3 highest)
#define TFFT_WAVE_PRIO(n) __builtin_amdgcn_s_setprio(n)
#define TFFT_ESZ(p) ((unsigned)sizeof(*(p)))
#define GLDU2(p, ub, uo, off, A, B) tfft_bld2<0>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p), (A), (B))
#define GSTU2(p, ub, uo, off, A, B) tfft_bst2<0>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p), (A), (B))
#define GLDUN2(p, ub, uo, off, A, B) tfft_bld2<2>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p), (A), (B))
#define GSTUN2(p, ub, uo, off, A, B) tfft_bst2<2>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p), (A), (B))
#define GLDU(p, ub, uo, off) tfft_bld<0>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p))
#define GSTU(p, ub, uo, off, v) tfft_bst<0>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p), (v))
// the same accesses marked non-temporal: tile data is touched once, so it need not displace
// the tables in the caches
#define GLDUN(p, ub, uo, off) tfft_bld<2>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p))
#define GSTUN(p, ub, uo, off, v) tfft_bst<2>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p), (v))
// agent-scope load (sc1): served by the XCD's L2, never by the CU's own L1 -- for data that blocks on
// other CUs of the XCD wrote during this kernel
#define GLDUS(p, ub, uo, off) tfft_bld<16>((p) + (ub), (unsigned)(off) * TFFT_ESZ(p), (unsigned)(uo) * TFFT_ESZ(p))
// plain global-pointer forms of the same accesses
#define GLDG(p, ub, uo, off) (((p) + ((ub) + (uo)))[(off)])
#define GSTG(p, ub, uo, off, v) (((p) + ((ub) + (uo)))[(off)] = (v))
typedef float tfft_f2v __attribute__((ext_vector_type(2)));
typedef double tfft_d2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float2 tfft_gldn(const float2* p) {
    const tfft_f2v t = __builtin_nontemporal_load((const tfft_f2v*)p); float2 r; r.x = t.x; r.y = t.y; return r;
}
__device__ __forceinline__ double2 tfft_gldn(const double2* p) {
    const tfft_d2v t = __builtin_nontemporal_load((const tfft_d2v*)p); double2 r; r.x = t.x; r.y = t.y; return r;
}
__device__ __forceinline__ void tfft_gstn(float2* p, float2 v) {
    tfft_f2v t; t.x = v.x; t.y = v.y; __builtin_nontemporal_store(t, (tfft_f2v*)p);
}
__device__ __forceinline__ void tfft_gstn(double2* p, double2 v) {
    tfft_d2v t; t.x = v.x; t.y = v.y; __builtin_nontemporal_store(t, (tfft_d2v*)p);
}
#define GLDGN(p, ub, uo, off) tfft_gldn(((p) + ((ub) + (uo))) + (off))
#define GSTGN(p, ub, uo, off, v) tfft_gstn(((p) + ((ub) + (uo))) + (off), (v))
#define TWLG(p, i) ((p)[(i)])
#define TWLGU(p, c, i) ((p)[(c) + (i)])
#define TWLD(p, i) tfft_bld<0>((p), (unsigned)(i) * TFFT_ESZ(p), 0u)
#define TWLDU(p, c, i) tfft_bld<0>((p), (unsigned)(i) * TFFT_ESZ(p), (unsigned)(c) * TFFT_ESZ(p))
#define LLD(i) (lds[(i)])
#define LST(i, v) (lds[(i)] = (v))
// compact checksum table: one 32-bit word holds two half-precision values
typedef _Float16 tfft_h2v __attribute__((ext_vector_type(2)));
#define CKW(p, c, i) (((const unsigned*)(p))[(c) + (i)])
__device__ __forceinline__ float tfft_ckh(unsigned w, int hi) {
    const tfft_h2v h = __builtin_bit_cast(tfft_h2v, w);
    return hi ? (float)h.y : (float)h.x;
}
#define CKH(w, hi) tfft_ckh((w), (hi))
#define CKF(w) __uint_as_float(w)
// Partial checksums handed from block to block: device-scope relaxed atomic accesses, which go
// past the XCD's own L2 to memory.  With them the hand-off needs no device-scope fence -- on this
// part a release writes the whole L2 back and an acquire invalidates it, and thousands of blocks
// doing that per launch made the launch four to six times slower.
// What orders the hand-off instead: every wave waits until its own stores have been acknowledged
// (TFFT_WAIT_VMEM: vector-memory counter zero, the other counters left alone) before the block
// barrier that precedes the ticket; an acknowledged agent-scope store is in memory.
#define TFFT_WAIT_VMEM() __builtin_amdgcn_s_waitcnt(0x0F70)     // gfx9 encoding: vmcnt = 0, expcnt = 7, lgkmcnt = 15 (no wait)
template <typename T> __device__ __forceinline__ void tfft_ps_store(T* p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
template <typename T> __device__ __forceinline__ T tfft_ps_load(const T* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// a thread's compact-table words parked in LDS behind the exchange buffer, four to an access
typedef uint4 tfft_cw4;
#define CWL_ST(off, i, v) (((tfft_cw4*)(lds_raw + (off)))[(i)] = (v))
#define CWL_LD(off, i) (((const tfft_cw4*)(lds_raw + (off)))[(i)])
// makes a per-lane value opaque to the optimiser (no code is emitted): used to keep
// tile-independent table reads inside the tile loop instead of hoisted into registers
#define OPAQUE(v) asm volatile("" : "+v"(v))
// a block-uniform value back into a scalar register (the integer divisions of the tile-group
// formula run on the vector unit and leave their results, and everything derived, in VGPRs)
__device__ __forceinline__ unsigned tfft_uni(unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ int tfft_uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ long long tfft_uni(long long v) {
    const unsigned lo = tfft_uni((unsigned)v), hi = tfft_uni((unsigned)((unsigned long long)v >> 32));
    return (long long)(((unsigned long long)hi << 32) | lo);
}
// instruction-scheduling fence: nothing may be moved across it
#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
// thread-level verification: one word per wavefront at byte `off` of the block's LDS says whether any of
// its lanes objected to the tile (a wave vote, then lane 0 writes); the block reads the words behind a barrier
#define TL_VOTE(off, bad) { const int wany_ = __any((bad) ? 1 : 0); if ((tx & 63u) == 0u) ((unsigned*)(lds_raw + (off)))[tx >> 6] = wany_ ? 1u : 0u; }

// ---- teams of a fused pair (tfft_fuse_args) ----
// A team is `team` blocks that arrived one after the other on one XCD; its first member is its leader.
// Every wait is thread 0's, on an agent-scope counter, and bounded: after limit_ms the waiting block sets
// the give-up word, which every other wait reads on each eighth poll, and all blocks leave.  What orders
// the slot's data: a block waits until its own stores are acknowledged (they are in the L2 then) before it
// counts itself in, and the readers use agent-scope loads.
// The leader names pieces two rounds ahead (word r % 2 of the pair holds round r's name, tagged r + 1):
// when a member leaves the meeting of round r the name of round r + 1 has long been there, so it can
// start fetching that piece while it still works on this one.
struct tfft_team { unsigned slot, member, xcc, index; unsigned* a; unsigned* b; unsigned long long* cur; long long t_limit; };

__device__ __forceinline__ bool tfft_team_give_up(const tfft_fuse_args& f, long long t_limit, unsigned polls) {
    if ((polls & 7u) != 7u) return false;
    if (tfft_ps_load(&f.ctl[0])) return true;
    if ((long long)wall_clock64() > t_limit) {
        atomicExch(&f.ctl[0], 1u);
        if (f.err_host) __hip_atomic_store(f.err_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        return true;
    }
    return false;
}
// thread 0: until *p >= k
__device__ __forceinline__ bool tfft_team_wait(unsigned* p, unsigned k, const tfft_fuse_args& f, long long t_limit) {
    for (unsigned polls = 0;; ++polls) {
        if (tfft_ps_load(p) >= k) return true;
        if (tfft_team_give_up(f, t_limit, polls)) return false;
        __builtin_amdgcn_s_sleep(2);
    }
}
// thread 0: the name of `round` (piece + 1, 0: none), 0 also when the wait gave up
__device__ __forceinline__ unsigned tfft_team_name(const tfft_fuse_args& f, const tfft_team& tm, unsigned round) {
    for (unsigned polls = 0;; ++polls) {
        const unsigned long long v = tfft_ps_load(tm.cur + 16 * (round & 1u));
        if ((unsigned)(v >> 32) == round + 1u) return (unsigned)v;
        if (tfft_team_give_up(f, tm.t_limit, polls)) return 0u;
        __builtin_amdgcn_s_sleep(2);
    }
}
// thread 0 of the leader: take a piece off the queue and name it for `round`
__device__ __forceinline__ void tfft_team_claim(const tfft_fuse_args& f, const tfft_team& tm, unsigned round, bool take) {
    unsigned p1 = 0;
    if (take) { const unsigned p = atomicAdd(&f.ctl[32], 1u); p1 = (long long)p < f.npieces ? p + 1u : 0u; }
    tfft_ps_store(tm.cur + 16 * (round & 1u), ((unsigned long long)(round + 1u) << 32) | p1);
}
// false: this block has no team (its XCD's teams were full when it arrived)
__device__ __forceinline__ bool tfft_team_join(const tfft_fuse_args& f, tfft_team& tm, unsigned* w) {
    const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7u;      // XCC_ID[3:0] of the hardware register
    if (threadIdx.x == 0) w[0] = atomicAdd(&f.ctl[96 + 32 * xcc], 1u);
    __syncthreads();
    const unsigned idx = tfft_uni(w[0]);
    __syncthreads();
    const unsigned team = idx / (unsigned)f.team;
    tm.xcc = xcc; tm.index = team; tm.member = idx % (unsigned)f.team;
    tm.slot = xcc * (unsigned)f.teams_per_xcd + team;
    unsigned* base = f.ctl + 352 + 128 * (size_t)tm.slot;
    tm.a = base; tm.b = base + 32; tm.cur = (unsigned long long*)(base + 64);
    tm.t_limit = (long long)wall_clock64() + (long long)f.limit_ms * 100000ll;   // 100 MHz counter
    if (f.limit_ms < 0) {
        // no time at all (the host's way of exercising the give-up path): say so and take no part
        if (threadIdx.x == 0) {
            atomicExch(&f.ctl[0], 1u);
            if (f.err_host) __hip_atomic_store(f.err_host, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        return false;
    }
    return team < (unsigned)f.teams_per_xcd;
}
// The team's first piece, or -1 when there is none.  The leader waits until the team is complete -- or the queue
// empty: then a team that forms late has nothing to do -- and names rounds 0 and 1.
__device__ __forceinline__ long long tfft_team_first(const tfft_fuse_args& f, const tfft_team& tm, unsigned* w) {
    if (threadIdx.x == 0) {
        bool ok = true;
        if (tm.member == 0) {
            bool complete = false;
            for (unsigned polls = 0;; ++polls) {
                if (tfft_ps_load(&f.ctl[96 + 32 * tm.xcc]) >= (tm.index + 1u) * (unsigned)f.team) { complete = true; break; }
                if ((long long)tfft_ps_load(&f.ctl[32]) >= f.npieces) break;
                if (tfft_team_give_up(f, tm.t_limit, polls)) { ok = false; break; }
                __builtin_amdgcn_s_sleep(2);
            }
            if (ok) { tfft_team_claim(f, tm, 0u, complete); tfft_team_claim(f, tm, 1u, complete); }
        }
        w[1] = ok ? tfft_team_name(f, tm, 0u) : 0u;
    }
    __syncthreads();
    const unsigned name = tfft_uni(w[1]);
    __syncthreads();
    return (long long)name - 1;
}
// Between the two launches of a piece: every member's tiles are in the slot.  `next` is the piece of the next
// round (-1: none).  The leader, once every member has arrived (all have read this round's name by then, whose
// word is the one written now), names the round after the next.
__device__ __forceinline__ bool tfft_team_meet(const tfft_fuse_args& f, const tfft_team& tm, unsigned round, unsigned* w, long long& next) {
    TFFT_WAIT_VMEM();
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicAdd(tm.a, 1u);
        const bool ok = tfft_team_wait(tm.a, (unsigned)f.team * (round + 1u), f, tm.t_limit);
        unsigned name = 0;
        if (ok) {
            name = tfft_team_name(f, tm, round + 1u);
            if (tm.member == 0) tfft_team_claim(f, tm, round + 2u, name != 0u);
        }
        w[1] = name;
        w[2] = ok ? 1u : 0u;
    }
    __syncthreads();
    const unsigned ok = tfft_uni(w[2]), name = tfft_uni(w[1]);
    __syncthreads();
    next = (long long)name - 1;
    return ok != 0u;
}
// before a member's first store of `round` (> 0) into the slot: every member has finished reading what the
// round before left there
__device__ __forceinline__ bool tfft_team_free(const tfft_fuse_args& f, const tfft_team& tm, unsigned round, unsigned* w) {
    if (threadIdx.x == 0) w[2] = tfft_team_wait(tm.b, (unsigned)f.team * round, f, tm.t_limit) ? 1u : 0u;
    __syncthreads();
    const unsigned ok = tfft_uni(w[2]);
    __syncthreads();
    return ok != 0u;
}
// after the row launch of a piece: this member no longer reads the slot (what it loaded from the slot has been
// computed with, so those loads have returned; its stores to memory are nobody's business here)
__device__ __forceinline__ void tfft_team_release(const tfft_team& tm) {
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(tm.b, 1u);
}
// every block of the grid, last thing: the last one to leave clears the control block for the next launch
__device__ __forceinline__ void tfft_team_leave(const tfft_fuse_args& f, unsigned* w) {
    __syncthreads();
    if (threadIdx.x == 0) w[3] = atomicAdd(&f.ctl[64], 1u) == gridDim.x - 1u ? 1u : 0u;
    __syncthreads();
    if (w[3]) {
        const unsigned words = 352u + 128u * 8u * (unsigned)f.teams_per_xcd;
        for (unsigned i = threadIdx.x; i < words; i += blockDim.x) tfft_ps_store(&f.ctl[i], 0u);
    }
}
#else
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
struct float2 { float x, y; };
struct double2 { double x, y; };
#define TFFT_DEV static inline
struct tfft_sim_bounds_t { long long in_elems, out_elems, tw_elems, lds_elems, twhi_elems, twlo_elems; };
extern tfft_sim_bounds_t tfft_sim_bounds;
extern long long tfft_sim_errors;
#define TFFT_CHK(i, n, what)                                                              \
    (((long long)(i) < 0 || (long long)(i) >= (long long)(n))                             \
         ? (tfft_sim_errors++ == 0 ? fprintf(stderr, "tfft sim: %s index %lld out of [0,%lld) at %s:%d\n", \
                                             what, (long long)(i), (long long)(n), __FILE__, __LINE__) : 0, 0LL) \
         : (long long)(i))
#define GLDU(p, ub, uo, off) ((p)[TFFT_CHK((long long)(ub) + (long long)(uo) + (long long)(off), p##_limit, #p)])
#define GSTU(p, ub, uo, off, v) ((p)[TFFT_CHK((long long)(ub) + (long long)(uo) + (long long)(off), p##_limit, #p)] = (v))
#define GLDG(p, ub, uo, off) GLDU(p, ub, uo, off)
#define GSTG(p, ub, uo, off, v) GSTU(p, ub, uo, off, v)
#define GLDUN(p, ub, uo, off) GLDU(p, ub, uo, off)
#define GLDUS(p, ub, uo, off) GLDU(p, ub, uo, off)
#define GSTUN(p, ub, uo, off, v) GSTU(p, ub, uo, off, v)
#define GLDGN(p, ub, uo, off) GLDU(p, ub, uo, off)
#define GSTGN(p, ub, uo, off, v) GSTU(p, ub, uo, off, v)
#define TFFT_WAVE_PRIO(n) ((void)0)
#define GLDU2(p, ub, uo, off, A, B) { (A) = GLDU(p, ub, uo, off); (B) = GLDU(p, ub, (uo) + 1, off); }
#define GSTU2(p, ub, uo, off, A, B) { GSTU(p, ub, uo, off, A); GSTU(p, ub, (uo) + 1, off, B); }
#define GLDUN2(p, ub, uo, off, A, B) GLDU2(p, ub, uo, off, A, B)
#define GSTUN2(p, ub, uo, off, A, B) GSTU2(p, ub, uo, off, A, B)
#define TWLG(p, i) TWLD(p, i)
#define TWLGU(p, c, i) TWLDU(p, c, i)
#define TWLD(p, i) ((p)[TFFT_CHK((i), p##_limit, #p)])
#define TWLDU(p, c, i) ((p)[TFFT_CHK((long long)(c) + (long long)(i), p##_limit, #p)])
#define OPAQUE(v)
template <typename T> static inline T tfft_uni(T v) { return v; }
#define SCHED_FENCE()
#define TL_VOTE(off, bad) ((void)0)
// compact checksum table (ck_limit counts complex elements of the buffer the launcher passed)
#define CKW(p, c, i) (((const unsigned*)(p))[TFFT_CHK((long long)(c) + (long long)(i), (long long)(sizeof(*(p)) / 4) * ck_limit, "compact checksum table")])
static inline float tfft_ckh(unsigned w, int hi) {
    const unsigned h = hi ? (w >> 16) : (w & 0xffffu);
    const unsigned sgn = (h >> 15) & 1u, ex = (h >> 10) & 31u, man = h & 1023u;
    float v;
    if (ex == 0) v = std::ldexp((float)man, -24);
    else if (ex == 31) v = man ? NAN : INFINITY;
    else v = std::ldexp((float)(man | 1024u), (int)ex - 25);
    return sgn ? -v : v;
}
#define CKH(w, hi) tfft_ckh((w), (hi))
static inline float tfft_ckf(unsigned w) { float f; memcpy(&f, &w, sizeof f); return f; }
#define CKF(w) tfft_ckf(w)
struct tfft_cw4 { unsigned x, y, z, w; };
template <typename T> static inline void tfft_ps_store(T* p, T v) { *p = v; }
template <typename T> static inline T tfft_ps_load(const T* p) { return *p; }
#define CWL_ST(off, i, v) (cwl[TFFT_CHK((i), cwl_limit, "parked checksum words")] = (v))
#define CWL_LD(off, i) (cwl[TFFT_CHK((i), cwl_limit, "parked checksum words")])
#define LLD(i) (lds[TFFT_CHK((i), lds_limit, "lds")])
#define LST(i, v) (lds[TFFT_CHK((i), lds_limit, "lds")] = (v))
// cross-lane fetch in the lock-step flavour: the partner's registers as snapshotted
// before the stage
#define XLANE(i, MASK, dst) { dst = ts[tx ^ (MASK)].sh[i]; }
#define SNAP() { for (unsigned z_ = 0; z_ < sizeof(ts[tx].sh) / sizeof(ts[tx].sh[0]); ++z_) ts[tx].sh[z_] = r[z_]; }
#endif

TFFT_DEV float2 cadd(float2 a, float2 b) { float2 c; c.x = a.x + b.x; c.y = a.y + b.y; return c; }
TFFT_DEV float2 csub(float2 a, float2 b) { float2 c; c.x = a.x - b.x; c.y = a.y - b.y; return c; }
TFFT_DEV float2 cmul(float2 a, float2 b) { float2 c; c.x = a.x * b.x - a.y * b.y; c.y = a.y * b.x + a.x * b.y; return c; }
TFFT_DEV float2 cmulc(float2 a, float cr, float ci) { float2 c; c.x = a.x * cr - a.y * ci; c.y = a.y * cr + a.x * ci; return c; }
TFFT_DEV float2 cmul_mi(float2 a) { float2 c; c.x = a.y; c.y = -a.x; return c; }   // * (-i)
TFFT_DEV float2 cmul_pi(float2 a) { float2 c; c.x = -a.y; c.y = a.x; return c; }   // * (+i)
TFFT_DEV float2 cneg(float2 a) { float2 c; c.x = -a.x; c.y = -a.y; return c; }
TFFT_DEV float2 czero(float2) { float2 c; c.x = 0.f; c.y = 0.f; return c; }
TFFT_DEV float2 cswap(float2 a) { float2 c; c.x = a.y; c.y = a.x; return c; }       // (re, im) -> (im, re)

TFFT_DEV double2 cadd(double2 a, double2 b) { double2 c; c.x = a.x + b.x; c.y = a.y + b.y; return c; }
TFFT_DEV double2 csub(double2 a, double2 b) { double2 c; c.x = a.x - b.x; c.y = a.y - b.y; return c; }
TFFT_DEV double2 cmul(double2 a, double2 b) { double2 c; c.x = a.x * b.x - a.y * b.y; c.y = a.y * b.x + a.x * b.y; return c; }
TFFT_DEV double2 cmulc(double2 a, double cr, double ci) { double2 c; c.x = a.x * cr - a.y * ci; c.y = a.y * cr + a.x * ci; return c; }
TFFT_DEV double2 cmul_mi(double2 a) { double2 c; c.x = a.y; c.y = -a.x; return c; }
TFFT_DEV double2 cmul_pi(double2 a) { double2 c; c.x = -a.y; c.y = a.x; return c; }
TFFT_DEV double2 cneg(double2 a) { double2 c; c.x = -a.x; c.y = -a.y; return c; }
TFFT_DEV double2 czero(double2) { double2 c; c.x = 0.0; c.y = 0.0; return c; }
TFFT_DEV double2 cswap(double2 a) { double2 c; c.x = a.y; c.y = a.x; return c; }

#ifndef TFFT_SIM
// Cross-lane fetch of the value held by lane (lane ^ MASK): DPP quad permutes for
// MASK 1 and 2, the ds_swizzle crossbar (bit mode, no LDS memory touched) for 4.
template <int MASK> TFFT_DEV int xl_i32(int v) {
    static_assert(MASK == 1 || MASK == 2 || MASK == 4, "cross-lane distance");
    if (MASK == 1) return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);        // quad_perm [1,0,3,2]
    if (MASK == 2) return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);        // quad_perm [2,3,0,1]
    return __builtin_amdgcn_ds_swizzle(v, 0x101F);                                   // and 0x1f, or 0, xor 4
}
template <int MASK> TFFT_DEV float xl_r(float v) { return __int_as_float(xl_i32<MASK>(__float_as_int(v))); }
template <int MASK> TFFT_DEV double xl_r(double v) {
    const long long b = __double_as_longlong(v);
    const int lo = xl_i32<MASK>((int)(b & 0xffffffffll)), hi = xl_i32<MASK>((int)(b >> 32));
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
#define XLANE(i, MASK, dst) { dst.x = xl_r<MASK>(r[i].x); dst.y = xl_r<MASK>(r[i].y); }
#define SNAP()

// Sum over the 64 lanes of a wavefront; every lane receives the total: six butterfly steps
// of __shfl_xor (a ds_bpermute each; no LDS memory is touched).
TFFT_DEV float wave_sum(float v) {
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    v += __shfl_xor(v, 8, 64);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
TFFT_DEV double wave_sum(double v) {
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    v += __shfl_xor(v, 8, 64);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
#endif
