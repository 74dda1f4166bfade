// Streaming kernels of known traffic, for the measurements the FFT kernels are judged against:
// what a plain copy reaches on this device with 8-byte and with 16-byte lanes (the reason the fp32
// kernels move one float2 per lane), and what read-only and write-only sweeps reach.  Also the
// kernels of known size that rocprofv3's FETCH_SIZE / WRITE_SIZE counters can be scaled with.
// Measurement only: nothing here is used by turbofft_exec.  No counterpart in the reference, which
// quotes its bandwidth against the data sheet (readme.md).
#include <hip/hip_runtime.h>
#include <cstring>

#include "../../include/turbofft.h"

void tfft_set_error(const char* fmt, ...);   // turbofft_host.cpp

namespace {

typedef float v2 __attribute__((ext_vector_type(2)));
typedef float v4 __attribute__((ext_vector_type(4)));

// AUX: cache-policy immediate of the buffer instructions (0 default, 2 non-temporal), as in the FFT kernels
typedef unsigned u2 __attribute__((ext_vector_type(2)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t mb_rsrc(const void* p) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, -1, 0x00020000); }
template <int AUX> __device__ __forceinline__ v2 mb_ld(const v2* p, unsigned off) { const u2 t = __builtin_amdgcn_raw_buffer_load_b64(mb_rsrc(p), off, 0, AUX); v2 r; r.x = __uint_as_float(t.x); r.y = __uint_as_float(t.y); return r; }
template <int AUX> __device__ __forceinline__ v4 mb_ld(const v4* p, unsigned off) { const u4 t = __builtin_amdgcn_raw_buffer_load_b128(mb_rsrc(p), off, 0, AUX); v4 r; r.x = __uint_as_float(t.x); r.y = __uint_as_float(t.y); r.z = __uint_as_float(t.z); r.w = __uint_as_float(t.w); return r; }
template <int AUX> __device__ __forceinline__ void mb_st(v2* p, unsigned off, v2 v) { u2 t; t.x = __float_as_uint(v.x); t.y = __float_as_uint(v.y); __builtin_amdgcn_raw_buffer_store_b64(t, mb_rsrc(p), off, 0, AUX); }
template <int AUX> __device__ __forceinline__ void mb_st(v4* p, unsigned off, v4 v) { u4 t; t.x = __float_as_uint(v.x); t.y = __float_as_uint(v.y); t.z = __float_as_uint(v.z); t.w = __float_as_uint(v.w); __builtin_amdgcn_raw_buffer_store_b128(t, mb_rsrc(p), off, 0, AUX); }

// tile of this block: with `xcd_chunk` > 0 the blocks are renumbered as in the FFT kernels, so that
// each of the 8 XCDs (hardware deals block ids round-robin) works on runs of consecutive tiles
__device__ __forceinline__ size_t mb_tile(int xcd_chunk) {
    unsigned bx = blockIdx.x;
    if (xcd_chunk > 0) {
        const unsigned xc = (unsigned)xcd_chunk, span = 8u * xc, full = (gridDim.x / span) * span;
        if (bx < full) { const unsigned q = bx >> 3, xcd = bx & 7u; bx = (q / xc) * span + xcd * xc + q % xc; }
    }
    return (size_t)bx;
}

// a block of 256 threads moves one contiguous tile of 256*U vectors: every load is issued before
// the first store, as in the FFT kernels; the lanes of a wavefront touch consecutive vectors.
// Dynamic LDS that the kernels do not touch limits the blocks resident per CU, as the exchange
// buffer of an FFT kernel does.
template <class V, int U, int AUX>
__global__ __launch_bounds__(256) void tfft_mb_copy(const V* __restrict__ in, V* __restrict__ out, int xcd_chunk) {
    const size_t base = mb_tile(xcd_chunk) * 256 * U;
    const unsigned lane = threadIdx.x * (unsigned)sizeof(V);
    V r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = mb_ld<AUX>(in + base, lane + (unsigned)(e * 256 * sizeof(V)));
#pragma unroll
    for (int e = 0; e < U; ++e) mb_st<AUX>(out + base, lane + (unsigned)(e * 256 * sizeof(V)), r[e]);
}

template <class V, int U, int AUX>
__global__ __launch_bounds__(256) void tfft_mb_read(const V* __restrict__ in, float* __restrict__ sink, int xcd_chunk) {
    const size_t base = mb_tile(xcd_chunk) * 256 * U;
    const unsigned lane = threadIdx.x * (unsigned)sizeof(V);
    V r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = mb_ld<AUX>(in + base, lane + (unsigned)(e * 256 * sizeof(V)));
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < U; ++e) acc += r[e].x;
    if (acc == 123456.789f) sink[0] = acc;       // keeps the loads alive, never true for the test data
}

template <class V, int U, int AUX>
__global__ __launch_bounds__(256) void tfft_mb_write(V* __restrict__ out, int xcd_chunk) {
    const size_t base = mb_tile(xcd_chunk) * 256 * U;
    const unsigned lane = threadIdx.x * (unsigned)sizeof(V);
    V v;
    v.x = (float)threadIdx.x;
    v.y = 1.f;
#pragma unroll
    for (int e = 0; e < U; ++e) mb_st<AUX>(out + base, lane + (unsigned)(e * 256 * sizeof(V)), v);
}

// Strided tiles: 64 KiB made of rows of RUN bytes, row r of a tile at tile base + r << log_stride; tiles side by side
// along a row first.  The access pattern of the column kernels (runs of BS elements at the stride of the digit) and
// of the transposed store of the last launch.  Non-temporal, XCD-aware tile order.
template <class V, int RUN, bool WRITE>
__global__ __launch_bounds__(256) void tfft_mb_strided(const V* __restrict__ in, V* __restrict__ out, float* __restrict__ sink, int xcd_chunk, unsigned log_stride) {
    constexpr unsigned W = sizeof(V), TILE = 65536, LPR = RUN / W, U = TILE / (256 * W);
    const size_t t = mb_tile(xcd_chunk);
    const unsigned tiles_per_row = (1u << log_stride) / RUN, rows = TILE / RUN;
    const size_t base = (t / tiles_per_row) * rows * ((size_t)1 << log_stride) + (t % tiles_per_row) * RUN;       // bytes
    const unsigned lane = (threadIdx.x % LPR) * W + ((threadIdx.x / LPR) << log_stride);
    const unsigned step = (256 / LPR) << log_stride;
    if (WRITE) {
        V v;
        v.x = (float)threadIdx.x;
        v.y = 1.f;
        if constexpr (sizeof(V) == 16) { v.z = (float)threadIdx.x; v.w = 1.f; }
#pragma unroll
        for (unsigned e = 0; e < U; ++e) mb_st<2>((V*)((char*)out + base), lane + e * step, v);
    } else {
        float acc = 0.f;
#pragma unroll
        for (unsigned e = 0; e < U; ++e) acc += mb_ld<2>((const V*)((const char*)in + base), lane + e * step).x;
        if (acc == 123456.789f) sink[0] = acc;
    }
}

// ---- two passes through a ring that stays in the XCD's L2 (the question a fused pass pair of a
// two-launch plan would have to answer first) ----
// Synthetic: in -> ring -> out as ONE persistent kernel (`lag`: how many groups the second pass runs behind the first in ticket order).  The data is cut into "transforms" of 512 KiB;
// each of the 8 XCDs (a block reads its XCD from the hardware register) owns every eighth transform and a
// ring of R slots of G transforms that is reused for every group, so the intermediate is only ever written
// to addresses that are still in that XCD's L2.  Items are handed out per XCD in ticket order
//   P1(g0) | P1(g1) P2(g0) | P1(g2) P2(g1) | ...          (lag 1; with lag K: P1(g0) ... P1(gK-1) | P1(gK) P2(g0) | ...)
// (P1: 32 KiB of a transform in -> slot, 16 per transform; P2: 64 KiB slot -> out, 8 per transform).  A P2
// item needs every P1 item of its group (as a row pass needs every column tile), a P1 item of group g
// needs slot g % R drained by P2(g - R).  Every wait is for items with lower tickets, which running blocks
// hold, so the order cannot deadlock whatever the grid; each wait is also bounded by a wall-clock limit after
// which the block raises an error flag and every block leaves at its next ticket.
constexpr long long kFusedTransform = 512 << 10;
constexpr int kFusedP1 = 32 << 10, kFusedP2 = 64 << 10, kFusedMaxGroups = 2048;
struct FusedQueue { unsigned next; unsigned pad0[31]; unsigned done1[kFusedMaxGroups]; unsigned done2[kFusedMaxGroups]; };
struct FusedCtl { unsigned err, pad0[31]; unsigned waits, spins, pad1[30]; unsigned xcc_blocks[32]; FusedQueue q[8]; };   // the flag every block reads has a line of its own

__global__ void tfft_mb_fused_clear(FusedCtl* c) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < sizeof(FusedCtl) / 4) ((unsigned*)c)[i] = 0;
}

template <int U, int LAUX, int SAUX>
__device__ __forceinline__ void fused_copy_item(const char* src, char* dst) {
    u4 r[U];
#pragma unroll
    for (int e = 0; e < U; ++e) r[e] = __builtin_amdgcn_raw_buffer_load_b128(mb_rsrc(src), (threadIdx.x + e * 256) * 16u, 0, LAUX);
#pragma unroll
    for (int e = 0; e < U; ++e) __builtin_amdgcn_raw_buffer_store_b128(r[e], mb_rsrc(dst), (threadIdx.x + e * 256) * 16u, 0, SAUX);
}

// thread 0 waits until *p >= k; false after the time limit or when another block gave up.  The statistics stay in the
// caller's registers until the block ends and the give-up flag is read on every eighth poll: counters that every
// waiting block updates in one line serialise the waits of the whole grid.
__device__ __forceinline__ bool fused_wait(unsigned* p, unsigned k, FusedCtl* c, long long t_limit, unsigned& waits, unsigned& spins_total) {
    unsigned spins = 0;
    for (;;) {
        if (__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= k) {
            if (spins) { ++waits; spins_total += spins; }
            return true;
        }
        if ((spins & 7u) == 7u) {
            if (__hip_atomic_load(&c->err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return false;
            if ((long long)wall_clock64() > t_limit) { atomicExch(&c->err, 1u); return false; }
        }
        __builtin_amdgcn_s_sleep(2);
        ++spins;
    }
}

__global__ __launch_bounds__(256) void tfft_mb_fused(const char* __restrict__ in, char* __restrict__ scratch, char* __restrict__ out, FusedCtl* c,
                                                    int ntrans_per_xcd, int G, int R, int limit_ms, int lag) {
    __shared__ unsigned s_t;
    __shared__ int s_ok;
    const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7u;     // XCC_ID[3:0] of the hardware register
    FusedQueue* q = &c->q[xcc];
    const long long t_limit = (long long)wall_clock64() + (long long)limit_ms * 100000ll;   // 100 MHz counter
    if (threadIdx.x == 0) atomicAdd(&c->xcc_blocks[xcc], 1u);
    const int ngroups = ntrans_per_xcd / G;
    const unsigned n1 = (unsigned)(kFusedTransform / kFusedP1 * G), n2 = (unsigned)(kFusedTransform / kFusedP2 * G);
    const unsigned total = (unsigned)ngroups * (n1 + n2);
    char* ring = scratch + (size_t)xcc * R * G * kFusedTransform;
    unsigned waits = 0, spins = 0;
    for (;;) {
        if (threadIdx.x == 0) {
            unsigned t = atomicAdd(&q->next, 1u);
            if (__hip_atomic_load(&c->err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) t = 0xffffffffu;
            s_t = t;
        }
        __syncthreads();
        const unsigned t = (unsigned)__builtin_amdgcn_readfirstlane((int)s_t);
        __syncthreads();
        if (t >= total) break;
        // ticket order with the second pass `lag` groups behind the first: segment s holds P1(s) (s < ngroups) then P2(s - lag) (s >= lag)
        bool is1; unsigned g, i;
        const unsigned K = (unsigned)lag, head = K * n1, mid = ((unsigned)ngroups - K) * (n1 + n2);
        if (t < head) { is1 = true; g = t / n1; i = t % n1; }
        else if (t - head < mid) {
            const unsigned u = t - head, seg = K + u / (n1 + n2), r = u % (n1 + n2);
            if (r < n1) { is1 = true; g = seg; i = r; } else { is1 = false; g = seg - K; i = r - n1; }
        } else { const unsigned u = t - head - mid; is1 = false; g = (unsigned)ngroups - K + u / n2; i = u % n2; }
        char* slot = ring + (size_t)(g % R) * G * kFusedTransform;
        if (is1) {
            if (g >= (unsigned)R) {
                if (threadIdx.x == 0) s_ok = fused_wait(&q->done2[g - R], n2, c, t_limit, waits, spins) ? 1 : 0;
                __syncthreads();
                const int ok = s_ok;
                __syncthreads();
                if (!ok) break;
            }
            const unsigned per = (unsigned)(kFusedTransform / kFusedP1), k = i / per, j = i % per;
            const size_t T = (size_t)(g * G + k) * 8 + xcc;
            fused_copy_item<kFusedP1 / 4096, 2, 0>(in + T * kFusedTransform + (size_t)j * kFusedP1, slot + (size_t)k * kFusedTransform + (size_t)j * kFusedP1);
            __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): this wave's stores are acknowledged by the L2
            __syncthreads();
            if (threadIdx.x == 0) atomicAdd(&q->done1[g], 1u);
        } else {
            if (threadIdx.x == 0) s_ok = fused_wait(&q->done1[g], n1, c, t_limit, waits, spins) ? 1 : 0;
            __syncthreads();
            const int ok = s_ok;
            __syncthreads();
            if (!ok) break;
            const unsigned per = (unsigned)(kFusedTransform / kFusedP2), k = i / per, j = i % per;
            const size_t T = (size_t)(g * G + k) * 8 + xcc;
            // agent-scope loads of the ring: never served from this CU's L1, which may hold the slot's previous contents
            constexpr int U2 = kFusedP2 / 4096;
            const char* from = slot + (size_t)k * kFusedTransform + (size_t)j * kFusedP2;
            char* to = out + T * kFusedTransform + (size_t)j * kFusedP2;
            u4 r[U2];
#pragma unroll
            for (int e = 0; e < U2; ++e) r[e] = __builtin_amdgcn_raw_buffer_load_b128(mb_rsrc(from), (threadIdx.x + e * 256) * 16u, 0, 16);
            __builtin_amdgcn_s_waitcnt(0x0F70);       // the slot's loads have returned: it is handed back before the stores to
            __syncthreads();                          // memory are issued, whose acknowledgement nobody waits for here
            if (threadIdx.x == 0) atomicAdd(&q->done2[g], 1u);
#pragma unroll
            for (int e = 0; e < U2; ++e) __builtin_amdgcn_raw_buffer_store_b128(r[e], mb_rsrc(to), (threadIdx.x + e * 256) * 16u, 0, 2);
        }
    }
    if (threadIdx.x == 0 && waits) { atomicAdd(&c->waits, waits); atomicAdd(&c->spins, spins); }
}

// ---- the same question with teams: T blocks of one XCD share one 512 KiB piece at a time ----
// Every team owns ONE slot, reused for every piece it handles, so an XCD's slots (teams x 512 KiB) are all the
// intermediate there is.  Per piece: every member copies its 1/T of the piece in -> slot, the team meets at a
// barrier (a counter per team, agent-scope atomics, bounded polling), every member copies another 1/T of the slot
// (2 KiB from each member's part, as a row tile takes a strip of every column tile) slot -> out, and the team meets
// again before the slot is overwritten -- that second wait is taken after the next piece's loads have been issued.
// Needs every block of the grid resident at once (the grid is sized from the occupancy query) and the blocks dealt
// evenly to the XCDs; a member that never shows up ends in the time limit and the error flag, not in a hang.
struct TeamBar { unsigned a, pad0[31]; unsigned b, pad1[31]; };      // one line for each counter
struct TeamCtl { unsigned err, pad0[31]; unsigned waits, polls, pad1[30]; unsigned arrive[32]; unsigned long long ticks[16]; TeamBar bar[8][64]; };

__global__ void tfft_mb_team_clear(TeamCtl* c) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < sizeof(TeamCtl) / 4) ((unsigned*)c)[i] = 0;
}

// One thread's wait for a counter of its team.  The flag that ends every wait after a time-out sits in a line of its
// own and is read on every eighth poll only, and the statistics stay in the caller's registers until the block ends:
// a line that every waiting block reads and updates would serialise the waits of the whole grid.
__device__ __forceinline__ bool team_wait(unsigned* p, unsigned k, TeamCtl* c, long long t_limit, unsigned& waits, unsigned& polls_total) {
    unsigned polls = 0;
    for (;;) {
        if (__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= k) {
            if (polls) { ++waits; polls_total += polls; }
            return true;
        }
        if ((polls & 7u) == 7u) {
            if (__hip_atomic_load(&c->err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) return false;
            if ((long long)wall_clock64() > t_limit) { atomicExch(&c->err, 1u); return false; }
        }
        __builtin_amdgcn_s_sleep(2);
        ++polls;
    }
}

// T: blocks per team; PIECE: bytes a team moves per round (one slot); every member moves PIECE / T per pass
// POL: cache policy of the accesses to memory, loads of `in` in bits 0-1 and stores to `out` in bits 2-3:
// 0 nt, 1 nt + sc0, 2 nt + sc1, 3 nt + sc0 + sc1.  The slot is written with the default policy; how it is read is bits 4-5:
// 0 sc1 loads, 1 sc0 loads, 2 nt loads, 3 default loads behind an invalidation of the CU's vector L1 (buffer_inv sc1)
template <int T, int PIECE, int POL = 0>
__global__ __launch_bounds__(256) void tfft_mb_team(const char* __restrict__ in, char* __restrict__ scratch, char* __restrict__ out, TeamCtl* c,
                                                   int ntrans, int limit_ms) {
    constexpr int SHARE = PIECE / T, U = SHARE / 4096;
    constexpr int kAux[4] = {2, 3, 18, 19};
    constexpr int LAUX = kAux[POL & 3], SAUX = kAux[(POL >> 2) & 3];
    constexpr int kSlotAux[4] = {16, 1, 2, 0};
    constexpr int RAUX = kSlotAux[(POL >> 4) & 3];
    static_assert(U >= 1 && U <= 32 && SHARE / T >= 16, "a share fits the registers of a block");      // bytes per member and pass; 16-byte accesses per thread
    __shared__ unsigned s_idx;
    __shared__ int s_ok;
    const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7u;
    const long long t_limit = (long long)wall_clock64() + (long long)limit_ms * 100000ll;
    if (threadIdx.x == 0) s_idx = atomicAdd(&c->arrive[xcc], 1u);
    __syncthreads();
    const unsigned idx = (unsigned)__builtin_amdgcn_readfirstlane((int)s_idx);
    const unsigned nteams = (gridDim.x / 8u) / (unsigned)T;
    const unsigned team = idx / (unsigned)T, member = idx % (unsigned)T;
    if (team >= nteams) return;                                   // blocks beyond whole teams have nothing to do
    TeamBar* bar = &c->bar[xcc][team];
    char* slot = scratch + ((size_t)xcc * nteams + team) * (size_t)PIECE;
    u4 r[U];
    unsigned round = 0, waits = 0, polls = 0;
    // time per part of a round as thread 0 sees it (100 MHz ticks): [0] until the piece's loads have returned, [1] the wait for
    // the slot, [2] slot stores acknowledged, [3] the team barrier, [4] the slot's loads have returned, [5] the rest
    long long tk[6] = {0, 0, 0, 0, 0, 0}, tl = (long long)wall_clock64();
#define MB_TICK(k) { const long long now_ = (long long)wall_clock64(); tk[k] += now_ - tl; tl = now_; }
    for (size_t t = xcc + 8 * (size_t)team; t < (size_t)ntrans; t += 8 * (size_t)nteams, ++round) {
        // pass 1: this member's contiguous part of the piece
        const char* src = in + t * (size_t)PIECE + (size_t)member * SHARE;
#pragma unroll
        for (int e = 0; e < U; ++e) r[e] = __builtin_amdgcn_raw_buffer_load_b128(mb_rsrc(src), (threadIdx.x + e * 256) * 16u, 0, LAUX);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        MB_TICK(0)
        if (round) {                                               // the slot's previous contents have been read by every member
            if (threadIdx.x == 0) s_ok = team_wait(&bar->b, (unsigned)T * round, c, t_limit, waits, polls) ? 1 : 0;
            __syncthreads();
            const int ok = s_ok;
            __syncthreads();
            if (!ok) return;
        }
        MB_TICK(1)
        char* mine = slot + (size_t)member * SHARE;
#pragma unroll
        for (int e = 0; e < U; ++e) __builtin_amdgcn_raw_buffer_store_b128(r[e], mb_rsrc(mine), (threadIdx.x + e * 256) * 16u, 0, 0);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        MB_TICK(2)
        __syncthreads();
        if (threadIdx.x == 0) { atomicAdd(&bar->a, 1u); s_ok = team_wait(&bar->a, (unsigned)T * (round + 1), c, t_limit, waits, polls) ? 1 : 0; }
        __syncthreads();
        const int ok1 = s_ok;
        __syncthreads();
        if (!ok1) return;
        MB_TICK(3)
        // pass 2: a strip of every member's part: piece j of this member's second-pass share is bytes
        // [member * (SHARE / T), +SHARE / T) of member j's part
        if constexpr (((POL >> 4) & 3) == 3) asm volatile("buffer_inv sc1" ::: "memory");   // nothing of the slot's last contents is left in this CU's L1
        constexpr int STRIP = SHARE / T;                           // bytes taken from each part
        constexpr int PER = STRIP / 16;                            // 16-byte accesses per strip
#pragma unroll
        for (int e = 0; e < U; ++e) {
            const unsigned q = threadIdx.x + e * 256, j = q / PER, w = q % PER;
            r[e] = __builtin_amdgcn_raw_buffer_load_b128(mb_rsrc(slot), j * (unsigned)SHARE + member * (unsigned)STRIP + w * 16u, 0, RAUX);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);                        // the slot's loads have returned: hand the slot back before the stores
        MB_TICK(4)
        __syncthreads();                                           // to memory are issued, whose acknowledgement nobody has to wait for here
        if (threadIdx.x == 0) atomicAdd(&bar->b, 1u);
        char* dst = out + t * (size_t)PIECE;
#pragma unroll
        for (int e = 0; e < U; ++e) {
            const unsigned q = threadIdx.x + e * 256, j = q / PER, w = q % PER;
            __builtin_amdgcn_raw_buffer_store_b128(r[e], mb_rsrc(dst), j * (unsigned)SHARE + member * (unsigned)STRIP + w * 16u, 0, SAUX);
        }
        MB_TICK(5)
    }
#undef MB_TICK
    if (threadIdx.x == 0) {
        if (waits) { atomicAdd(&c->waits, waits); atomicAdd(&c->polls, polls); }
        for (int k = 0; k < 6; ++k) atomicAdd(&c->ticks[k], (unsigned long long)tk[k]);
        atomicAdd(&c->ticks[6], (unsigned long long)round);
    }
}

// `reps` timed launches between two events, after `warmup` untimed ones
template <class F>
int mb_time(F launch, int warmup, int reps, hipStream_t st, float* ms_per_pass, const char* what) {
    for (int i = 0; i < warmup; ++i) launch();
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) { tfft_set_error("%s: hipEventCreate failed", what); return TURBOFFT_EHIP; }
    if (hipEventCreate(&e1) != hipSuccess) { (void)hipEventDestroy(e0); tfft_set_error("%s: hipEventCreate failed", what); return TURBOFFT_EHIP; }
    hipError_t e = hipEventRecord(e0, st);
    for (int i = 0; i < reps; ++i) launch();
    if (e == hipSuccess) e = hipEventRecord(e1, st);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess) e = hipGetLastError();
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (e != hipSuccess) { tfft_set_error("%s: %s", what, hipGetErrorString(e)); return TURBOFFT_EHIP; }
    *ms_per_pass = ms / reps;
    return TURBOFFT_OK;
}

}  // namespace

extern "C" int turbofft_membench_strided(int write, int lane_bytes, int run_bytes, int log_stride, int xcd_chunk, const void* src_d,
                                         void* dst_d, size_t bytes, int warmup, int reps, void* stream, float* ms_per_pass) {
    if (!src_d || !dst_d || !ms_per_pass || reps < 1 || warmup < 0) { tfft_set_error("membench: bad argument"); return TURBOFFT_EINVAL; }
    if ((lane_bytes != 8 && lane_bytes != 16) || (run_bytes != 128 && run_bytes != 256 && run_bytes != 512) || log_stride < 10 || log_stride > 22 ||
        xcd_chunk < 0 || bytes == 0 || bytes % ((size_t)65536 / run_bytes << log_stride) || bytes / 65536 > 0x7fffffffull) {
        tfft_set_error("membench: lanes of 8 or 16 bytes, runs of 128, 256 or 512 bytes, stride 2^10..2^22 bytes, bytes a multiple of (65536 / run) * stride");
        return TURBOFFT_EINVAL;
    }
    const void* fns[2][2][3] = {
        {{(const void*)tfft_mb_strided<v2, 128, false>, (const void*)tfft_mb_strided<v2, 256, false>, (const void*)tfft_mb_strided<v2, 512, false>},
         {(const void*)tfft_mb_strided<v4, 128, false>, (const void*)tfft_mb_strided<v4, 256, false>, (const void*)tfft_mb_strided<v4, 512, false>}},
        {{(const void*)tfft_mb_strided<v2, 128, true>, (const void*)tfft_mb_strided<v2, 256, true>, (const void*)tfft_mb_strided<v2, 512, true>},
         {(const void*)tfft_mb_strided<v4, 128, true>, (const void*)tfft_mb_strided<v4, 256, true>, (const void*)tfft_mb_strided<v4, 512, true>}}};
    const void* fn = fns[write ? 1 : 0][lane_bytes == 16][run_bytes == 128 ? 0 : (run_bytes == 256 ? 1 : 2)];
    const unsigned grid = (unsigned)(bytes / 65536);
    hipStream_t st = (hipStream_t)stream;
    auto launch = [&]() {
        const void* in_a = src_d; void* out_a = dst_d; float* sink = (float*)dst_d; int xca = xcd_chunk; unsigned ls = (unsigned)log_stride;
        void* args[5] = {&in_a, &out_a, &sink, &xca, &ls};
        (void)hipLaunchKernel(fn, dim3(grid), dim3(256), args, 0, st);
    };
    return mb_time(launch, warmup, reps, st, ms_per_pass, "membench");
}

extern "C" int turbofft_membench_fused(int group, int ring_slots, int lag, int blocks_per_cu, const void* src_d, void* scratch_d, size_t scratch_bytes,
                                       void* dst_d, size_t bytes, int limit_ms, int warmup, int reps, void* stream, float* ms_per_pass,
                                       unsigned stats[12]) {
    if (!src_d || !dst_d || !scratch_d || !ms_per_pass || !stats || reps < 1 || warmup < 0) { tfft_set_error("membench: bad argument"); return TURBOFFT_EINVAL; }
    const long long ntrans = (long long)(bytes / kFusedTransform), per_xcd = ntrans / 8;
    // (R > lag: P1 of group g waits for P2 of group g - R, which has to come earlier in ticket order: segment g - R + lag < g)
    if (bytes == 0 || bytes % (8 * kFusedTransform) || group < 1 || lag < 1 || ring_slots <= lag || ring_slots > 16 || per_xcd % group || per_xcd / group > kFusedMaxGroups || per_xcd / group <= lag ||
        blocks_per_cu < 1 || blocks_per_cu > 8 || limit_ms < 1 || limit_ms > 1000 || (unsigned long long)8 * ring_slots * group * kFusedTransform > scratch_bytes) {
        tfft_set_error("membench: fused copy needs bytes a multiple of 4 MiB, lag >= 1, lag+1..16 ring slots of `group` 512 KiB transforms per XCD inside `scratch`, "
                       "at most %d groups per XCD, 1..8 blocks per CU and a time limit of 1..1000 ms", kFusedMaxGroups);
        return TURBOFFT_EINVAL;
    }
    int dev = 0, cus = 0, occ = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, tfft_mb_fused, 256, 0) != hipSuccess || occ < 1) {
        (void)hipGetLastError();
        tfft_set_error("membench: cannot size the persistent grid");
        return TURBOFFT_EHIP;
    }
    if (blocks_per_cu > occ) blocks_per_cu = occ;
    FusedCtl* ctl = nullptr;
    if (hipMalloc((void**)&ctl, sizeof(FusedCtl)) != hipSuccess) { (void)hipGetLastError(); tfft_set_error("membench: hipMalloc failed"); return TURBOFFT_ENOMEM; }
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)(cus * blocks_per_cu);
    auto launch = [&]() {
        hipLaunchKernelGGL(tfft_mb_fused_clear, dim3((unsigned)((sizeof(FusedCtl) / 4 + 255) / 256)), dim3(256), 0, st, ctl);
        hipLaunchKernelGGL(tfft_mb_fused, dim3(grid), dim3(256), 0, st, (const char*)src_d, (char*)scratch_d, (char*)dst_d, ctl, (int)per_xcd, group, ring_slots, limit_ms, lag);
    };
    int rc = mb_time(launch, warmup, reps, st, ms_per_pass, "membench");
    unsigned head[96];
    if (rc == TURBOFFT_OK && hipMemcpy(head, ctl, sizeof head, hipMemcpyDeviceToHost) != hipSuccess) { (void)hipGetLastError(); tfft_set_error("membench: reading the control block failed"); rc = TURBOFFT_EHIP; }
    (void)hipFree(ctl);
    if (rc) return rc;
    stats[0] = head[0]; stats[1] = head[32]; stats[2] = head[33]; stats[3] = grid;    // error flag, waits, polls, blocks
    for (int x = 0; x < 8; ++x) stats[4 + x] = head[64 + x];                          // blocks that ran on each XCD
    return TURBOFFT_OK;
}

template <int T, int PIECE>
static const void* mb_team_fn() {
    if constexpr (PIECE / T >= 4096 && PIECE / T <= 131072 && PIECE / T / T >= 16) return (const void*)tfft_mb_team<T, PIECE>;
    else return nullptr;
}
template <int POL>
static const void* mb_team_pol(int policy) {      // the other cache policies: teams of 8 with pieces of 512 KiB only
    if constexpr (POL > 63) return nullptr;
    else return policy == POL ? (const void*)tfft_mb_team<8, 512 << 10, POL> : mb_team_pol<POL + 1>(policy);
}
template <int PIECE>
static const void* mb_team_fn_t(int team_blocks) {
    switch (team_blocks) {
        case 4: return mb_team_fn<4, PIECE>();
        case 8: return mb_team_fn<8, PIECE>();
        case 16: return mb_team_fn<16, PIECE>();
        case 32: return mb_team_fn<32, PIECE>();
        default: return nullptr;
    }
}

extern "C" int turbofft_membench_team(int team_blocks, int piece_kib, int policy, int blocks_per_cu, const void* src_d, void* scratch_d, size_t scratch_bytes,
                                      void* dst_d, size_t bytes, int limit_ms, int warmup, int reps, void* stream, float* ms_per_pass,
                                      unsigned stats[12]) {
    if (!src_d || !dst_d || !scratch_d || !ms_per_pass || !stats || reps < 1 || warmup < 0) { tfft_set_error("membench: bad argument"); return TURBOFFT_EINVAL; }
    const void* fn = nullptr;
    fn = piece_kib == 128 ? mb_team_fn_t<128 << 10>(team_blocks) : piece_kib == 256 ? mb_team_fn_t<256 << 10>(team_blocks)
                   : piece_kib == 512 ? mb_team_fn_t<512 << 10>(team_blocks) : piece_kib == 1024 ? mb_team_fn_t<1024 << 10>(team_blocks) : nullptr;
    if (policy) fn = (team_blocks == 8 && piece_kib == 512) ? mb_team_pol<1>(policy) : nullptr;
    const size_t piece = (size_t)piece_kib << 10;
    if (!fn || bytes == 0 || bytes % (8 * piece) || blocks_per_cu < 1 || blocks_per_cu > 8 || limit_ms < 1 || limit_ms > 1000) {
        tfft_set_error("membench: team copy needs teams of 4, 8, 16 or 32 blocks, pieces of 128, 256, 512 or 1024 KiB with 4..128 KiB per member, "
                       "bytes a multiple of 8 pieces, 1..8 blocks per CU and a time limit of 1..1000 ms");
        return TURBOFFT_EINVAL;
    }
    int dev = 0, cus = 0, occ = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, 256, 0) != hipSuccess || occ < 1) {
        (void)hipGetLastError();
        tfft_set_error("membench: cannot size the persistent grid");
        return TURBOFFT_EHIP;
    }
    if (blocks_per_cu > occ) blocks_per_cu = occ;           // every block has to be resident: its team waits for it
    const unsigned grid = (unsigned)(cus * blocks_per_cu), nteams = (grid / 8) / (unsigned)team_blocks;
    if (nteams < 1 || nteams > 64 || (unsigned long long)8 * nteams * piece > scratch_bytes) {
        tfft_set_error("membench: %u teams per XCD need 1..64 slots of %d KiB per XCD inside `scratch`", nteams, piece_kib);
        return TURBOFFT_EINVAL;
    }
    TeamCtl* ctl = nullptr;
    if (hipMalloc((void**)&ctl, sizeof(TeamCtl)) != hipSuccess) { (void)hipGetLastError(); tfft_set_error("membench: hipMalloc failed"); return TURBOFFT_ENOMEM; }
    hipStream_t st = (hipStream_t)stream;
    const int ntrans = (int)(bytes / piece);
    auto launch = [&]() {
        hipLaunchKernelGGL(tfft_mb_team_clear, dim3((unsigned)((sizeof(TeamCtl) / 4 + 255) / 256)), dim3(256), 0, st, ctl);
        const char* in_a = (const char*)src_d; char* sc_a = (char*)scratch_d; char* out_a = (char*)dst_d; int nt = ntrans, lm = limit_ms;
        void* args[6] = {&in_a, &sc_a, &out_a, &ctl, &nt, &lm};
        (void)hipLaunchKernel(fn, dim3(grid), dim3(256), args, 0, st);
    };
    int rc = mb_time(launch, warmup, reps, st, ms_per_pass, "membench");
    unsigned head[128];
    if (rc == TURBOFFT_OK && hipMemcpy(head, ctl, sizeof head, hipMemcpyDeviceToHost) != hipSuccess) { (void)hipGetLastError(); tfft_set_error("membench: reading the control block failed"); rc = TURBOFFT_EHIP; }
    (void)hipFree(ctl);
    if (rc) return rc;
    stats[0] = head[0]; stats[1] = head[32]; stats[2] = head[33]; stats[3] = grid;
    // [4..9]: mean time per round of each part, in ticks of 10 ns; [10]: rounds per block; [11]: unused
    unsigned long long tk[7];
    memcpy(tk, head + 96, sizeof tk);
    for (int k = 0; k < 6; ++k) stats[4 + k] = tk[6] ? (unsigned)(tk[k] / tk[6]) : 0u;
    stats[10] = (unsigned)(tk[6] / (grid ? grid : 1));
    stats[11] = 0;
    return TURBOFFT_OK;
}

extern "C" int turbofft_membench(int mode, const void* src_d, void* dst_d, size_t bytes, int warmup, int reps,
                                 void* stream, float* ms_per_pass) {
    if (!src_d || !dst_d || !ms_per_pass || reps < 1 || warmup < 0) { tfft_set_error("membench: bad argument"); return TURBOFFT_EINVAL; }
    const size_t tile8 = 256 * 32 * 8, tile16 = 256 * 16 * 16;     // 64 KiB per block either way
    if (bytes == 0 || bytes % tile8 || bytes / tile8 > 0x7fffffffull) { tfft_set_error("membench: bytes must be a multiple of 65536"); return TURBOFFT_EINVAL; }
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)(bytes / tile8);
    static_assert(tile8 == tile16, "same tile bytes for both lane widths");
    // mode: bits 0-1 the kernel (0 copy with 8-byte lanes, 1 copy with 16-byte lanes, 2 read only, 3 write only),
    // bit 2 non-temporal accesses, bit 3 XCD-aware tile order (runs of 16 tiles), bits 4-7 blocks per CU (0: no limit)
    const int kind = mode & 3, nt = (mode >> 2) & 1, xc = ((mode >> 3) & 1) ? 16 : 0, bpc = (mode >> 4) & 15;
    if (mode < 0 || mode > 255) { tfft_set_error("membench: mode is a bit field below 256 (kernel | 4 non-temporal | 8 XCD-aware order | 16 * blocks per CU)"); return TURBOFFT_EINVAL; }
    const size_t lds = bpc ? (size_t)(160 * 1024 / bpc) / 1024 * 1024 : 0;
    const void* fns[8] = {(const void*)tfft_mb_copy<v2, 32, 0>, (const void*)tfft_mb_copy<v4, 16, 0>, (const void*)tfft_mb_read<v2, 32, 0>, (const void*)tfft_mb_write<v2, 32, 0>,
                          (const void*)tfft_mb_copy<v2, 32, 2>, (const void*)tfft_mb_copy<v4, 16, 2>, (const void*)tfft_mb_read<v2, 32, 2>, (const void*)tfft_mb_write<v2, 32, 2>};
    const void* fn = fns[kind + 4 * nt];
    if (lds > 48 * 1024 && hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        tfft_set_error("membench: cannot reserve %zu bytes of LDS per block", lds);
        return TURBOFFT_EHIP;
    }
    auto launch = [&]() {
        int xca = xc;
        const void* in_a = src_d; void* out_a = dst_d;
        if (kind == 3) { void* args[2] = {&out_a, &xca}; (void)hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st); }
        else { void* args[3] = {&in_a, &out_a, &xca}; (void)hipLaunchKernel(fn, dim3(grid), dim3(256), args, lds, st); }
    };
    return mb_time(launch, warmup, reps, st, ms_per_pass, "membench");
}
