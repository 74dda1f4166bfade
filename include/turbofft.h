/* turbofft.h -- C ABI of libturbofft_hip.so, the MI355X (gfx950) batched
 * radix-2 C2C forward FFT engine.
 *
 * The reference (shixun404/TurboFFT) has no library API: its two seams are
 * the kernel ABI `fft_radix_2<T,logN,dim,ft,err>(in,out,twiddle,checksum_DFT,
 * BS,thread_bs)` selected from a function-pointer table
 * (include/TurboFFT.h:22-25, include/TurboFFT_radix_2_template.h:1-3,
 * launched at main.cu:48) and the `turbofft` executable with its flags
 * (include/utils/CommandLineParser.h:26-45).  Every entry point below names
 * the reference code it stands in for.  Plain pointers and sizes only; all
 * functions return 0 on success and a negative code on error, with a message
 * available from turbofft_last_error().  Nothing in the library exits the
 * process or falls back to a CPU computation.
 *
 * Data layout (main.cu:99-101, initializeData.h): interleaved {re,im},
 * batch-major x[b*N + n]; the result is out-of-place, natural order, same
 * shape.  `in` is never written.  When the plan uses more than one launch
 * `out` must hold 2*N*bs elements (initializeData.h:21, main.cu:11-12); the
 * transform is left in out[0 .. N*bs), the second half is workspace.  `in`
 * must not overlap `out` (workspace included): TURBOFFT_EINVAL otherwise.
 */
#ifndef TURBOFFT_H
#define TURBOFFT_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct turbofft_plan turbofft_plan_t;

#define TURBOFFT_FP32 0   /* float2,  --datatype 0 (CommandLineParser.h:75-77) */
#define TURBOFFT_FP64 1   /* double2, --datatype 1 */

#define TURBOFFT_OK            0
#define TURBOFFT_EINVAL       -1  /* bad argument                                   */
#define TURBOFFT_ENOPLAN      -2  /* no plan row / no compiled kernel for the shape */
#define TURBOFFT_EHIP         -3  /* a HIP runtime call failed                       */
#define TURBOFFT_ENOMEM       -4

/* Last error message of the calling thread ("" if none). */
const char* turbofft_last_error(void);

/* Create a plan for N = 2^logN.
 * Stands in for: load_parameters + params[logN] (main.cu:83, readCSV.h:14-33),
 * the TurboFFT_Kernel_Entry lookup (TurboFFT.h:22-25), the launch-geometry
 * and shared-memory attribute setup of test_turbofft (main.cu:21-42), the
 * twiddle table of initializeData (initializeData.h:31-37) and the DFT
 * checksum table (abft.h:21-61, main.cu:85-93).
 *   datatype   TURBOFFT_FP32 / TURBOFFT_FP64
 *   if_ft      1: fault-tolerant kernels (fused two-sided checksums over groups of
 *              thread_bs tiles: the scheme of the reference's current generator,
 *              fft_codegen.py:354-384,432-503)
 *              2: thread-level verification (the scheme of the reference's
 *              data_ft/ft_scheme_thread_bs=1_* tables, of which its generator keeps only the
 *              per-thread sums; the command line's --ft_scheme 1): every thread applies the same
 *              two-sided checksum (output side r[o%3], input side c_R = W_R^T r, abft.h:21-61)
 *              to the radix-R DFTs it computes in registers, pass by pass, and objects when
 *              |in - out| / (err_smoothing + |in| + |out|) > err_threshold for its two sums;
 *              nothing is summed across threads, the block only agrees on whether any thread
 *              objected, and a tile one did object to is recomputed before it is stored
 *              (bit-identical to an undisturbed run; correct = 0 stores it as computed).
 *              Every tile is its own group: `checked` counts tiles, the flagged list names
 *              them, thread_bs only shapes the grid and the injection cadence.  Runs the plain
 *              plan rows; no checksum table, no delayed correction.
 *   if_err     1: inject errors with the reference cadence and correct them
 *              (implies if_ft, CommandLineParser.h:66-68)
 *   thread_bs  tiles per block = checksum group size (--thread_bs).  Without
 *              fault tolerance it only shapes the grid; 1 (the reference's
 *              default) then lets the plan row use its own tuned value.
 *   param_csv  plan CSV in the reference's 11-column format, row index ==
 *              logN; NULL selects the built-in gfx950 table.  Up to 19 more
 *              columns per row are optional tuning flags of this library
 *              (per-launch split exchange, prefetch, cross-lane last pass,
 *              tiles per block, per-launch wavefronts per SIMD, per-launch
 *              non-temporal accesses, per-launch tiles per XCD); a reference
 *              CSV without them is valid.
 * Returns NULL on error. */
turbofft_plan_t* turbofft_plan_create(int logN, int datatype, int if_ft, int if_err,
                                      int thread_bs, const char* param_csv);

/* Stands in for the cudaFree calls at the end of TurboFFT_main (main.cu:130-132). */
void turbofft_plan_destroy(turbofft_plan_t* plan);

/* Asynchronous transform of `bs` length-N sequences on `stream`
 * (a hipStream_t; NULL = the null stream).  Device pointers.
 * Stands in for the launch loop of test_turbofft (main.cu:46-49, 55-58). */
int turbofft_exec(turbofft_plan_t* plan, const void* in_d, void* out_d, long long bs, void* stream);

/* turbofft_exec for callers that can neither allocate nor spare a 2*N*bs output buffer (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): `out_d` holds
 * N*bs elements whatever the number of launches, and the intermediate of a multi-launch plan
 * lives in a workspace that is part of the library image (a file-scope device array of
 * TURBOFFT_STATIC_WORKSPACE_BYTES per GPU, held until the process ends).  Same kernels and
 * bit-identical results as turbofft_exec.  No counterpart in the reference, whose driver
 * allocates the doubled output itself (initializeData.h:21).  Calls no allocating routine.
 * A multi-launch plan needs N*bs*sizeof(T) <= TURBOFFT_STATIC_WORKSPACE_BYTES: larger batches
 * return TURBOFFT_EINVAL (single-launch plans use no workspace and have no limit).  All calls
 * on one GPU share that GPU's workspace: executions of multi-launch plans that overlap in time
 * (two streams, two threads) race; the workspace is fully overwritten before it is read, so
 * nothing has to be cleared between calls. */
#define TURBOFFT_STATIC_WORKSPACE_BYTES (64ull << 20)
int turbofft_exec_static(turbofft_plan_t* plan, const void* in_d, void* out_d, long long bs, void* stream);

/* The unnormalised inverse transform, out[n] = sum_k in[k] exp(+2 pi i n k / N),
 * with the same plan, buffers and rules as turbofft_exec (turbofft_exec_inverse
 * of a turbofft_exec result is N times the input).  No counterpart in the
 * reference, which is forward only (the sign is fixed in its twiddle table,
 * initializeData.h:31-37, and in the generated butterflies).  inverse =
 * swap(re,im) . forward . swap(re,im): the first launch runs a flavour of its
 * kernel that exchanges re and im of what it loads, the last launch one that
 * exchanges them before storing (compile-time flavours, built for the built-in
 * plan rows).  Plain plans only: a fault-tolerant plan, or a caller's CSV whose
 * inverse flavours were not built, returns TURBOFFT_ENOPLAN. */
int turbofft_exec_inverse(turbofft_plan_t* plan, const void* in_d, void* out_d, long long bs, void* stream);

/* Same, from and to host memory (allocates device buffers, copies, runs,
 * synchronises, frees).  Stands in for initializeData's H2D copy plus the
 * D2H copy at main.cu:72.  A plain plan whose batch exceeds one piece (64 MiB
 * of input; TURBOFFT_HOST_PIECE_BYTES in the environment overrides) streams
 * the batch through three device slots on three streams of its own: copies in,
 * kernels and copies out overlap when the host buffers are page-locked
 * (hipHostMalloc), and the device memory needed is three pieces, not the
 * batch.  The result has the bits of turbofft_exec on the whole batch.
 * Fault-tolerant plans run the batch in one piece (tile groups and flagged
 * tile numbers refer to the batch as passed). */
int turbofft_exec_host(turbofft_plan_t* plan, const void* in_h, void* out_h, long long bs);

/* Timed runs with HIP events on `stream`: `warmup` untimed executions, then
 * `reps` timed ones with no host synchronisation in between; *ms_per_exec
 * receives the mean.  Stands in for the timing of test_turbofft
 * (main.cu:44-67; the reference synchronises after every launch, this does not). */
int turbofft_time(turbofft_plan_t* plan, const void* in_d, void* out_d, long long bs,
                  int warmup, int reps, void* stream, float* ms_per_exec);

/* The reference's own timing protocol: as turbofft_time, but the host waits for every launch
 * before issuing the next and once more after each execution (main.cu:53-62), so launch
 * latency and the idle device between launches are part of the figure. */
int turbofft_time_sync(turbofft_plan_t* plan, const void* in_d, void* out_d, long long bs,
                       int warmup, int reps, void* stream, float* ms_per_exec);

/* Like turbofft_time, with HIP events around every launch of the plan:
 * ms_per_launch[i] receives the mean duration of launch i (entries beyond the
 * plan's launch count are set to 0).  Always times the plan's own row (the one
 * turbofft_plan_info describes), also for a batch that turbofft_exec would hand
 * to the small-batch row.  No counterpart in the reference, which times whole
 * plans only (main.cu:52-67). */
int turbofft_time_launches(turbofft_plan_t* plan, const void* in_d, void* out_d, long long bs,
                           int warmup, int reps, void* stream, float ms_per_launch[3]);

/* Plan description: launches, per-launch log2 size, BS, n, dynamic LDS bytes,
 * threads per block (the CSV row, main.cu:8-9,22-27). */
int turbofft_plan_info(const turbofft_plan_t* plan, int* launches, int logNi[3], int BSi[3],
                       int ni[3], size_t lds_bytes[3], int threads[3]);

/* Small batches.  The plan rows are tuned with the device full (logBS+logN = 28); a batch of
 * a few transforms of 2^13..2^18 points would occupy a handful of CUs.  For those sizes the
 * built-in table holds a second row of narrow tiles in two launches (param_<T>_small.csv), and
 * a plain plan made from the built-in table runs it for bs <= turbofft_plan_small_batch_max()
 * (0: none).  Results meet the same accuracy bar; they are not bit-identical to the large-batch
 * row's, whose decomposition differs.  Buffers are unchanged (`out` as documented above).  For
 * the sizes whose large-batch row is a single launch the intermediate of the two launches is a
 * buffer the plan owns, one per stream: the first is allocated with the plan, a further stream
 * gets its own at its first small batch (up to 8 per plan; a stream beyond that, or one that is
 * being captured into a graph and has none yet, runs the large-batch row instead).  Executions
 * on different streams therefore never share an intermediate; two host threads must not issue
 * small batches of one plan on the SAME stream at once.  turbofft_plan_set_small_batch(plan, 0)
 * switches the row off.  No counterpart in the reference, which has one row per size
 * (main.cu:99,123). */
long long turbofft_plan_small_batch_max(const turbofft_plan_t* plan);
int turbofft_plan_set_small_batch(turbofft_plan_t* plan, int enable);
/* What a batch of `bs` transforms actually runs (the small-batch row up to its cap, else the
 * plan's own row, which turbofft_plan_info / _grid / _kernel_name describe): its number of
 * launches and the kernel of each. */
int turbofft_plan_launches_for_batch(const turbofft_plan_t* plan, long long bs);
const char* turbofft_plan_kernel_name_for_batch(const turbofft_plan_t* plan, int launch, long long bs);

/* Name of the kernel that launch `launch` of a forward execution runs with the plan's current
 * settings (correction scheme, checksum table, threshold); the role of reading
 * TurboFFT_Kernel_Entry's table entry (TurboFFT.h:22-25).  Describes the plan's own row;
 * turbofft_plan_kernel_name_for_batch tells what a given batch runs. */
const char* turbofft_plan_kernel_name(const turbofft_plan_t* plan, int launch);

/* Grid size of launch `launch` for `bs` transforms (main.cu:32). */
long long turbofft_plan_grid(const turbofft_plan_t* plan, int launch, long long bs);

/* Tile interleave distance of launch `launch` (the reference's tb_gap,
 * fft_codegen.py:216-218, with resident blocks measured on this device). */
int turbofft_plan_tb_gap(const turbofft_plan_t* plan, int launch);
/* Override it (tests use this to make groups reproducible). */
int turbofft_plan_set_tb_gap(turbofft_plan_t* plan, int launch, int tb_gap);

/* A checksum group is the reference's thread_bs tiles of one block (fft_codegen.py:216-218,
 * 354-384).  Here a group longer than `tiles` tiles is walked by several blocks, `tiles` each:
 * every block leaves its threads' running checksums in slots the plan owns and takes a ticket,
 * and the block that takes a group's last ticket adds the parts up in order and applies the
 * reference's rule to the whole group.  Same groups, same sums, same decisions (to rounding: the
 * sums are added in another order); no block waits for another.  A located tile is recomputed
 * by a second launch of the same kernel that follows at once (the tile's first store came from
 * another block, perhaps on another XCD; the kernel boundary orders the two stores), which
 * returns at once when nothing was located.  Default 8 tiles per block (TURBOFFT_FT_PART_LEN
 * at plan creation overrides; 0 = one block per group, as the reference), so groups of 16 and
 * more are shared; recompute-correcting kernels that do not prefetch only.  The slots (128 MiB
 * and 12 MiB of tickets and queue) are allocated by the first execution that shares a group;
 * an execution that would need more, or whose stream is being captured into a graph before
 * the slots exist, runs one block per group.  turbofft_plan_grid keeps returning
 * the number of groups.  Executions of one fault-tolerant plan must not overlap in time (they
 * share the slots). */
int turbofft_plan_set_ft_part_len(turbofft_plan_t* plan, int launch, int tiles);
int turbofft_plan_ft_part_len(const turbofft_plan_t* plan, int launch);

/* ---- fault tolerance (no counterpart API in the reference; its generator
 * bakes these into the kernel text: fft_codegen.py:412-415, 495, 714-719) ---- */

/* Detection rule |delta| / (err_smoothing + |mag|) > err_threshold, and what happens to a
 * located tile:
 *   correct 0  detect and report only
 *   correct 1  recompute the tile from its input (the correction the reference's if_err=1
 *              kernels run, fft_codegen.py:149-193); the result is bit-identical to an
 *              undisturbed run
 *   correct 2  delayed batch correction: every thread keeps the sums of the inputs and of the
 *              outputs of its group's tiles (the live sums of fft_codegen.py:355-357,421-423)
 *              and the located tile is patched in place with FFT(sum x) - sum y (the lines
 *              commented at fft_codegen.py:401-404,427-429; test.ipynb cell 0).  The tile's
 *              input is not read again; the patched result equals the undisturbed one to
 *              rounding, not bit for bit.  Kernels of this flavour are built for the built-in
 *              fault-tolerant plan rows; TURBOFFT_ENOPLAN otherwise. */
int turbofft_set_ft_params(turbofft_plan_t* plan, double err_smoothing, double err_threshold, int correct);

/* Which checksum table the plan's kernels read: 0 = exact angles (the default), 1 = the
 * reference's own table, whose angles 2*pi*i*j are rounded to float before the division by N
 * (abft.h:34-35,55-56, built at main.cu:85-93).  Waits for the plan's last execution, then
 * replaces the tables.  The environment variable TURBOFFT_CHECKSUM_MODE=1 selects mode 1 at
 * plan creation. */
int turbofft_set_checksum_mode(turbofft_plan_t* plan, int mode);
/* Compact checksum table.  For some sizes the built-in fault-tolerant rows (columns 31-33 of
 * param_<T>_ft.csv) run a kernel flavour that does not hold the complex input-side vector c_N in
 * registers (2n per lane) but reads one real number per element: with the exact cube root,
 * c_N[m] = kappa (1 - i cot(pi (m/N + 1/3))), kappa = (1 - rho^N)/2.  The cotangents are stored
 * in half precision for fp32 kernels and in single precision for fp64 kernels (a quarter of the
 * complex table), which leaves a residual of up to 1e-4 (1e-8) of the checksum magnitude on clean
 * data: the flavour runs while err_threshold >= 5e-4 (1e-6) and the checksum mode is 0, otherwise
 * the same launch runs its full-table flavour.  TURBOFFT_COMPACT_CHECKSUM=0 in the environment
 * at plan creation keeps the full tables always.  The checksum arithmetic is otherwise the
 * reference's (fft_codegen.py:354-367); it has no compact form. */

/* Error injection for the launch `launch` (-1 = last, the reference's choice):
 *   mode 0  none
 *   mode 1  reference cadence: in every `every`-th block, the tile with
 *           cnt == block % thread_bs + 1 gets `mag` added to re of element
 *           (s, m) after the input checksum (s = m = 0 in the reference);
 *           m is limited to the first Ni/n elements of the sub-FFT
 *   mode 2  tiles with tile % every == tile_phase                              */
int turbofft_set_injection(turbofft_plan_t* plan, int mode, int launch, int every,
                           long long tile_phase, int s, int m, double mag);

/* Counters accumulated since the last reset: groups checked, detected, corrected,
 * uncorrectable (located tile out of range); flagged[2*i] = launch, flagged[2*i+1] = tile
 * (-1 if not locatable), up to `cap` pairs in no particular order; *nflagged receives the
 * number written.  The plan records at most 4096 pairs between resets, in 64 sub-lists of 64
 * chosen by the low bits of the detecting block's index (so that a launch in which every
 * group detects does not queue on one counter): the list is truncated when *detected
 * exceeds *nflagged.  All four counters live on the device (`checked` is added by the first
 * block of every launch), so replays of a captured HIP graph are counted.  Waits for the
 * stream of the plan's most recent turbofft_exec only, not for the device: work the caller
 * put on other streams (a graph replayed elsewhere) has to be synchronised by the caller. */
int turbofft_get_ft_counters(turbofft_plan_t* plan, unsigned long long* checked,
                             unsigned long long* detected, unsigned long long* corrected,
                             unsigned long long* uncorrectable, long long* flagged, int cap,
                             int* nflagged);
int turbofft_reset_ft_counters(turbofft_plan_t* plan);

/* ---- host tables (no device needed) ---- */

/* tw[c-1+m] = exp(-2 pi i m / c), c = 1,2,4..N; 2N-1 entries of T
 * (initializeData.h:31-37). */
int turbofft_build_twiddle_table(int datatype, long long N, void* out);

/* c_N[i] = sum_j W_N^{ij} r[j%3], N entries of T (abft.h:21-61).
 * mode 0: exact angles; mode 1: the reference's float-rounded angles. */
int turbofft_build_checksum_vector(int datatype, long long N, int mode, void* out);

/* Built-in gfx950 plan row for logN: writes the 11 CSV columns. */
int turbofft_builtin_plan_row(int datatype, int logN, int row[11]);

/* Number of compiled kernels and their names (registry introspection; the
 * role of test.py, which prints the reference's dispatch tables). */
int turbofft_kernel_count(void);
const char* turbofft_kernel_name(int i);

/* ---- vendor-library side-by-side (measurement and cross-check only) ----
 * The role of profiler::cufft::test_cufft (include/cufft/cufft.h:14-56 fp32,
 * :59-101 fp64; called at main.cu:99,105,121) with hipFFT where the reference
 * uses cuFFT.  hipFFT is opened with dlopen at first use; when it is absent
 * these return TURBOFFT_ENOPLAN and the rest of the library is unaffected.
 * No transform of this library is computed by the vendor code. */

/* 1 when libhipfft.so can be opened, else 0. */
int turbofft_vendor_available(void);

/* One forward C2C/Z2Z transform of `bs` length-2^logN sequences by hipFFT,
 * device pointers, synchronised on return (hipfftPlan1d + exec + destroy,
 * cufft.h:23-31,48-52). */
int turbofft_vendor_exec(int logN, int datatype, const void* in_d, void* out_d, long long bs, void* stream);

/* Timed like turbofft_time: `warmup` untimed and `reps` timed executions of one
 * hipFFT plan between two HIP events, no host synchronisation in between
 * (cufft.h:26-42 synchronises after every execution). */
int turbofft_vendor_time(int logN, int datatype, const void* in_d, void* out_d, long long bs,
                         int warmup, int reps, void* stream, float* ms_per_exec);

/* ---- offline checksums (measurement and cross-check only) ----
 * The baseline the fused scheme is compared with (include/cufft/cufft_ft.h:19-95:
 * checksum pass over the input, library transform, checksum pass over the output,
 * each its own launch; the reference pairs cuBLAS gemv with cuFFT).  Same
 * arithmetic as the fused kernels, per transform:
 *   in_sums[b]  = re+im of sum_m x[b][m] c_N[m],   out_sums[b] = re+im of sum_k y[b][k] r[k%3]. */

/* The two checksum passes alone, on a given input and an already computed
 * output; in_sums_d / out_sums_d receive bs values of the real type (float or
 * double) in device memory.  Synchronised on return. */
int turbofft_offline_checksums(int logN, int datatype, const void* in_d, const void* out_d, long long bs,
                               void* in_sums_d, void* out_sums_d, void* stream);

/* Timed like turbofft_time: input pass, this library's plain plan, output pass
 * and the per-transform comparison |in - out| / (1000 + mag) > 1e-3, `reps`
 * times between two HIP events.  out_d as for turbofft_exec (2*N*bs elements
 * when the plan has more than one launch).  *flagged_rows (may be NULL)
 * receives the number of transforms the last repetition flagged. */
int turbofft_offline_ft_time(int logN, int datatype, const void* in_d, void* out_d, long long bs,
                             int warmup, int reps, void* stream, float* ms_per_exec,
                             unsigned long long* flagged_rows);

/* ---- streaming kernels of known traffic (measurement only) ----
 * One pass over `bytes` (a multiple of 65536) in 64 KiB tiles per 256-thread block, all loads
 * of a tile issued before its first store, timed like turbofft_time:
 *   mode bits 0-1: 0  copy src -> dst, 8-byte lanes      1  copy, 16-byte lanes
 *                  2  read src only                      3  write dst only
 *   mode bit 2 (+4):  non-temporal accesses, as the FFT kernels mark their tile data
 *   mode bit 3 (+8):  XCD-aware tile order (runs of 16 consecutive tiles per XCD), as the FFT kernels use
 *   mode bits 4-7 (+16*k): at most k blocks resident per CU (unused LDS reserved per block; 0: no limit)
 * The yardsticks the FFT kernels are compared with, and kernels of known size for scaling
 * hardware traffic counters.  No counterpart in the reference. */
int turbofft_membench(int mode, const void* src_d, void* dst_d, size_t bytes, int warmup, int reps,
                      void* stream, float* ms_per_pass);

/* Read-only (write = 0: sweeps src) or write-only (write = 1: fills dst) pass over `bytes` in 64 KiB tiles that
 * are rows of `run_bytes` (128, 256, 512) at a stride of 2^log_stride bytes -- the access pattern of the column
 * kernels (runs of BS elements at the stride of their digit) and of the transposed store of the last launch --
 * with lanes of `lane_bytes` (8, 16), non-temporal accesses and runs of `xcd_chunk` consecutive tiles per XCD
 * (0: plain block order).  `bytes` is a multiple of (65536 / run_bytes) << log_stride. */
int turbofft_membench_strided(int write, int lane_bytes, int run_bytes, int log_stride, int xcd_chunk, const void* src_d,
                              void* dst_d, size_t bytes, int warmup, int reps, void* stream, float* ms_per_pass);

/* Two passes through a ring that is meant to stay in the XCD's L2: a copy src -> ring -> dst as ONE persistent
 * kernel (`blocks_per_cu` blocks per CU), the data cut into 512 KiB pieces that the 8 XCDs own in turn, each XCD
 * with `ring_slots` (lag+1..16) slots of `group` pieces inside `scratch_d` (8 * ring_slots * group * 512 KiB), reused for
 * every group; the second pass of a group starts when its first pass is complete, as the row pass of a two-launch
 * plan needs every column tile of its transform, and is handed out `lag` groups behind the first pass, so that with a
 * large enough lag no block finds a group's first pass still running.  Measures whether a fused pass pair could keep its intermediate
 * on chip (rocprofv3's FETCH_SIZE / WRITE_SIZE of the kernel tell where the ring's traffic went).  Every wait inside
 * the kernel is for work that running blocks hold and is bounded by `limit_ms` per launch: on a time-out the kernel
 * drains and stats[0] is 1.  stats: [0] time-out flag, [1] waits that had to poll, [2] polls, [3] blocks launched,
 * [4..11] blocks that ran on each XCD.  dst equals src afterwards.  `bytes` is a multiple of 4 MiB. */
int turbofft_membench_fused(int group, int ring_slots, int lag, int blocks_per_cu, const void* src_d, void* scratch_d, size_t scratch_bytes,
                            void* dst_d, size_t bytes, int limit_ms, int warmup, int reps, void* stream, float* ms_per_pass,
                            unsigned stats[12]);

/* The same copy with teams instead of tickets: `team_blocks` (4, 8, 16, 32) blocks of one XCD share one piece of
 * `piece_kib` KiB (128, 256, 512, 1024; 4..128 KiB per member) at a time and one slot of `scratch_d` (blocks per XCD /
 * team_blocks slots per XCD), meeting at a team barrier between the pass that fills the slot and the pass that drains
 * it (each member drains a strip of every member's part) and again before the slot is overwritten.  The whole grid
 * (`blocks_per_cu`, at most what fits) has to be resident at once; waits are bounded by `limit_ms` as in
 * turbofft_membench_fused.  stats: [0] time-out flag, [1] waits that had to poll, [2] polls, [3] blocks launched, [4..9] mean
 * time per round, in units of 10 ns, that a block spends waiting for the piece's loads, waiting for the slot, on the slot's
 * stores, in the team barrier, on the slot's loads, on the rest, [10] rounds per block.  `bytes` is a multiple of 8 pieces.  `policy` (teams of 8
 * with pieces of 512 KiB only, else 0) picks the cache policy of the accesses to memory: loads of src in bits 0-1,
 * stores to dst in bits 2-3, each 0 non-temporal, 1 that with sc0, 2 with sc1, 3 with both. */
int turbofft_membench_team(int team_blocks, int piece_kib, int policy, int blocks_per_cu, const void* src_d, void* scratch_d, size_t scratch_bytes,
                           void* dst_d, size_t bytes, int limit_ms, int warmup, int reps, void* stream, float* ms_per_pass,
                           unsigned stats[12]);

/* Fused pairs.  For some sizes a plain built-in two-launch plan also holds ONE kernel that runs both launches
 * (param/gfx950/param_<T>_pair.csv): teams of blocks on one XCD take pieces of a few whole transforms from a queue,
 * run the column launch of a piece into a slot that the XCD's L2 holds, meet, and run the row launch out of the slot,
 * so the plan's intermediate never travels to memory.  It runs for batches that give every team a piece; `out` may
 * then hold N*bs elements only.  Every block of its grid has to be resident at once: it is sized for a GPU it has to
 * itself, shares the CUs with other kernels correctly as long as those finish on their own, and bounds every wait
 * (TURBOFFT_FUSED_LIMIT_MS, default 2000): should the limit ever be reached the output of that execution is
 * incomplete, the next turbofft_exec on that stream returns TURBOFFT_EHIP saying so, and the plan goes back to its
 * two launches.  Every stream that runs the fused kernel owns a set of slots (8 sets per plan; later streams, and
 * streams that first show up while being captured, run the two launches).
 * turbofft_plan_set_fused switches it off or on for a plan; TURBOFFT_FUSED=0 in the environment leaves it out of
 * new plans.  turbofft_plan_fused_info returns 1 when the plan holds an enabled fused kernel, 0 when not, and fills
 * in (where non-null) the blocks per team, transforms per piece, teams per XCD and blocks of its grid.
 * No counterpart in the reference, whose multi-launch plans always store and reload the intermediate
 * (main.cu:16-30). */
int turbofft_plan_set_fused(turbofft_plan_t* plan, int enable);
int turbofft_plan_fused_info(const turbofft_plan_t* plan, int* team_blocks, int* transforms_per_piece, int* teams_per_xcd, int* grid_blocks);

/* The `turbofft` command line (main.cu:137-169 + CommandLineParser.h): same
 * flags and output lines.  Returns the process exit code. */
int turbofft_main(int argc, char** argv);

#ifdef __cplusplus
}
#endif
#endif
