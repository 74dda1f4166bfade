/* Kernel argument block shared by the host driver and every generated kernel.
 *
 * Plain C, passed by value as the last kernel argument (it lands in SGPRs).
 * It replaces the reference kernel ABI's trailing `int BS, int thread_bs`
 * (include/TurboFFT_radix_2_template.h:1-3, fft_codegen.py:207-211): the
 * reference bakes every stride into the generated text, these kernels take the
 * launch geometry at run time so one kernel per (type, kind, Ni, BS, n) serves
 * every logN that uses that tile shape.
 */
#ifndef TURBOFFT_KARGS_H
#define TURBOFFT_KARGS_H

#ifdef __cplusplus
extern "C" {
#endif

#define TFFT_FT_SUB0 16            /* first sub-counter word            */
#define TFFT_FT_SUB_STRIDE 16      /* words per sub-counter line (128 B) */
#define TFFT_FT_COUNTER_WORDS (TFFT_FT_SUB0 + 64 * TFFT_FT_SUB_STRIDE)

typedef struct tfft_ft_args {
    const void* cksum;            /* Ni entries of T: (re c + im c, re c - im c) of the input-
                                     side encoding vector c_Ni, so that re+im of x*c costs two
                                     fused multiply-adds                                      */
    unsigned long long* counters; /* TFFT_FT_COUNTER_WORDS words: [0] checksum groups run (added once per
                                     launch by its first block); 64 sub-counter lines at word
                                     TFFT_FT_SUB0 + TFFT_FT_SUB_STRIDE * (block & 63): [+0] detections
                                     (also the next free slot of that line's part of `flagged`),
                                     [+1] detections whose located tile was out of range.  Corrected
                                     = detected - unlocatable while `correct` is set.            */
    long long* flagged;           /* flagged tiles as (launch, tile) pairs: sub-counter line k owns
                                     pairs [k * cap/64, (k+1) * cap/64)                       */
    int flagged_cap;              /* pairs in `flagged`, a multiple of 64                     */
    int launch;                   /* launch index written into `flagged`                   */
    int correct;                  /* 1: recompute the located tile (the if_err=1 variants) */
    int inj_mode;                 /* 0 none; 1 reference cadence (tile cnt == block %
                                     thread_bs + 1 of every `inj_every`-th block);
                                     2 host-chosen tile(s): tile % inj_every == inj_tile   */
    int inj_every;
    long long inj_tile;
    int inj_s;                    /* sub-FFT inside the tile                               */
    int inj_m;                    /* element of that sub-FFT, 0 <= inj_m < Ni/n            */
    double inj_mag;               /* added to the real part after the input checksum       */
    double err_smoothing;         /* |delta| / (err_smoothing + |mag|) > err_threshold     */
    double err_threshold;
    /* A checksum group walked by several blocks (parts > 1, recompute-correcting kernels): the
       launch has groups * parts blocks, block b is part b / groups of group b % groups and walks
       tiles [part * part_len, (part + 1) * part_len) of the group's thread_bs.  Each block leaves
       the four running checksums of every thread in `part_sums`, takes a ticket, and the block
       that takes the group's last one adds the parts up in order and decides.  A located tile was
       stored by another block, perhaps on another XCD, whose write-back L2 may still hold it: it
       is not stored again by this launch but queued in `fix_list`, and a second launch of the
       same kernel with fix_mode = 1 (any grid) recomputes the queued tiles and empties the queue. */
    int parts;
    int part_len;
    void* part_sums;              /* [((group * parts + part) * 4 + v) * threads + thread] of the
                                     kernel's real type, v = in1, in2, out1, out2             */
    unsigned* tickets;            /* one word per group, zero between launches              */
    long long* fix_list;          /* tiles to recompute, one slot per group                 */
    unsigned* fix_ctl;            /* [0] tiles queued, [1] blocks of the fix-up launch that are
                                     done; both zero between executions                       */
    int fix_mode;                 /* 1: this launch only recomputes the queued tiles          */
} tfft_ft_args;

typedef struct tfft_kargs {
    long long ntiles;     /* tiles in this launch (a tile = BS sub-FFTs of length Ni)      */
    long long nrows;      /* row1: number of transforms (guards a ragged last tile)        */
    int thread_bs;        /* tiles a block processes in sequence (one checksum group)      */
    int tb_gap;           /* interleave distance between a block's consecutive tiles       */
    int log_ncols;        /* col : log2(contiguous columns per outer block)                */
    int logQ;             /* rowT: rows of a transform are q + Q*s', q<Q, s'<C             */
    int logC;
    int logN;             /* rowT: log2 of the whole transform                             */
    int tw_lo_bits;       /* col : W^e = tw_hi[e >> lo_bits] * tw_lo[e & mask]             */
    int xcd_chunk;        /* >0: blocks are renumbered so that each of the 8 XCDs (block % 8)
                             works on chunks of this many consecutive tiles; 0: identity      */
    const void* tw_hi;
    const void* tw_lo;
    tfft_ft_args ft;
} tfft_kargs;

/* Extra argument of a fused pair: one kernel that runs both launches of a two-launch plan.  A team of
 * `team` blocks of one XCD takes pieces of `piece_elems` elements (whole transforms) from a queue, runs
 * the column launch of a piece into the team's slot (slot k of `slots`, piece_elems elements each, meant
 * to stay in that XCD's L2), meets, and runs the row launch out of the slot.  `ctl` is the control block
 * (32-bit words, 128-byte lines so that no two counters share one; all zero between launches: the last
 * block to leave clears it):
 *   word 0                    set when a wait ran out of time (the output is then incomplete; err_host keeps the fact)
 *   word 32                   the next piece of the queue
 *   word 64                   blocks that have left
 *   word 96 + 32 * x          blocks that have arrived on XCD x (x < 8)
 *   word 352 + 128 * slot     + 0: members that finished the column launch, + 32: members that finished
 *                             reading the slot, + 64 and + 96 (two words each): the piece of even and of odd
 *                             rounds, (round + 1) << 32 | piece + 1 as named by the team's first member, piece + 1 = 0
 *                             when the queue is empty
 * A block that arrives when its XCD's `teams_per_xcd` teams are full has nothing to do. */
typedef struct tfft_fuse_args {
    void* slots;
    unsigned* ctl;
    unsigned* err_host;           /* host-visible word set together with word 0 of ctl (may be null) */
    long long piece_elems;
    long long npieces;
    int tiles_a, tiles_b;         /* tiles of the column launch and of the row launch per piece        */
    int team;                     /* blocks per team                                                  */
    int teams_per_xcd;
    int limit_ms;                 /* longest time a block waits for other blocks; negative: every block gives
                                     up as it starts (sets word 0 and err_host, does nothing else)      */
    unsigned long long* prof;     /* diagnostic builds of the kernels only (else null): 8 words per block, ticks of the
                                     100 MHz counter spent in [0] the column launch, [1] the meeting, [2] the row launch,
                                     [3] the wait for the slot to be free, [4] rounds                                 */
} tfft_fuse_args;

#define TFFT_FUSE_CTL_WORDS(slots) (352 + 128 * (slots))

#ifdef __cplusplus
}
#endif
#endif
