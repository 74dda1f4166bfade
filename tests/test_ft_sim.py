"""Fault-tolerance path of the generated kernels, run in the CPU lock-step
flavour: detection, location, recompute-correction, injection cadence and the
counters, against the oracle's model of the reference checksum scheme."""
import ctypes as C

import numpy as np
import pytest

from oracle import turbofft_oracle as O
from tests import simlib
from turbofft_amd.codegen.fft_codegen import KernelSpec
from turbofft_amd.codegen.plan import KernelKey


def rnd(shape, seed):
    rng = np.random.default_rng(seed)
    return rng.uniform(-1, 1, shape) + 1j * rng.uniform(-1, 1, shape)


def run_ft(dtype, logNi, BS, n, ntiles, thread_bs, tb_gap, inj_mode, correct, inj_every=1, inj_tile=0, inj_s=0,
           inj_m=0, mag=100.0, seed=0, split=0, pf=0, ft=1, ck=0, part_len=0):
    sp = KernelSpec(KernelKey(dtype, "row1", logNi, BS, n, ft, split, pf, ck=ck))
    N = 1 << logNi
    bs = ntiles * BS
    x = rnd((bs, N), seed).astype(simlib.ctype_of(dtype))
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = ntiles, bs, thread_bs, tb_gap
    st = simlib.FtState(ka)
    ka.ft.launch = 0
    ka.ft.correct = correct
    ka.ft.inj_mode, ka.ft.inj_every, ka.ft.inj_tile, ka.ft.inj_s, ka.ft.inj_m, ka.ft.inj_mag = \
        inj_mode, inj_every, inj_tile, inj_s, inj_m, mag
    ka.ft.err_smoothing, ka.ft.err_threshold = 1000.0, 1e-3
    grid = (ntiles + thread_bs - 1) // thread_bs
    if part_len:
        # every group is shared by ceil(thread_bs / part_len) blocks (block b: part b / groups of group b % groups)
        parts = -(-thread_bs // part_len)
        sums = np.full(grid * parts * 4 * sp.threads, np.nan, dtype=np.float32 if dtype == "float2" else np.float64)
        tickets = np.zeros(grid, dtype=np.uint32)
        fix_list = np.full(grid, -9, dtype=np.int64)
        fix_ctl = np.zeros(2, dtype=np.uint32)
        ka.ft.parts, ka.ft.part_len, ka.ft.part_sums, ka.ft.tickets = parts, part_len, sums.ctypes.data, tickets.ctypes.data
        ka.ft.fix_list, ka.ft.fix_ctl = fix_list.ctypes.data, fix_ctl.ctypes.data
        grid *= parts
    cv = O.dft_checksum_vector(N, dtype).astype(np.complex128)
    ck = (cv.real + cv.imag) + 1j * (cv.real - cv.imag)      # device form of the table
    if sp.ck16:
        ck = O.compact_table_words(N, n, dtype).view(simlib.ctype_of(dtype))   # the compact table, as the buffer type the launcher passes
    y = simlib.run_sim(sp, x, bs * N, ka, grid, simlib.twiddle_table(N, dtype), ck=ck)
    if part_len:
        # the fix-up launch: the same kernel recomputes the tiles the first launch queued and empties the queue
        queued = int(fix_ctl[0])
        ka.ft.parts, ka.ft.fix_mode = 1, 1
        y = simlib.run_sim(sp, x, bs * N, ka, 3, simlib.twiddle_table(N, dtype), ck=ck, out=y)
        assert not fix_ctl.any()
        assert queued == (st.detected - st.unlocatable if correct else 0)
    y = y.reshape(bs, N)
    # the kernels keep detections and unlocatable detections; the host derives the rest the same
    # way the library does: [0] checked, [1] detected, [2] corrected, [3] uncorrectable
    counters = [st.checked, st.detected, st.detected - st.unlocatable if correct else 0, st.unlocatable]
    fl = st.pairs()
    if part_len:
        assert not tickets.any()            # every group's last block leaves its ticket word at zero
    return sp, x, y, counters, fl


@pytest.mark.parametrize("dtype", ["float2", "double2"])
def test_clean_run_detects_nothing(dtype):
    sp, x, y, c, fl = run_ft(dtype, 8, 4, 16, 24, 4, 3, inj_mode=0, correct=1)
    assert c[1] == 0 and c[2] == 0 and not fl
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, 8)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("logNi,BS,n", [(8, 4, 16), (7, 8, 8), (10, 1, 8)])
def test_reference_cadence_detect_locate_correct(dtype, logNi, BS, n):
    ntiles, tbs, gap = 24, 4, 3
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=1, correct=1)
    groups = O.tile_groups(ntiles, tbs, gap)
    injs = O.reference_injections(groups, tbs, 100.0)
    assert c[1] == len(injs) == c[2] and c[3] == 0
    # located tiles are exactly the injected ones (decision parity with the oracle model)
    assert sorted(t for _, t in fl) == sorted(i.tile for i in injs)
    xt = x.reshape(ntiles, BS, -1)
    yt = O.fft_ref(xt).astype(simlib.ctype_of(dtype))
    for inj in injs:
        yt[inj.tile, inj.s, :] += inj.mag
    dec = O.ft_launch_model(xt, yt, n, groups, dtype, O.dft_checksum_vector(1 << logNi, dtype))
    assert sorted(d.tile for d in dec if d.detected) == sorted(t for _, t in fl)
    # corrected output equals the clean transform
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, logNi)


def test_detection_without_correction_leaves_the_error():
    sp, x, y, c, fl = run_ft("double2", 8, 4, 16, 8, 2, 2, inj_mode=1, correct=0)
    assert c[1] == 4 and c[2] == 0
    err = np.abs(y - O.fft_ref(x)).reshape(8, 4, 256)
    groups = O.tile_groups(8, 2, 2)
    for inj in O.reference_injections(groups, 2, 100.0):
        assert np.allclose(err[inj.tile, 0], 100.0, rtol=1e-9)      # every output of that sub-FFT is off by mag
        assert err[inj.tile, 1:].max() < 1e-9


def test_host_chosen_injection_single_tile():
    # mode 2: one tile in the whole run, arbitrary element
    ntiles, tbs, gap = 20, 5, 2
    sp, x, y, c, fl = run_ft("float2", 8, 4, 16, ntiles, tbs, gap, inj_mode=2, correct=1, inj_every=1000,
                             inj_tile=13, inj_s=2, inj_m=11, mag=100.0)
    assert c[1] == 1 and c[2] == 1 and fl == [(0, 13)]
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance("float2", 8)


def test_injection_on_arbitrary_element_matches_model_delta():
    # error on x[m] shifts y[k] by mag*W^{mk}; the model must see the same delta sign/size
    ntiles, tbs, gap = 4, 4, 1
    sp, x, y, c, fl = run_ft("double2", 7, 8, 8, ntiles, tbs, gap, inj_mode=2, correct=0, inj_every=1000,
                             inj_tile=2, inj_s=5, inj_m=3, mag=50.0)
    assert c[1] == 1 and fl == [(0, 2)]
    k = np.arange(128)
    err = (y - O.fft_ref(x)).reshape(4, 8, 128)[2, 5]
    assert np.allclose(err, 50.0 * np.exp(-2j * np.pi * 3 * k / 128), atol=1e-9)


def test_ft_with_split_exchange():
    sp, x, y, c, fl = run_ft("double2", 8, 4, 16, 24, 4, 3, inj_mode=1, correct=1, split=1)
    assert c[1] == 6 == c[2]
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance("double2", 8)


def test_ft_with_prefetch_recomputes_the_located_tile():
    sp, x, y, c, fl = run_ft("float2", 8, 4, 16, 24, 4, 3, inj_mode=1, correct=1, pf=1)
    assert c[1] == 6 == c[2]
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance("float2", 8)
    sp, x, y, c, fl = run_ft("double2", 10, 1, 8, 20, 5, 2, inj_mode=2, correct=1, inj_every=1000, inj_tile=13, pf=1)
    assert c[1] == 1 and c[2] == 1 and fl == [(0, 13)]
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance("double2", 10)


def test_table_in_registers_or_read_per_tile():
    """Blocks of up to 512 threads read their checksum-table entries once and keep them for
    all their tiles; 1024-thread blocks (128 registers per lane) re-read them per tile in
    batches.  Same arithmetic either way: decisions and correction as usual."""
    from turbofft_amd.codegen.fft_codegen import KernelEmitter
    for logNi, BS, n, resident in ((10, 8, 16, True), (10, 8, 8, False)):
        sp = KernelSpec(KernelKey("double2", "row1", logNi, BS, n, 1))
        assert KernelEmitter(sp).ft_table_resident() == resident and (sp.threads < 1024) == resident
        ntiles, tbs, gap = 6, 3, 2
        sp, x, y, c, fl = run_ft("double2", logNi, BS, n, ntiles, tbs, gap, inj_mode=2, correct=1, inj_every=1000,
                                 inj_tile=4, inj_s=5, inj_m=17, mag=1.0e4)
        assert c[1] == 1 and c[2] == 1 and fl == [(0, 4)]
        assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance("double2", logNi)
        sp, x, y, c, fl = run_ft("double2", logNi, BS, n, ntiles, tbs, gap, inj_mode=0, correct=1)
        assert c[1] == 0 and not fl


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("logNi,BS,n,split", [(8, 4, 16, 0), (7, 8, 8, 0), (10, 1, 8, 1), (6, 8, 4, 0)])
def test_delayed_batch_correction_flavour(dtype, logNi, BS, n, split):
    # the `_fd` kernels keep per-thread sums of the group's inputs and outputs and patch the
    # located tile with FFT(sum x) - sum y instead of recomputing it from its input
    ntiles, tbs, gap = 22, 4, 3                    # ragged last group
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=1, correct=1, split=split, ft=2)
    groups = O.tile_groups(ntiles, tbs, gap)
    injs = O.reference_injections(groups, tbs, 100.0)
    assert c[0] == len(groups)
    assert c[1] == len(injs) == c[2] and c[3] == 0
    assert sorted(t for _, t in fl) == sorted(i.tile for i in injs)
    ref = O.fft_ref(x)
    assert O.rel_l2(y, ref) < O.tolerance(dtype, logNi)
    # tile by tile against the oracle's delayed correction of the same group
    xt = x.reshape(ntiles, BS, -1)
    yt = O.fft_ref(xt)
    ct = simlib.ctype_of(dtype)
    for inj in injs:
        g = next(gr for gr in groups if inj.tile in gr)
        yg = yt[g].astype(ct)
        yg[g.index(inj.tile), inj.s, :] += inj.mag
        want = O.delayed_batch_correction(xt[g], yg, g.index(inj.tile), n, dtype)
        got = y.reshape(ntiles, BS, -1)[inj.tile]
        assert O.rel_l2(got, want) < O.tolerance(dtype, logNi)
    # without correction the error stays, and a clean run is untouched by the extra sums
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=0, correct=1, split=split, ft=2)
    assert c[1] == 0 and O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, logNi)


def test_delayed_batch_correction_ragged_rows():
    # a last tile with fewer transforms than BS: the patch reads and writes only rows that exist
    dtype, logNi, BS, n = "double2", 7, 8, 8
    sp = KernelSpec(KernelKey(dtype, "row1", logNi, BS, n, 2))
    N, bs = 1 << logNi, 8 * 5 + 3
    ntiles = (bs + BS - 1) // BS
    x = rnd((bs, N), 9).astype(np.complex128)
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = ntiles, bs, 3, 2
    st = simlib.FtState(ka)
    ka.ft.correct, ka.ft.inj_mode, ka.ft.inj_every, ka.ft.inj_tile, ka.ft.inj_mag = 1, 2, 1 << 30, ntiles - 1, 100.0
    ka.ft.err_smoothing, ka.ft.err_threshold = 1000.0, 1e-3
    cv = O.dft_checksum_vector(N, dtype).astype(np.complex128)
    ck = (cv.real + cv.imag) + 1j * (cv.real - cv.imag)
    y = simlib.run_sim(sp, x, bs * N, ka, (ntiles + 2) // 3, simlib.twiddle_table(N, dtype), ck=ck).reshape(bs, N)
    assert st.detected == 1 and st.unlocatable == 0 and st.pairs() == [(0, ntiles - 1)]
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, logNi)


def _ft_args(ka, ntiles, correct, inj_tile, mag):
    st = simlib.FtState(ka)
    ka.ft.correct, ka.ft.inj_mode, ka.ft.inj_every, ka.ft.inj_tile, ka.ft.inj_mag = correct, 2, 1 << 30, inj_tile, mag
    ka.ft.inj_s, ka.ft.inj_m = 1, 0
    ka.ft.err_smoothing, ka.ft.err_threshold = 1000.0, 1e-3
    return st


@pytest.mark.parametrize("ft,tbs", [(1, 3), (2, 3), (2, 1)])
@pytest.mark.parametrize("dtype,logNi,BS,n,log_ncols", [("double2", 7, 16, 8, 8), ("float2", 8, 16, 16, 6)])
def test_column_kernel_corrects_an_injected_tile(ft, tbs, dtype, logNi, BS, n, log_ncols):
    # recompute (ft=1) and delayed batch correction (ft=2) in a column launch: the patch of
    # the delayed flavour is formed before the inter-launch twiddle and multiplied by it
    sp = KernelSpec(KernelKey(dtype, "col", logNi, BS, n, ft))
    Ni, ncols, outer = 1 << logNi, 1 << log_ncols, 3
    x = rnd((outer, Ni, ncols), 5)
    ka = simlib.KArgs()
    ka.ntiles = outer * ncols // BS
    ka.thread_bs, ka.tb_gap, ka.log_ncols = tbs, 2, log_ncols
    lo_bits, hi, lo = simlib.split_tables(logNi + log_ncols, dtype)
    ka.tw_lo_bits = lo_bits
    st = _ft_args(ka, ka.ntiles, 1, 7, 1e4)
    cv = O.dft_checksum_vector(Ni, dtype).astype(np.complex128)
    ck = (cv.real + cv.imag) + 1j * (cv.real - cv.imag)
    grid = (ka.ntiles + tbs - 1) // tbs
    y = simlib.run_sim(sp, x, x.size, ka, grid, simlib.twiddle_table(Ni, dtype), hi, lo, ck=ck).reshape(outer, Ni, ncols)
    assert st.checked == grid and st.detected == 1 and st.unlocatable == 0 and st.pairs() == [(0, 7)]
    ref = np.fft.fft(x.astype(simlib.ctype_of(dtype)).astype(np.complex128), axis=1)
    k = np.arange(Ni)[:, None]
    col = np.arange(ncols)[None, :]
    ref = ref * np.exp(-2j * np.pi * ((k * col) % (Ni * ncols)) / (Ni * ncols))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, logNi)


@pytest.mark.parametrize("ft,tbs", [(1, 2), (2, 2), (2, 1)])
@pytest.mark.parametrize("dtype,logA,BS,n,logQ,logC", [("double2", 8, 8, 8, 0, 4), ("float2", 8, 16, 16, 3, 4)])
def test_transposing_kernel_corrects_an_injected_tile(ft, tbs, dtype, logA, BS, n, logQ, logC):
    sp = KernelSpec(KernelKey(dtype, "rowT", logA, BS, n, ft))
    A, Q, Cc = 1 << logA, 1 << logQ, 1 << logC
    bs = 2
    x = rnd((bs, Cc, Q, A), 7)
    ka = simlib.KArgs()
    ka.ntiles = bs * Q * Cc // BS
    ka.thread_bs, ka.tb_gap = tbs, 3
    ka.logQ, ka.logC, ka.logN = logQ, logC, logA + logQ + logC
    st = _ft_args(ka, ka.ntiles, 1, ka.ntiles - 1, 1e4)
    cv = O.dft_checksum_vector(A, dtype).astype(np.complex128)
    ck = (cv.real + cv.imag) + 1j * (cv.real - cv.imag)
    grid = (ka.ntiles + tbs - 1) // tbs
    y = simlib.run_sim(sp, x, x.size, ka, grid, simlib.twiddle_table(A, dtype), ck=ck).reshape(bs, A, Q, Cc)
    assert st.checked == grid and st.detected == 1 and st.unlocatable == 0 and st.pairs() == [(0, ka.ntiles - 1)]
    xc = x.astype(simlib.ctype_of(dtype)).astype(np.complex128)
    ref = np.transpose(np.fft.fft(xc, axis=3), (0, 3, 2, 1))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, logA)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("logNi,BS,n", [(8, 4, 16), (10, 1, 8)])
def test_delayed_flavour_checks_a_single_tile_group_before_storing(dtype, logNi, BS, n):
    # thread_bs = 1: every group is one tile, the reference cadence injects into every tile.  The
    # `_fd` kernels hold such a tile in registers until it is checked and transform the saved
    # input again when it is flagged, so the result is bit-identical to an undisturbed run.
    ntiles = 9
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, 1, 3, inj_mode=1, correct=1, ft=2)
    assert c[0] == ntiles and c[1] == ntiles == c[2] and c[3] == 0
    assert sorted(t for _, t in fl) == list(range(ntiles))
    sp, x0, y0, c0, fl0 = run_ft(dtype, logNi, BS, n, ntiles, 1, 3, inj_mode=0, correct=1, ft=2)
    assert c0[1] == 0 and np.array_equal(x, x0) and np.array_equal(y, y0)
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, logNi)
    # detect only: the held tile is stored as computed, error included
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, 1, 3, inj_mode=1, correct=0, ft=2)
    assert c[1] == ntiles and c[2] == 0
    err = np.abs(y - O.fft_ref(x)).reshape(ntiles, BS, -1)
    assert np.allclose(err[:, 0, :], 100.0, rtol=1e-3) and (BS == 1 or err[:, 1:, :].max() < 1e-2)


@pytest.mark.parametrize("dtype,ck", [("float2", 1), ("float2", 2), ("float2", 3), ("double2", 1), ("double2", 2), ("double2", 3)])
@pytest.mark.parametrize("logNi,BS,n,split", [(8, 4, 16, 0), (10, 1, 8, 1), (7, 8, 8, 0)])
def test_compact_checksum_table_flavour(dtype, ck, logNi, BS, n, split):
    # `_h` / `_h2` kernels read one reduced-precision cotangent per element instead of a complex
    # entry (kept in registers, or read again per tile): same decisions on the reference cadence,
    # clean data stays clean, and the decisions equal the oracle model fed the compact vector
    ntiles, tbs, gap = 24, 4, 3
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=1, correct=1, split=split, ck=ck)
    groups = O.tile_groups(ntiles, tbs, gap)
    injs = O.reference_injections(groups, tbs, 100.0)
    assert c[1] == len(injs) == c[2] and c[3] == 0
    assert sorted(t for _, t in fl) == sorted(i.tile for i in injs)
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, logNi)
    ct = simlib.ctype_of(dtype)
    xt = x.reshape(ntiles, BS, -1)
    yt = O.fft_ref(xt).astype(ct)
    for inj in injs:
        yt[inj.tile, inj.s, :] += inj.mag
    dec = O.ft_launch_model(xt, yt, n, groups, dtype, O.dft_checksum_vector(1 << logNi, dtype, "compact"))
    assert sorted(d.tile for d in dec if d.detected) == sorted(t for _, t in fl)
    sp, x, y, c, fl = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=0, correct=1, split=split, ck=ck)
    assert c[1] == 0 and not fl and O.rel_l2(y, O.fft_ref(x)) < O.tolerance(dtype, logNi)
    clean = O.ft_launch_model(xt, O.fft_ref(xt).astype(ct), n, groups, dtype,
                              O.dft_checksum_vector(1 << logNi, dtype, "compact"))
    # the table's rounding leaves a residual well under the rule the flavour is used with
    assert max(abs(d.delta) / (1000.0 + abs(d.mag)) for d in clean) < (2e-4 if dtype == "float2" else 1e-7)


@pytest.mark.parametrize("dtype,logNi,BS,n,split,pf,ck", [("float2", 8, 4, 16, 0, 0, 0), ("double2", 10, 1, 8, 1, 0, 0),
                                                          ("float2", 9, 2, 8, 0, 0, 1), ("float2", 10, 1, 8, 1, 0, 3),
                                                          ("double2", 7, 8, 8, 0, 0, 2)])
@pytest.mark.parametrize("tbs,part_len,ntiles,gap", [(8, 4, 37, 3), (5, 2, 23, 2), (32, 4, 100, 2), (6, 1, 13, 1)])
def test_groups_shared_by_several_blocks(dtype, logNi, BS, n, split, pf, ck, tbs, part_len, ntiles, gap):
    """A checksum group walked by several blocks (each leaves its threads' running sums in the
    group's slots, the block with the last ticket decides): same groups, same flagged tiles, same
    counters and the same corrected output as one block per group, on the reference cadence, on
    clean data and with a ragged last group.  (Kernels that prefetch their next tile keep whole
    groups: the library does not share theirs.)"""
    for inj_mode in (1, 0):
        one = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=inj_mode, correct=1, split=split, pf=pf, ck=ck)
        many = run_ft(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=inj_mode, correct=1, split=split, pf=pf, ck=ck, part_len=part_len)
        assert many[3] == one[3]                       # checked, detected, corrected, uncorrectable
        assert sorted(many[4]) == sorted(one[4])       # flagged (launch, tile) pairs
        assert np.array_equal(many[2], one[2])         # recomputed tiles are bit-identical
        if inj_mode == 1:
            assert one[3][1] > 0                        # the cadence raises detections (long groups may miss some)


# ---- thread-level verification (`_tt` kernels) ----

def run_tl(dtype, logNi, BS, n, ntiles, thread_bs, tb_gap, inj_mode, correct, inj_every=1, inj_tile=0, inj_s=0, inj_m=0,
           mag=100.0, seed=0, split=0, threshold=1e-3, smoothing=1000.0):
    sp = KernelSpec(KernelKey(dtype, "row1", logNi, BS, n, 3, split))
    N = 1 << logNi
    bs = ntiles * BS
    x = rnd((bs, N), seed).astype(simlib.ctype_of(dtype))
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = ntiles, bs, thread_bs, tb_gap
    st = simlib.FtState(ka)
    ka.ft.launch, ka.ft.correct = 0, correct
    ka.ft.inj_mode, ka.ft.inj_every, ka.ft.inj_tile, ka.ft.inj_s, ka.ft.inj_m, ka.ft.inj_mag = \
        inj_mode, inj_every, inj_tile, inj_s, inj_m, mag
    ka.ft.err_smoothing, ka.ft.err_threshold = smoothing, threshold
    grid = (ntiles + thread_bs - 1) // thread_bs
    y = simlib.run_sim(sp, x, bs * N, ka, grid, simlib.twiddle_table(N, dtype)).reshape(bs, N)
    return sp, x, y, st


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("logNi,BS,n,split", [(8, 4, 16, 0), (7, 8, 8, 0), (10, 1, 8, 1), (5, 16, 8, 0), (3, 64, 8, 0), (13, 1, 32, 1)])
def test_thread_level_verification(dtype, logNi, BS, n, split):
    """Every thread checks the register-level DFTs of each pass against the checksum vectors of
    their radix; a tile that a thread objects to is recomputed before it is stored.  Clean data
    raises nothing; the reference cadence (100 on register 0 of thread 0 of one tile per block,
    after the input sums) is caught in exactly the injected tiles, as the oracle's model of the
    scheme says, and the stored result is bit-identical to an undisturbed run."""
    ntiles, tbs, gap = (24, 4, 3) if logNi < 13 else (6, 2, 2)
    sp, x, y0, st = run_tl(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=0, correct=1, split=split)
    assert st.checked == ntiles and st.detected == 0 and not st.pairs()
    assert O.rel_l2(y0, O.fft_ref(x)) < O.tolerance(dtype, logNi)
    sp, x, y, st = run_tl(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=1, correct=1, split=split)
    groups = O.tile_groups(ntiles, tbs, gap)
    injs = O.reference_injections(groups, tbs, 100.0)
    flagged, verdicts, quiet = O.thread_level_model(x.reshape(ntiles, BS, -1), n, dtype, injs)
    assert sorted(np.nonzero(flagged)[0]) == sorted(i.tile for i in injs)          # the model catches every injection
    assert quiet < 0.1 * 1e-3 and all(v.ratio > 10 * 1e-3 for v in verdicts)       # and nothing sits near the rule
    assert st.detected == len(injs) and sorted(t for _, t in st.pairs()) == sorted(i.tile for i in injs)
    assert np.array_equal(y, y0)
    # detect only: the flagged tile is stored as computed, every output of the hit sub-FFT off by the magnitude
    sp, x, y, st = run_tl(dtype, logNi, BS, n, ntiles, tbs, gap, inj_mode=1, correct=0, split=split)
    assert st.detected == len(injs)
    err = np.abs(y - y0).reshape(ntiles, BS, -1)
    for inj in injs:
        assert np.allclose(err[inj.tile, 0], 100.0, rtol=1e-3)
    assert err[[t for t in range(ntiles) if t not in {i.tile for i in injs}]].max() == 0


def test_thread_level_host_chosen_element_and_threshold():
    # mode 2: one tile, sub-FFT 2, element 11 (register 0 of thread 11); the objecting thread is the model's
    ntiles, tbs, gap = 20, 5, 2
    sp, x, y, st = run_tl("float2", 8, 4, 16, ntiles, tbs, gap, inj_mode=2, correct=1, inj_every=1000, inj_tile=13,
                          inj_s=2, inj_m=11, mag=100.0)
    assert st.detected == 1 and st.pairs() == [(0, 13)]
    flagged, verdicts, quiet = O.thread_level_model(x.reshape(ntiles, 4, -1), 16, "float2", [O.Injection(13, 2, 11, 100.0)])
    assert [(v.tile, v.s, v.q, v.thread) for v in verdicts] == [(13, 2, 0, 11)]
    assert O.rel_l2(y, O.fft_ref(x)) < O.tolerance("float2", 8)
    # an error far below the rule stays (model and kernel agree that nobody objects)
    sp, x, y, st = run_tl("float2", 8, 4, 16, ntiles, tbs, gap, inj_mode=2, correct=1, inj_every=1000, inj_tile=13,
                          inj_s=2, inj_m=11, mag=0.05)
    flagged, verdicts, quiet = O.thread_level_model(x.reshape(ntiles, 4, -1), 16, "float2", [O.Injection(13, 2, 11, 0.05)])
    assert not flagged.any() and quiet < 0.5e-3 and st.detected == 0


@pytest.mark.parametrize("dtype,logNi,BS,n,log_ncols", [("double2", 7, 16, 8, 8), ("float2", 8, 16, 16, 6)])
def test_thread_level_column_kernel(dtype, logNi, BS, n, log_ncols):
    sp = KernelSpec(KernelKey(dtype, "col", logNi, BS, n, 3))
    Ni, ncols, outer = 1 << logNi, 1 << log_ncols, 3
    x = rnd((outer, Ni, ncols), 5)
    ref = np.fft.fft(x.astype(simlib.ctype_of(dtype)).astype(np.complex128), axis=1)
    k = np.arange(Ni)[:, None]
    col = np.arange(ncols)[None, :]
    ref = ref * np.exp(-2j * np.pi * ((k * col) % (Ni * ncols)) / (Ni * ncols))
    lo_bits, hi, lo = simlib.split_tables(logNi + log_ncols, dtype)
    for inj_tile, want in ((7, [(0, 7)]), (1 << 40, [])):
        ka = simlib.KArgs()
        ka.ntiles = outer * ncols // BS
        ka.thread_bs, ka.tb_gap, ka.log_ncols = 3, 2, log_ncols
        ka.tw_lo_bits = lo_bits
        st = _ft_args(ka, ka.ntiles, 1, inj_tile, 100.0)
        y = simlib.run_sim(sp, x, x.size, ka, (ka.ntiles + 2) // 3, simlib.twiddle_table(Ni, dtype), hi, lo).reshape(outer, Ni, ncols)
        assert st.checked == ka.ntiles and st.pairs() == want and st.detected == len(want)
        assert O.rel_l2(y, ref) < O.tolerance(dtype, logNi)


@pytest.mark.parametrize("dtype,logA,BS,n,logQ,logC", [("double2", 8, 8, 8, 0, 4), ("float2", 8, 16, 16, 3, 4)])
def test_thread_level_transposing_kernel(dtype, logA, BS, n, logQ, logC):
    sp = KernelSpec(KernelKey(dtype, "rowT", logA, BS, n, 3))
    A, Q, Cc = 1 << logA, 1 << logQ, 1 << logC
    bs = 2
    x = rnd((bs, Cc, Q, A), 7)
    xc = x.astype(simlib.ctype_of(dtype)).astype(np.complex128)
    ref = np.transpose(np.fft.fft(xc, axis=3), (0, 3, 2, 1))
    ntiles = bs * Q * Cc // BS
    for inj_tile, want in ((ntiles - 1, [(0, ntiles - 1)]), (1 << 40, [])):
        ka = simlib.KArgs()
        ka.ntiles = ntiles
        ka.thread_bs, ka.tb_gap = 2, 3
        ka.logQ, ka.logC, ka.logN = logQ, logC, logA + logQ + logC
        st = _ft_args(ka, ka.ntiles, 1, inj_tile, 100.0)
        y = simlib.run_sim(sp, x, x.size, ka, (ntiles + 1) // 2, simlib.twiddle_table(A, dtype)).reshape(bs, A, Q, Cc)
        assert st.checked == ntiles and st.pairs() == want and st.detected == len(want)
        assert O.rel_l2(y, ref) < O.tolerance(dtype, logA)
