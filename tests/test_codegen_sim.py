"""CPU lock-step runs of the generated kernels against the fp64 DFT.

These tests execute the *same generated phase text* that hipcc compiles for
gfx950, one barrier-separated phase at a time for all threads of a block,
with bounds checks on every global, table and LDS access.
"""
import math

import numpy as np
import pytest

from oracle import turbofft_oracle as O
from tests import simlib
from turbofft_amd.codegen.fft_codegen import KernelSpec
from turbofft_amd.codegen.plan import KernelKey


def rnd(shape, seed):
    rng = np.random.default_rng(seed)
    return rng.uniform(-1, 1, shape) + 1j * rng.uniform(-1, 1, shape)


ROW1 = [("double2", 10, 1, 8), ("float2", 10, 1, 16), ("float2", 13, 1, 32), ("double2", 7, 4, 8),
        ("float2", 7, 8, 8), ("float2", 3, 64, 4), ("double2", 1, 128, 2), ("float2", 4, 16, 4),
        ("double2", 12, 1, 16), ("float2", 8, 4, 16), ("float2", 6, 32, 32),
        # one whole transform per thread: fp32 kernels of this shape move two elements per access
        ("float2", 1, 256, 2), ("float2", 2, 64, 4), ("float2", 3, 128, 8), ("float2", 4, 64, 16)]


@pytest.mark.parametrize("dtype,logNi,BS,n", ROW1)
@pytest.mark.parametrize("thread_bs", [1, 3])
def test_row1(dtype, logNi, BS, n, thread_bs):
    sp = KernelSpec(KernelKey(dtype, "row1", logNi, BS, n, 0))
    N = 1 << logNi
    bs = BS * 5 + (BS // 2)           # ragged last tile when BS > 1
    x = rnd((bs, N), logNi)
    ka = simlib.KArgs()
    ka.ntiles = (bs + BS - 1) // BS
    ka.nrows = bs
    ka.thread_bs = thread_bs
    ka.tb_gap = 2
    grid = (ka.ntiles + thread_bs - 1) // thread_bs
    y = simlib.run_sim(sp, x, bs * N, ka, grid, simlib.twiddle_table(N, dtype)).reshape(bs, N)
    assert O.rel_l2(y, O.fft_ref(x.astype(simlib.ctype_of(dtype)))) < O.tolerance(dtype, logNi)


COL = [("double2", 7, 16, 8, 8), ("float2", 8, 16, 16, 6), ("float2", 3, 64, 4, 7), ("double2", 5, 8, 4, 3)]


@pytest.mark.parametrize("dtype,logNi,BS,n,log_ncols", COL)
def test_col(dtype, logNi, BS, n, log_ncols):
    sp = KernelSpec(KernelKey(dtype, "col", logNi, BS, n, 0))
    Ni, ncols, outer = 1 << logNi, 1 << log_ncols, 3
    x = rnd((outer, Ni, ncols), 5)
    ka = simlib.KArgs()
    ka.ntiles = outer * ncols // BS
    ka.thread_bs = 2
    ka.tb_gap = 3
    ka.log_ncols = log_ncols
    lo_bits, hi, lo = simlib.split_tables(logNi + log_ncols, dtype)
    ka.tw_lo_bits = lo_bits
    grid = (ka.ntiles + 1) // 2
    y = simlib.run_sim(sp, x, x.size, ka, grid, simlib.twiddle_table(Ni, dtype), hi, lo).reshape(outer, Ni, ncols)
    xc = x.astype(simlib.ctype_of(dtype))
    ref = np.fft.fft(xc.astype(np.complex128), axis=1)
    k = np.arange(Ni)[:, None]
    col = np.arange(ncols)[None, :]
    ref = ref * np.exp(-2j * np.pi * ((k * col) % (Ni * ncols)) / (Ni * ncols))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, logNi)


ROWT = [("double2", 8, 8, 8, 0, 4), ("float2", 8, 16, 16, 3, 4), ("float2", 7, 16, 8, 0, 5), ("double2", 4, 16, 4, 2, 4),
        ("float2", 5, 64, 32, 1, 6)]


@pytest.mark.parametrize("dtype,logA,BS,n,logQ,logC", ROWT)
def test_rowT(dtype, logA, BS, n, logQ, logC):
    sp = KernelSpec(KernelKey(dtype, "rowT", logA, BS, n, 0))
    A, Q, Cc = 1 << logA, 1 << logQ, 1 << logC
    bs = 2
    N = A * Q * Cc
    x = rnd((bs, Cc, Q, A), 7)                     # rows (kc, kb) of length A
    ka = simlib.KArgs()
    ka.ntiles = bs * Q * Cc // BS
    ka.thread_bs = 1
    ka.tb_gap = 4
    ka.logQ, ka.logC, ka.logN = logQ, logC, logA + logQ + logC
    y = simlib.run_sim(sp, x, x.size, ka, ka.ntiles, simlib.twiddle_table(A, dtype)).reshape(bs, A, Q, Cc)
    xc = x.astype(simlib.ctype_of(dtype)).astype(np.complex128)
    ref = np.transpose(np.fft.fft(xc, axis=3), (0, 3, 2, 1))          # [b, ka, kb, kc]
    assert O.rel_l2(y, ref) < O.tolerance(dtype, logA)


@pytest.mark.parametrize("chunk,bs", [(1, 37), (2, 40), (3, 100), (64, 20)])
def test_xcd_renumbering_is_a_bijection(chunk, bs):
    # the XCD-aware block renumbering must still visit every tile exactly once
    sp = KernelSpec(KernelKey("float2", "row1", 9, 1, 8, 0))
    N = 512
    x = rnd((bs, N), 11)
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap, ka.xcd_chunk = bs, bs, 1, 4, chunk
    y = simlib.run_sim(sp, x, bs * N, ka, bs, simlib.twiddle_table(N, "float2")).reshape(bs, N)
    assert not np.isnan(y).any()
    assert O.rel_l2(y, O.fft_ref(x.astype(np.complex64))) < O.tolerance("float2", 9)


SPLIT = [("row1", "float2", 10, 1, 16), ("row1", "double2", 9, 2, 8), ("row1", "float2", 13, 1, 32), ("row1", "float2", 7, 8, 8)]


@pytest.mark.parametrize("kind,dtype,logNi,BS,n", SPLIT)
def test_split_exchange_row1(kind, dtype, logNi, BS, n):
    # re and im go through a half-size LDS buffer in two rounds
    sp = KernelSpec(KernelKey(dtype, kind, logNi, BS, n, 0, 1))
    full = KernelSpec(KernelKey(dtype, kind, logNi, BS, n, 0, 0))
    assert sp.lds_bytes <= full.lds_bytes // 2 + 4096
    N = 1 << logNi
    bs = BS * 3
    x = rnd((bs, N), logNi + 50)
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = bs // BS, bs, 2, 2
    y = simlib.run_sim(sp, x, bs * N, ka, (ka.ntiles + 1) // 2, simlib.twiddle_table(N, dtype)).reshape(bs, N)
    assert O.rel_l2(y, O.fft_ref(x.astype(simlib.ctype_of(dtype)))) < O.tolerance(dtype, logNi)


def test_split_exchange_col_and_rowT():
    dtype = "float2"
    sp = KernelSpec(KernelKey(dtype, "col", 8, 16, 16, 0, 1))
    Ni, ncols, outer, log_ncols = 256, 64, 2, 6
    x = rnd((outer, Ni, ncols), 5)
    ka = simlib.KArgs()
    ka.ntiles, ka.thread_bs, ka.tb_gap, ka.log_ncols = outer * ncols // 16, 1, 3, log_ncols
    lo_bits, hi, lo = simlib.split_tables(8 + log_ncols, dtype)
    ka.tw_lo_bits = lo_bits
    y = simlib.run_sim(sp, x, x.size, ka, ka.ntiles, simlib.twiddle_table(Ni, dtype), hi, lo).reshape(outer, Ni, ncols)
    ref = np.fft.fft(x.astype(np.complex64).astype(np.complex128), axis=1)
    ref = ref * np.exp(-2j * np.pi * ((np.arange(Ni)[:, None] * np.arange(ncols)[None, :]) % (Ni * ncols)) / (Ni * ncols))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, 8)
    sp = KernelSpec(KernelKey(dtype, "rowT", 8, 16, 16, 0, 1))
    A, Q, Cc = 256, 2, 16
    x = rnd((1, Cc, Q, A), 7)
    ka = simlib.KArgs()
    ka.ntiles, ka.thread_bs, ka.tb_gap = Q * Cc // 16, 1, 4
    ka.logQ, ka.logC, ka.logN = 1, 4, 13
    y = simlib.run_sim(sp, x, x.size, ka, ka.ntiles, simlib.twiddle_table(A, dtype)).reshape(1, A, Q, Cc)
    ref = np.transpose(np.fft.fft(x.astype(np.complex64).astype(np.complex128), axis=3), (0, 3, 2, 1))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, 8)


PF = [("row1", "float2", 10, 1, 16, 0), ("row1", "double2", 7, 8, 8, 0), ("row1", "float2", 12, 1, 16, 1)]


@pytest.mark.parametrize("kind,dtype,logNi,BS,n,split", PF)
@pytest.mark.parametrize("tbs", [1, 4])
@pytest.mark.parametrize("pf", [1, 3])
def test_prefetch_row1(kind, dtype, logNi, BS, n, split, tbs, pf):
    # pf = 1: the whole next tile is fetched ahead; pf = 3: only a thread's first three elements,
    # issued at the start of the tile's last pass
    sp = KernelSpec(KernelKey(dtype, kind, logNi, BS, n, 0, split, pf))
    N = 1 << logNi
    bs = BS * 9 + BS // 2
    x = rnd((bs, N), logNi + 70)
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = (bs + BS - 1) // BS, bs, tbs, 3
    grid = (ka.ntiles + tbs - 1) // tbs
    y = simlib.run_sim(sp, x, bs * N, ka, grid, simlib.twiddle_table(N, dtype)).reshape(bs, N)
    assert O.rel_l2(y, O.fft_ref(x.astype(simlib.ctype_of(dtype)))) < O.tolerance(dtype, logNi)


@pytest.mark.parametrize("pf", [1, 3])
def test_prefetch_col_and_rowT(pf):
    dtype = "float2"
    sp = KernelSpec(KernelKey(dtype, "col", 8, 16, 16, 0, 0, pf))
    Ni, ncols, outer, log_ncols = 256, 64, 3, 6
    x = rnd((outer, Ni, ncols), 5)
    ka = simlib.KArgs()
    ka.ntiles, ka.thread_bs, ka.tb_gap, ka.log_ncols = outer * ncols // 16, 5, 2, log_ncols
    lo_bits, hi, lo = simlib.split_tables(8 + log_ncols, dtype)
    ka.tw_lo_bits = lo_bits
    y = simlib.run_sim(sp, x, x.size, ka, (ka.ntiles + 4) // 5, simlib.twiddle_table(Ni, dtype), hi, lo).reshape(outer, Ni, ncols)
    ref = np.fft.fft(x.astype(np.complex64).astype(np.complex128), axis=1)
    ref = ref * np.exp(-2j * np.pi * ((np.arange(Ni)[:, None] * np.arange(ncols)[None, :]) % (Ni * ncols)) / (Ni * ncols))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, 8)
    sp = KernelSpec(KernelKey(dtype, "rowT", 8, 16, 16, 0, 0, pf))
    A, Q, Cc = 256, 2, 32
    x = rnd((2, Cc, Q, A), 7)
    ka = simlib.KArgs()
    ka.ntiles, ka.thread_bs, ka.tb_gap = 2 * Q * Cc // 16, 3, 2
    ka.logQ, ka.logC, ka.logN = 1, 5, 14
    y = simlib.run_sim(sp, x, x.size, ka, (ka.ntiles + 2) // 3, simlib.twiddle_table(A, dtype)).reshape(2, A, Q, Cc)
    ref = np.transpose(np.fft.fft(x.astype(np.complex64).astype(np.complex128), axis=3), (0, 3, 2, 1))
    assert O.rel_l2(y, ref) < O.tolerance(dtype, 8)


XL = [("float2", 7, 8, 8), ("double2", 10, 1, 8), ("float2", 8, 4, 8), ("float2", 10, 2, 16), ("float2", 11, 1, 16),
      ("double2", 11, 2, 8), ("float2", 9, 8, 4)]


@pytest.mark.parametrize("dtype,logNi,BS,n", XL)
def test_cross_lane_last_pass(dtype, logNi, BS, n):
    # the final radix-2/4/8 pass runs across adjacent lanes (DPP / ds_swizzle on the GPU)
    sp = KernelSpec(KernelKey(dtype, "row1", logNi, BS, n, 0, 0, 0, 1))
    assert sp.xl and sp.RL in (2, 4, 8) and len(sp.pads) == sp.npass - 2
    N = 1 << logNi
    bs = BS * 5 + BS // 2
    x = rnd((bs, N), logNi + 90)
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = (bs + BS - 1) // BS, bs, 2, 3
    y = simlib.run_sim(sp, x, bs * N, ka, (ka.ntiles + 1) // 2, simlib.twiddle_table(N, dtype)).reshape(bs, N)
    ref = O.fft_ref(x.astype(simlib.ctype_of(dtype)))
    for b in range(bs):
        assert O.rel_l2(y[b], ref[b]) < O.tolerance(dtype, logNi)


@pytest.mark.parametrize("dtype,logNi,BS,n,xl", [("float2", 10, 1, 16, 0), ("double2", 7, 4, 8, 0), ("double2", 11, 1, 8, 1)])
def test_inverse_flavour_of_a_single_launch_kernel(dtype, logNi, BS, n, xl):
    # the `_i` flavour exchanges re and im after the load and before the store, which turns the
    # forward kernel into the unnormalised inverse transform
    sp = KernelSpec(KernelKey(dtype, "row1", logNi, BS, n, 0, 0, 0, xl, 0, 0, 1))
    assert sp.name.endswith("_i")
    N = 1 << logNi
    bs = BS * 3 + BS // 2
    x = rnd((bs, N), logNi + 300)
    ka = simlib.KArgs()
    ka.ntiles, ka.nrows, ka.thread_bs, ka.tb_gap = (bs + BS - 1) // BS, bs, 1, 1
    y = simlib.run_sim(sp, x, bs * N, ka, ka.ntiles, simlib.twiddle_table(N, dtype)).reshape(bs, N)
    ref = np.fft.ifft(x.astype(simlib.ctype_of(dtype)).astype(np.complex128), axis=1) * N
    assert O.rel_l2(y, ref) < O.tolerance(dtype, logNi)


@pytest.mark.parametrize("pad", [(5, 0), (4, 1), (6, 2), (3, 0), (-1, 0)])
def test_padded_lds_index_of_base_plus_offset(pad):
    # The generator writes the padded index of base + off as (padded index of base) + constant
    # when off is a multiple of the padding period, and in full otherwise: both forms must name
    # the address phys(base + off) = (base + off) + (((base + off) >> ps) << pl).
    from turbofft_amd.codegen.fft_codegen import KernelEmitter
    em = KernelEmitter.__new__(KernelEmitter)          # the two methods use no state
    ps, pl = pad
    phys = (lambda a: a) if ps < 0 else (lambda a: a + ((a >> ps) << pl))
    rng = np.random.default_rng(ps * 10 + pl + 100)
    for off in [0, 1, 7, 32, 96, 256, 1024, 1056, 4096, 31 * 1024, 8 * 4096 + 64]:
        expr = em.lds_index_at("b0", "b0p", off, pad)
        for b0 in [0, 1, 31, 32, 33, 1023] + [int(v) for v in rng.integers(0, 1 << 15, 20)]:
            got = eval(expr.replace("u", ""), {"b0": b0, "b0p": phys(b0)})      # drop the C suffix of unsigned literals
            assert got == phys(b0 + off), (pad, off, b0, expr)
