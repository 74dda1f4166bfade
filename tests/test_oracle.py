"""Pins for the CPU oracle.  None of these retype the oracle's formulas: each
check is a closed form, an invariant or a brute-force computation that a
plausible mistake (wrong sign, dropped twiddle, transposed digit) fails."""
import math

import numpy as np
import pytest

from oracle import turbofft_oracle as O


def rng_cplx(shape, seed=0, normal=False):
    rng = np.random.default_rng(seed)
    if normal:
        return rng.standard_normal(shape) + 1j * rng.standard_normal(shape)
    return rng.uniform(-1, 1, shape) + 1j * rng.uniform(-1, 1, shape)


# ---------------- fft_ref -------------------------------------------------
@pytest.mark.parametrize("N", [2, 8, 64, 256])
def test_fft_ref_vs_bruteforce(N):
    x = rng_cplx((3, N), 1)
    assert O.rel_l2(O.fft_ref(x), O.dft_bruteforce(x)) < 1e-13


def test_fft_ref_closed_forms():
    N = 128
    k = np.arange(N)
    for m in (0, 1, 5, 127):
        d = np.zeros(N, complex); d[m] = 1
        # impulse at m -> W^{mk}; a sign error in the exponent fails for m=1
        assert np.allclose(O.fft_ref(d), np.exp(-2j * np.pi * m * k / N), atol=1e-13)
    assert np.allclose(O.fft_ref(np.ones(N)), N * (k == 0), atol=1e-12)
    tone = np.exp(2j * np.pi * 7 * k / N)
    assert np.allclose(O.fft_ref(tone), N * (k == 7), atol=1e-10)
    x, y = rng_cplx(N, 2), rng_cplx(N, 3)
    assert np.allclose(O.fft_ref(2 * x - 3j * y), 2 * O.fft_ref(x) - 3j * O.fft_ref(y), atol=1e-11)
    assert math.isclose(np.sum(np.abs(O.fft_ref(x)) ** 2), N * np.sum(np.abs(x) ** 2), rel_tol=1e-12)


# ---------------- tables --------------------------------------------------
def test_twiddle_table_layout():
    N = 64
    tw = O.twiddle_table(N, "double2")
    assert tw.shape == (2 * N - 1,)
    assert tw[0] == 1                                   # c=1
    assert np.allclose(tw[1:3], [1, -1])                # c=2: W_2^0, W_2^1
    assert np.allclose(tw[3:7], [1, -1j, -1, 1j])       # c=4: forward sign
    for c in (8, 64):
        assert np.allclose(tw[c - 1:2 * c - 1], np.exp(-2j * np.pi * np.arange(c) / c), atol=1e-15)
    assert O.twiddle_table(N, "float2").dtype == np.complex64


def test_checksum_vector_hand_values():
    s = O.SQRT3_2_LITERAL
    # N=2: c[0]=r0+r1, c[1]=r0-r1
    c2 = O.dft_checksum_vector(2, "double2")
    assert np.allclose(c2, [0.5 - 1j * s, 1.5 + 1j * s], atol=1e-15)
    # N=4: r = [r0,r1,r2,r0]; W_4 = -i
    r0, r1, r2 = 1, -0.5 - 1j * s, -0.5 + 1j * s
    c4 = [r0 + r1 + r2 + r0,
          r0 + (-1j) * r1 + (-1) * r2 + (1j) * r0,
          r0 - r1 + r2 - r0,
          r0 + (1j) * r1 - r2 + (-1j) * r0]
    assert np.allclose(O.dft_checksum_vector(4, "double2"), c4, atol=1e-14)


@pytest.mark.parametrize("N", [8, 128, 1024])
def test_checksum_vector_closed_form(N):
    c = O.dft_checksum_vector(N, "double2")
    ref = O.checksum_closed_form(N)
    # literal sqrt(3)/2 is float-rounded (1.55e-8 off): agreement ~1e-8*N
    assert np.max(np.abs(c - ref)) < 4e-8 * N
    # and it is the DFT-matrix column sum  W^T r
    W = np.exp(-2j * np.pi * (np.outer(np.arange(N), np.arange(N)) % N) / N)
    assert np.allclose(W @ O.checksum_r()[np.arange(N) % 3], c, atol=1e-9)


def test_checksum_reference_mode_matches_exact_for_small_N():
    # the float-rounded angle is harmless while 2*pi*i*j is small
    for N in (2, 4, 16):
        a = O.dft_checksum_vector(N, "double2", "reference")
        b = O.dft_checksum_vector(N, "double2", "exact")
        assert np.max(np.abs(a - b)) < 1e-5


REF_ROWS = {256: [0, 1, 2, 85, 128, 255], 1024: [0, 1, 3, 341, 512, 1023], 8192: [1, 2731, 8191]}
WRONG_READINGS = ["unrounded_angle", "float_two_pi", "r_shifted", "positive_angle", "exact_sqrt3"]


@pytest.mark.parametrize("N", [256, 1024, 8192])
def test_checksum_reference_mode_pinned_by_multiprecision(N):
    """abft.h:21-61 evaluated independently: float32 angle from struct, cos/sin and the sum
    over j in 40-digit arithmetic.  The fp64 variant of the oracle must agree to accumulation
    rounding (~1e-15*sqrt(N)), the fp32 variant to the rounding of N float additions; every
    wrong reading of the source lines (angle not rounded to float, 2*pi rounded first, r
    started at the wrong residue, +i exponent, exact sqrt(3)/2 instead of the float literal,
    and -- where i*j exceeds 2^24 -- the index product rounded first) is off by orders of
    magnitude more and must be told apart."""
    import mp_checksum as M
    rows = REF_ROWS[N]
    want = M.checksum_rows(N, rows)
    o64 = O.dft_checksum_vector(N, "double2", "reference")
    o32 = O.dft_checksum_vector(N, "float2", "reference")
    tol64, tol32 = 4e-15 * N ** 0.5 * 4, 2e-5
    assert max(abs(o64[i] - want[i]) for i in rows) < tol64
    assert max(abs(complex(o32[i]) - want[i]) for i in rows) < tol32
    wrong = WRONG_READINGS + (["float_index_product"] if N == 8192 else [])
    for v in wrong:
        bad = M.checksum_rows(N, rows, v)
        d = max(abs(bad[i] - want[i]) for i in rows)
        assert d > 100 * tol64, (v, d)
        if v != "exact_sqrt3":            # 1.5e-8 per term: below the fp32 accumulation noise
            assert d > 5 * tol32, (v, d)
    # the known quirk of the reference table: visibly wrong against the exact vector
    b = O.dft_checksum_vector(N, "double2", "exact")
    assert 1e-6 < np.max(np.abs(o64 - b)) / np.max(np.abs(b)) < 1e-1


@pytest.mark.parametrize("N", [64, 128, 1024, 8192])
def test_compact_checksum_form_matches_the_exact_vector(N):
    # kappa (1 - i cot(pi (m/N + 1/3))) is the geometric-series closed form of c_N for the exact
    # cube root; against the exact vector (built from the float-rounded sqrt(3)/2 by an FFT) it
    # may differ by float16 rounding of the cotangent only.  A wrong kappa for odd log2 N, a sign
    # error in the cotangent or a shifted angle is off by O(1) relative.
    c = O.dft_checksum_vector(N, "double2", "exact")
    h = O.dft_checksum_vector(N, "float2", "compact").astype(np.complex128)
    t = O.compact_cotangents(N).astype(np.float64)
    assert np.max(np.abs(h - c) / np.abs(c)) < 6e-4 + 2e-8 * N
    h32 = O.dft_checksum_vector(N, "double2", "compact").astype(np.complex128)      # single-precision cotangents
    h16 = O.dft_checksum_vector(N, "float2", "compact").astype(np.complex128)       # half-precision cotangents
    assert np.max(np.abs(h32 - c) / np.abs(c)) < 1e-7 + 2e-8 * N
    # the cotangent alone carries the rounding: unrounded, the form is exact up to what the
    # literal's 1.55e-8 contributes (its own pole, of height 1.55e-8 * N / pi, sits at m = N/3)
    a = np.pi * (3.0 * np.arange(N) + N) / (3.0 * N)
    full = O.compact_kappa(N) * (1 - 1j * np.cos(a) / np.sin(a))
    assert np.max(np.abs(full - c) / np.abs(c)) < 2e-8 * N
    assert np.max(np.abs(full - c)) / np.max(np.abs(c)) < 1e-7
    assert np.all(np.isfinite(t)) and np.max(np.abs(t)) < (3 * N / np.pi) * (1 + 2 ** -10)       # largest entry, float16-rounded
    # device layout: thread x, register pair q -> elements x + Tr*2q and x + Tr*(2q+1)
    n = 8
    w = O.compact_table_words(N, n)
    Tr = N // n
    bits = O.compact_cotangents(N).view(np.uint16)
    for x, q in ((0, 0), (1, 0), (Tr - 1, n // 2 - 1), (3 % Tr, 1)):
        assert w[x + Tr * q] & 0xffff == bits[x + Tr * 2 * q] and w[x + Tr * q] >> 16 == bits[x + Tr * (2 * q + 1)]


def test_checksum_table_offsets():
    t = O.dft_checksum_table("float2", max_log=6)
    assert t.shape == (32768,)
    for N in (2, 8, 64):
        assert np.allclose(t[N - 2:2 * N - 2], O.dft_checksum_vector(N, "float2"))


# ---------------- kernel algebra ------------------------------------------
def test_radix_passes():
    assert O.radix_passes(1024, 8) == [8, 8, 8, 2]
    assert O.radix_passes(8192, 32) == [32, 32, 8]
    assert O.radix_passes(128, 8) == [8, 8, 2]
    assert O.radix_passes(256, 16) == [16, 16]
    assert O.radix_passes(4, 4) == [4]
    assert O.radix_passes(2, 2) == [2]


@pytest.mark.parametrize("Ni,n", [(2, 2), (8, 8), (16, 4), (64, 8), (128, 8), (1024, 8), (1024, 16), (4096, 16), (8192, 32)])
def test_block_fft_matches_dft(Ni, n):
    x = rng_cplx((2, Ni), Ni)
    y = O.block_fft(x, n, "double2")
    assert O.rel_l2(y, O.fft_ref(x)) < 1e-13 * max(1, math.log2(Ni))
    y32 = O.block_fft(x, n, "float2")
    assert y32.dtype == np.complex64
    assert O.rel_l2(y32, O.fft_ref(x)) < 1e-5 * max(1, math.log2(Ni))


PLANS = [
    [6, 2, 3, 3, 0, 2, 2, 0, 4, 4, 0],          # 8 x 8
    [6, 3, 2, 2, 2, 2, 2, 2, 2, 4, 4],          # 4 x 4 x 4
    [7, 2, 3, 4, 0, 4, 2, 0, 8, 4, 0],          # unequal digits: transposed operand fails
    [9, 3, 2, 3, 4, 4, 2, 2, 4, 8, 4],          # all digits different
    [15, 2, 7, 8, 0, 16, 8, 0, 8, 8, 0],        # benchmark configuration 3 row
]


@pytest.mark.parametrize("row", PLANS)
def test_plan_fft_matches_dft(row):
    p = O.PlanRow.from_list(row)
    bs = 2 if p.logN > 10 else 4
    x = rng_cplx((bs, p.N), p.logN, normal=True)
    y = O.plan_fft(x, p, "double2")
    assert O.rel_l2(y, O.fft_ref(x)) < 1e-13 * p.logN
    y32 = O.plan_fft(x, p, "float2")
    assert O.rel_l2(y32, O.fft_ref(x)) < 1e-5 * p.logN


def test_plan_fft_impulse_lands_in_natural_order():
    # an impulse at n0 must give exactly W^{n0 k} at output index k: catches a
    # wrong output digit order (kb + B ka vs ka + A kb)
    p = O.PlanRow.from_list([9, 3, 2, 3, 4, 4, 2, 2, 4, 8, 4])
    N = p.N
    for n0 in (1, 16, 17 + 64):
        x = np.zeros((1, N), complex); x[0, n0] = 1
        y = O.plan_fft(x, p, "double2")[0]
        assert np.allclose(y, np.exp(-2j * np.pi * ((n0 * np.arange(N)) % N) / N), atol=1e-12)


# ---------------- geometry ------------------------------------------------
@pytest.mark.parametrize("row", PLANS)
def test_gather_is_a_partition(row):
    p = O.PlanRow.from_list(row)
    bs = 2
    ids = np.arange(bs * p.N).reshape(bs, p.N)
    for g in O.launch_geometry(p, bs):
        t = g.gather(ids)
        assert t.shape == (g.ntiles, g.BS, g.Ni)
        assert np.array_equal(np.sort(t.ravel()), ids.ravel())


def test_gather_col_addresses():
    # L=3 launch 1: element m of column a of outer block kc sits at a + A*m + A*B*kc
    p = O.PlanRow.from_list([9, 3, 2, 3, 4, 4, 2, 2, 4, 8, 4])
    C, B, A = 4, 8, 16
    ids = np.arange(p.N).reshape(1, p.N)
    g = O.launch_geometry(p, 1)[1]
    t = g.gather(ids)
    tiles_per_outer = A // g.BS
    for tile in (0, 3, tiles_per_outer * 2 + 1):
        kc, ct = divmod(tile, tiles_per_outer)
        for s in range(g.BS):
            a = ct * g.BS + s
            assert np.array_equal(t[tile, s], a + A * np.arange(B) + A * B * kc)
    # final launch: row (kb, kc) at A*(kb + B*kc); tile = BS adjacent kc
    g2 = O.launch_geometry(p, 1)[2]
    t2 = g2.gather(ids)
    tile = 5
    kct, kb = tile % (C // g2.BS), (tile // (C // g2.BS)) % B
    for s in range(g2.BS):
        kc = kct * g2.BS + s
        assert np.array_equal(t2[tile, s], A * (kb + B * kc) + np.arange(A))


@pytest.mark.parametrize("ntiles,tbs,gap", [(64, 4, 4), (64, 4, 3), (100, 8, 5), (7, 3, 2), (16, 1, 4), (33, 32, 256)])
def test_tile_groups_cover_once(ntiles, tbs, gap):
    groups = O.tile_groups(ntiles, tbs, gap)
    flat = [t for g in groups for t in g]
    assert sorted(flat) == list(range(ntiles))
    assert all(len(g) <= tbs for g in groups)


def test_tile_groups_reference_formula():
    # divisible case must equal the literal reference loop (fft_codegen.py:218,260-261)
    ntiles, tbs, gap = 96, 4, 5
    grid = ntiles // tbs
    groups = O.tile_groups(ntiles, tbs, gap)
    for bx in range(grid):
        delta = grid % gap if (bx // gap) == (grid // gap) else gap
        bid = (bx // gap) * gap * tbs + bx % gap
        tiles = []
        cnt = 0
        while cnt < tbs and bid < ntiles:
            tiles.append(bid); bid += delta; cnt += 1
        assert groups[bx] == tiles


# ---------------- FT model ------------------------------------------------
def _ft_setup(dtype, Ni=256, BS=4, n=8, ntiles=32, seed=0):
    x = rng_cplx((ntiles, BS, Ni), seed).astype(O._ctype(dtype))
    y = O.fft_ref(x).astype(O._ctype(dtype))
    c = O.dft_checksum_vector(Ni, dtype)
    return x, y, c


@pytest.mark.parametrize("dtype", ["float2", "double2"])
def test_ft_clean_data_no_detection(dtype):
    x, y, c = _ft_setup(dtype)
    groups = O.tile_groups(32, 4, 3)
    dec = O.ft_launch_model(x, y, 8, groups, dtype, c)
    assert not any(d.detected for d in dec)
    scale = 1e-3 if dtype == "float2" else 1e-11
    assert all(abs(d.delta) < scale * (1 + d.mag) for d in dec)


@pytest.mark.parametrize("Ni,expect", [(256, -100.0), (128, -100.0 * (1 - 0.5 - O.SQRT3_2_LITERAL))])
def test_injected_delta_closed_form(Ni, expect):
    # Ni = 1 mod 3 (even log2): the r-sum over k<Ni is r0 -> -mag;
    # Ni = 2 mod 3 (odd log2): r0 + r1 -> -mag*(0.5 - 0.866) = +0.366*mag
    assert math.isclose(O.injected_delta_closed_form(Ni, 100.0), expect, rel_tol=1e-6)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("Ni", [128, 256])
def test_ft_detects_and_locates_injection(dtype, Ni):
    x, y, c = _ft_setup(dtype, Ni=Ni)
    groups = O.tile_groups(32, 4, 3)
    injs = O.reference_injections(groups, 4, 100.0)
    assert len(injs) == len(groups)
    y = y.copy()
    for inj in injs:
        y[inj.tile, inj.s, :] += inj.mag           # error on x[0] shifts every output
    dec = O.ft_launch_model(x, y, 8, groups, dtype, c)
    for bx, (d, g) in enumerate(zip(dec, groups)):
        assert d.detected
        assert d.k == bx % 4 + 1                    # the two-sided checksum locates the tile
        assert d.tile == g[bx % 4]
        assert math.isclose(d.delta, O.injected_delta_closed_form(Ni, 100.0), rel_tol=2e-3)
        assert math.isclose(abs(d.delta2 / d.delta), d.k, rel_tol=1e-3)


def test_ft_plan_model_multi_launch():
    p = O.PlanRow.from_list([9, 3, 2, 3, 4, 4, 2, 2, 4, 8, 4])
    x = rng_cplx((4, p.N), 9)
    geoms = O.launch_geometry(p, 4)
    groups = O.tile_groups(geoms[2].ntiles, 2, 4)
    injs = O.reference_injections(groups, 2, 100.0)
    dec, out = O.ft_plan_model(x, p, "double2", 2, [4, 4, 4], injs)
    assert not any(d.detected for d in dec[0]) and not any(d.detected for d in dec[1])
    assert all(d.detected and d.k == bx % 2 + 1 for bx, d in enumerate(dec[2]))
    assert O.rel_l2(out, O.fft_ref(x)) < 1e-12


def test_compare_data():
    a = np.array([1 + 1j, 2 + 2j, 3 + 3j])
    assert O.compare_data(a, a) == -1
    b = a.copy(); b[1] = 2 + 2.01j
    assert O.compare_data(b, a) == 1
    b = a.copy(); b[2] = complex(np.nan, 3)
    assert O.compare_data(b, a) == 2


def test_metrics_formulas():
    # 2^28 points fp32 in 3.120 ms -> the reference's published 5592 GFLOPS, 1376.5 GB/s
    assert math.isclose(O.gflops(1 << 13, 1 << 15, 3.120), 5592.0, rel_tol=1e-3)
    assert math.isclose(O.algorithmic_gbs(1 << 13, 1 << 15, 3.120, "float2"), 1376.5, rel_tol=1e-3)


def test_rule_saturates_for_long_subffts():
    """An input error e moves delta by e*(re c[m] + im c[m]) and mag by about
    |e|*Ni/sqrt(n) (every output of the sub-FFT is off by |e|): the ratio the reference rule
    tests tends to a constant as e grows -- above the 1e-3 threshold for a 256-point
    sub-FFT, below it for a 2048-point one, which therefore cannot flag such an error."""
    rng = np.random.default_rng(5)
    seen = {}
    for Ni, n in ((256, 16), (2048, 16)):
        x = (rng.uniform(-1, 1, (4, 1, Ni)) + 1j * rng.uniform(-1, 1, (4, 1, Ni)))
        cv = O.dft_checksum_vector(Ni, "double2")
        ratios = []
        for mag in (1e9, 1e12):
            y = O.fft_ref(x)
            y[2, 0, :] += mag * np.exp(-2j * np.pi * 5 * np.arange(Ni) / Ni)      # error on x[5] of tile 2
            d = O.ft_launch_model(x, y, n, [[0, 1, 2, 3]], "double2", cv)[0]
            ratios.append(abs(d.delta) / (1000.0 + abs(d.mag)))
            seen[(Ni, mag)] = d.detected
        assert abs(ratios[0] / ratios[1] - 1) < 1e-3          # saturated: independent of the magnitude
    assert seen[(256, 1e12)] and not seen[(2048, 1e12)]


# ---------------- delayed batch correction ----------------------------------
@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("Ni,n,BS,T", [(64, 8, 4, 4), (256, 16, 2, 8), (1024, 8, 1, 3)])
def test_delayed_batch_correction_restores_the_clean_transform(dtype, Ni, n, BS, T):
    # linearity pins it: whatever the error on tile k looks like (one output, a whole
    # sub-FFT shifted as after an input-side upset, dense noise), y_k + FFT(sum x) - sum y is
    # the clean transform of x_k.  A flipped sign doubles the error, a dropped sum leaves
    # garbage of the size of the data, a wrong k patches a clean tile: all fail the bar.
    x = rng_cplx((T, BS, Ni), Ni + T)
    clean = O.fft_ref(x)
    tol = O.tolerance(dtype, int(math.log2(Ni))) * math.sqrt(T) * 2
    rng = np.random.default_rng(5)
    for k in range(T):
        for shape in ("one", "row", "dense"):
            y = clean.copy()
            if shape == "one":
                y[k, BS - 1, 3] += 100.0
            elif shape == "row":
                y[k, 0, :] += 100.0                     # x[k,0,0] += 100 after the input checksum
            else:
                y[k] += rng.standard_normal((BS, Ni)) * 50
            fixed = O.delayed_batch_correction(x, y, k, n, dtype)
            assert O.rel_l2(fixed, clean[k]) < tol, (k, shape)
            assert O.rel_l2(y[k], clean[k]) > 100 * tol
    # the patch goes to the located tile only: patching another tile moves the error there
    y = clean.copy()
    y[1, 0, :] += 100.0
    wrong = O.delayed_batch_correction(x, y, 0, n, dtype)
    assert O.rel_l2(wrong, clean[0]) > 100 * tol


# ---- thread-level verification model ----

@pytest.mark.parametrize("R", [2, 4, 8, 16, 32, 64])
def test_thread_level_vectors_satisfy_the_checksum_identity(R):
    # sum_o y_o r[o%3] == sum_i x_i c_R[i] for y = DFT_R(x), with the DFT taken by brute force: a
    # transposed index, a conjugated root or r used on the input side breaks this by O(|x|)
    rng = np.random.default_rng(R)
    x = rng.normal(size=(5, R)) + 1j * rng.normal(size=(5, R))
    y = O.dft_bruteforce(x)
    cR, rR = O.thread_level_vectors(R, "double2")
    assert np.allclose((y * rR).sum(axis=1), (x * cR).sum(axis=1), rtol=0, atol=1e-12 * R)
    assert np.allclose(rR, O.checksum_r()[np.arange(R) % 3])
    # and the input-side vector is the block-level one of the same length
    assert np.allclose(cR, O.dft_checksum_vector(R, "double2"), atol=1e-13 * R) if R >= 2 else True


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("logNi,BS,n", [(10, 2, 16), (7, 8, 8), (13, 1, 32), (4, 4, 4), (9, 2, 8)])
def test_thread_level_model_clean_and_injected(dtype, logNi, BS, n):
    Ni = 1 << logNi
    rng = np.random.default_rng(logNi)
    x = rng.uniform(-1, 1, (5, BS, Ni)) + 1j * rng.uniform(-1, 1, (5, BS, Ni))
    flagged, verdicts, quiet = O.thread_level_model(x, n, dtype)
    assert not flagged.any() and not verdicts
    assert quiet < (1e-6 if dtype == "float2" else 1e-14)          # rounding only
    # 100 on re of element m of one sub-FFT after the first pass's input sums moves every output of
    # that thread's first register-level DFT by 100: exactly one thread of pass 0 objects, by the
    # closed-form shift -100 * sum_{o<R}(re r + im r) of its radix; later passes see consistent data
    m = min(Ni // n - 1, 3)
    inj = O.Injection(2, BS - 1, m, 100.0)
    flagged, verdicts, quiet = O.thread_level_model(x, n, dtype, [inj])
    assert list(np.nonzero(flagged)[0]) == [2]
    assert [(v.tile, v.s, v.q, v.thread) for v in verdicts] == [(2, BS - 1, 0, m)]
    R0 = O.radix_passes(Ni, n)[0]
    # (sign: the model's delta is in - out, the block-level one in + (-out): the same quantity)
    assert abs(verdicts[0].delta - O.injected_delta_closed_form(R0, 100.0)) < (1e-3 if dtype == "float2" else 1e-10)
    assert quiet < (1e-6 if dtype == "float2" else 1e-14)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
def test_thread_level_model_sees_a_fault_in_any_pass(dtype):
    # a fault on one output of one register-level DFT, in each pass in turn: the owner thread of that
    # pass objects (x = rest mod Ni/n), nobody else, and the shift is the fault weighed with r[o % 3]
    logNi, BS, n = 10, 2, 8
    Ni, Tr = 1 << logNi, (1 << logNi) // n
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (3, BS, Ni)) + 1j * rng.uniform(-1, 1, (3, BS, Ni))
    passes = O.radix_passes(Ni, n)
    r = O.checksum_r()
    for q, R in enumerate(passes):
        rest, o, val = 37 % (Ni // R), R - 1, 5.0 - 2.0j
        flagged, verdicts, quiet = O.thread_level_model(x, n, dtype, out_faults=[(1, 1, q, rest, o, val)])
        assert list(np.nonzero(flagged)[0]) == [1]
        assert [(v.tile, v.s, v.q, v.thread) for v in verdicts] == [(1, 1, q, rest % Tr)]
        w = val * r[o % 3]
        assert abs(verdicts[0].delta + (w.real + w.imag)) < (1e-3 if dtype == "float2" else 1e-10)


def test_thread_level_plan_model_covers_every_launch():
    row = O.PlanRow.from_list([12, 2, 6, 6, 0, 16, 16, 0, 8, 8, 0])
    rng = np.random.default_rng(8)
    x = (rng.uniform(-1, 1, (4, 1 << 12)) + 1j * rng.uniform(-1, 1, (4, 1 << 12))).astype(np.complex128)
    res, out = O.thread_level_plan_model(x, row, "double2", [O.Injection(5, 3, 2, 100.0)], inj_launch=0)
    assert list(np.nonzero(res[0][0])[0]) == [5] and not res[1][0].any()
    assert O.rel_l2(out, O.fft_ref(x)) < O.tolerance("double2", 12)
    res, out = O.thread_level_plan_model(x, row, "double2", [O.Injection(9, 0, 0, 100.0)])
    assert not res[0][0].any() and list(np.nonzero(res[1][0])[0]) == [9]
