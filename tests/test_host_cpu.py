"""CPU-side checks of the product: the C-ABI library loads and exports every
declared symbol, the host table builders agree with the oracle, the plan CSVs
are well formed.  No compute call is made (there is no GPU here)."""
import ctypes
import os
import re

import numpy as np
import pytest

import turbofft_amd
from oracle import turbofft_oracle as O
from turbofft_amd.codegen import plan as P
from turbofft_amd.codegen.fft_codegen import KernelSpec, collect_keys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.skipif(not os.path.exists(turbofft_amd.LIB_PATH),
                                reason="libturbofft_hip.so not built (python turbofft_amd/build.py)")


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "turbofft.h")).read()
    names = set(re.findall(r"\b(turbofft_[a-z_0-9]+)\s*\(", hdr))
    assert {"turbofft_plan_create", "turbofft_exec", "turbofft_exec_host", "turbofft_main",
            "turbofft_get_ft_counters", "turbofft_set_injection"} <= names
    L = ctypes.CDLL(turbofft_amd.LIB_PATH)
    for n in sorted(names):
        assert hasattr(L, n), f"{n} declared in include/turbofft.h but not exported"


def test_registry_has_every_kernel_of_the_builtin_plans():
    have = set(turbofft_amd.kernel_names())
    for dtype in ("float2", "double2"):
        rows = P.load_plan_csv(os.path.join(ROOT, "turbofft_amd", "param", "gfx950", f"param_{dtype}.csv"))
        ft_rows = list(rows)          # fault-tolerant plans: same rows unless param_<T>_ft.csv replaces one
        for r in P.load_plan_csv(os.path.join(ROOT, "turbofft_amd", "param", "gfx950", f"param_{dtype}_ft.csv")):
            assert rows[r.logN].launches > 0
            ft_rows[r.logN] = r
        for key in collect_keys(rows, dtype, [0], inverse=True) + collect_keys(ft_rows, dtype, [1, 2]):
            assert key.name in have
        # the small-batch rows: two launches of narrow tiles, column 21 = largest batch served
        import dataclasses
        small = P.load_plan_csv(os.path.join(ROOT, "turbofft_amd", "param", "gfx950", f"param_{dtype}_small.csv"))
        assert small and all(r.launches == 2 and r.tiles >= 1 and rows[r.logN].launches in (1, 2) for r in small)
        for key in collect_keys([dataclasses.replace(r, tiles=0) for r in small], dtype, [0]):
            assert key.name in have


@pytest.mark.parametrize("dtype", ["float2", "double2"])
def test_builtin_rows_match_csv_and_are_consistent(dtype):
    rows = P.load_plan_csv(os.path.join(ROOT, "turbofft_amd", "param", "gfx950", f"param_{dtype}.csv"))
    assert len(rows) == 30                               # the reference's tables end at 2^25 (fp32) / 2^29 (fp64)
    for logN in range(1, 30):
        r = turbofft_amd.builtin_plan_row(dtype, logN)
        p = P.PlanRow.from_list(r)                       # the 11 reference columns
        full = rows[logN]                                # ... plus this build's optional flags
        assert (p.logN, p.launches, p.logNi, p.BS, p.n) == (full.logN, full.launches, full.logNi, full.BS, full.n)
        assert p.logN == logN and sum(p.logNi) == logN
        for i, k in enumerate(P.kernels_for_row(full, dtype, 0) + P.kernels_for_row(full, dtype, 1)):
            sp = KernelSpec(k)
            assert sp.threads % 64 == 0 and sp.threads <= 1024
            assert sp.lds_bytes <= 160 * 1024
    with pytest.raises(turbofft_amd.TurboFFTError):
        turbofft_amd.builtin_plan_row(dtype, 40)


def test_optional_plan_columns():
    """Columns beyond the reference's 11: per-launch split / prefetch / cross-lane flags,
    tiles per block, per-launch wavefronts per SIMD, per-launch tile access policy.
    Shorter rows mean zeros."""
    from turbofft_amd.codegen.fft_codegen import generate_source
    r = P.PlanRow.from_list([19, 2, 9, 10, 0, 32, 16, 0, 32, 32, 0, 1, 1, 0, 0, 0, 0, 0, 0, 0, 8, 4, 3])
    assert (r.split, r.pf, r.xl, r.tiles, r.wv) == ((1, 1), (0, 0), (0, 0), 8, (4, 3))
    plain = P.kernels_for_row(r, "float2", 0)
    assert [k.name for k in plain] == ["tfft_f32_col_N9_b32_n32_s_w4", "tfft_f32_rowT_N10_b16_n32_s_w3"]
    # the register budget hint and the cross-lane pass belong to the plain kernels only
    assert [k.name for k in P.kernels_for_row(r, "float2", 1)] == ["tfft_f32_col_N9_b32_n32_s_ft", "tfft_f32_rowT_N10_b16_n32_s_ft"]
    src = generate_source([KernelSpec(plain[0])], False)
    assert "amdgpu_waves_per_eu(4, 4)" in src
    # columns 25-27: non-temporal tile loads (1), stores (2) or both (3), for both flavours
    r = P.PlanRow.from_list([19, 2, 9, 10, 0, 32, 16, 0, 32, 32, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 3, 2])
    assert r.nt == (3, 2)
    assert [k.name for k in P.kernels_for_row(r, "float2", 0)] == ["tfft_f32_col_N9_b32_n32_t3", "tfft_f32_rowT_N10_b16_n32_t2"]
    assert [k.name for k in P.kernels_for_row(r, "float2", 1)] == ["tfft_f32_col_N9_b32_n32_t3_ft", "tfft_f32_rowT_N10_b16_n32_t2_ft"]
    src = generate_source([KernelSpec(P.kernels_for_row(r, "float2", 0)[1])], False)
    assert "GLDG(" in src and "GSTGN(" in src and "GLDGN(" not in src and "GSTG(" not in src
    # +4 in the same columns: the wave raises its priority while it issues its tile loads
    # (plain single-launch kernels; the fault-tolerant flavour of the row drops the bit)
    r = P.PlanRow.from_list([12, 1, 12, 0, 0, 1, 0, 0, 16, 0, 0] + [0] * 13 + [7])
    assert [k.name for k in P.kernels_for_row(r, "float2", 0)] == ["tfft_f32_row1_N12_b1_n16_t7"]
    assert [k.name for k in P.kernels_for_row(r, "float2", 1)] == ["tfft_f32_row1_N12_b1_n16_t3_ft"]
    src = generate_source([KernelSpec(P.kernels_for_row(r, "float2", 0)[0])], False)
    assert src.index("TFFT_WAVE_PRIO(3);") < src.index("GLDUN(") < src.index("TFFT_WAVE_PRIO(0);") < src.index("cadd(")
    assert "TFFT_WAVE_PRIO" not in generate_source([KernelSpec(P.kernels_for_row(r, "float2", 1)[0])], False)
    with pytest.raises(ValueError):
        P.PlanRow.from_list([13, 1, 13, 0, 0, 1, 0, 0, 32, 0, 0] + [0] * 13 + [8])
    # columns 28-30: tiles per XCD, a launch parameter (no kernel depends on it)
    r = P.PlanRow.from_list([20, 2, 10, 10, 0, 16, 16, 0, 32, 32, 0] + [0] * 16 + [8, 32])
    assert r.xc == (8, 32)
    assert [k.name for k in P.kernels_for_row(r, "float2", 0)] == ["tfft_f32_col_N10_b16_n32", "tfft_f32_rowT_N10_b16_n32"]
    # inverse plans: component-swapping flavours of the first and the last launch, plain only
    r3 = P.PlanRow.from_list([24, 3, 8, 8, 8, 32, 16, 32, 32, 32, 32])
    assert [k.name for k in P.kernels_for_row(r3, "float2", 0, inverse=True)] == \
        ["tfft_f32_col_N8_b32_n32_i", "tfft_f32_col_N8_b16_n32", "tfft_f32_rowT_N8_b32_n32_i"]
    with pytest.raises(ValueError):
        P.kernels_for_row(r3, "float2", 1, inverse=True)
    fwd = generate_source([KernelSpec(P.kernels_for_row(r3, "float2", 0)[0])], False)
    inv = generate_source([KernelSpec(P.kernels_for_row(r3, "float2", 0, inverse=True)[0])], False)
    assert "cswap(" not in fwd and inv.count("cswap(") == 32
    short = P.PlanRow.from_list([13, 1, 13, 0, 0, 1, 0, 0, 32, 0, 0])
    assert (short.split, short.tiles, short.wv) == ((0,), 0, (0,))
    assert "amdgpu_waves_per_eu" not in generate_source([KernelSpec(P.kernels_for_row(short, "float2", 0)[0])], False)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
def test_twiddle_table_matches_oracle(dtype):
    a = turbofft_amd.twiddle_table(1 << 12, dtype)
    b = O.twiddle_table(1 << 12, dtype)
    assert a.dtype == b.dtype and a.shape == b.shape
    assert np.max(np.abs(a - b)) <= (1e-7 if dtype == "float2" else 1e-15)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("N", [2, 4, 8, 128, 1024, 8192])
def test_checksum_vector_exact_matches_oracle(dtype, N):
    a = turbofft_amd.checksum_vector(N, dtype, "exact")
    b = O.dft_checksum_vector(N, dtype, "exact")
    scale = np.max(np.abs(b))
    assert np.max(np.abs(a - b)) <= scale * (1e-6 if dtype == "float2" else 1e-12)


@pytest.mark.parametrize("dtype", ["float2", "double2"])
@pytest.mark.parametrize("N", [256, 1024])
def test_checksum_vector_reference_mode_pinned_by_multiprecision(dtype, N):
    # the library's mode 1 against abft.h:21-61 evaluated in multiprecision (tests/mp_checksum.py),
    # not against the numpy restatement of the same lines
    import mp_checksum as M
    rows = [0, 1, 2, N // 3, N // 2, N - 1]
    want = M.checksum_rows(N, rows)
    a = turbofft_amd.checksum_vector(N, dtype, "reference")
    tol = 2e-5 if dtype == "float2" else 1e-12
    assert max(abs(complex(a[i]) - want[i]) for i in rows) < tol
    for v in ("unrounded_angle", "float_two_pi"):
        bad = M.checksum_rows(N, rows, v)
        assert max(abs(bad[i] - want[i]) for i in rows) > 5 * tol
    # and bit-for-bit the oracle's table in fp64, where libm and numpy share cos/sin of a double
    b = O.dft_checksum_vector(N, dtype, "reference")
    assert np.max(np.abs(a - b)) <= np.max(np.abs(b)) * (2e-5 if dtype == "float2" else 1e-13)


def test_bad_arguments_are_reported_not_fatal():
    L = turbofft_amd.lib()
    buf = np.zeros(64, dtype=np.complex128)
    assert L.turbofft_build_twiddle_table(0, 3, buf.ctypes.data) != 0
    assert b"power of two" in L.turbofft_last_error()
    assert L.turbofft_build_twiddle_table(0, 8, None) != 0
    assert b"null output" in L.turbofft_last_error()
    assert L.turbofft_build_checksum_vector(1, 1, 0, buf.ctypes.data) != 0
    assert b"power of two" in L.turbofft_last_error()
    assert L.turbofft_build_checksum_vector(7, 8, 0, buf.ctypes.data) != 0
    assert b"datatype" in L.turbofft_last_error()
    assert L.turbofft_exec(None, None, None, 1, None) != 0
    # plan creation needs a device: here it must fail with a message, not crash
    import torch
    if not torch.cuda.is_available():
        with pytest.raises(turbofft_amd.TurboFFTError):
            turbofft_amd.TurboFFT(10, "double2")


def test_vendor_side_by_side_rejects_bad_arguments_before_touching_a_device():
    L = turbofft_amd.lib()
    ms = ctypes.c_float(0)
    assert L.turbofft_vendor_exec(10, 0, None, None, 4, None) != 0
    assert b"null buffer" in L.turbofft_last_error()
    assert L.turbofft_vendor_time(10, 0, None, None, 4, 1, 10, None, ctypes.byref(ms)) != 0
    assert b"bad argument" in L.turbofft_last_error()
    assert turbofft_amd.vendor_available() in (True, False)      # opening the library needs no device
    assert L.turbofft_offline_checksums(10, 0, None, None, 4, None, None, None) != 0
    assert b"bad argument" in L.turbofft_last_error()
    assert L.turbofft_offline_ft_time(10, 0, None, None, 4, 1, 10, None, ctypes.byref(ms), None) != 0
    assert b"bad argument" in L.turbofft_last_error()


def test_cli_help_and_bad_flag():
    import subprocess
    r = subprocess.run([turbofft_amd.CLI_PATH, "--help"], capture_output=True, text=True)
    assert r.returncode == 1 and "--if_bench" in r.stdout and "--thread_bs" in r.stdout
    r = subprocess.run([turbofft_amd.CLI_PATH, "--bogus", "1"], capture_output=True, text=True)
    assert r.returncode == 1 and "Invalid or incomplete argument: --bogus" in r.stderr
