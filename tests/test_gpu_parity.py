"""GPU parity: the gfx950 kernels, called through the C ABI, against the fp64
numpy DFT on the same seeded inputs.  Tolerances are the ones the task states:
rel-L2 <= 1e-5*log2N (fp32), <= 1e-13*log2N (fp64)."""
import os
import subprocess

import numpy as np
import pytest

import turbofft_amd
from oracle import turbofft_oracle as O

pytestmark = pytest.mark.gpu


def _torch():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    return torch


def cdtype(dt):
    return np.complex64 if dt == "float2" else np.complex128


def make(bs, N, dt, seed=0, normal=False):
    rng = np.random.default_rng(seed)
    if normal:
        x = rng.standard_normal((bs, N)) + 1j * rng.standard_normal((bs, N))
    else:
        x = rng.uniform(-1, 1, (bs, N)) + 1j * rng.uniform(-1, 1, (bs, N))
    return x.astype(cdtype(dt))


def gpu_fft(plan, x):
    torch = _torch()
    print(f"[case] logN={plan.logN} dt={plan.datatype} bs={x.shape[0]} launches={plan.launches} "
          f"Ni={plan.logNi} BS={plan.BS} n={plan.n}", flush=True)
    y = plan.fft(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    return y.cpu().numpy()


SHAPES_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "turbofft_amd", "param", "gfx950")


def test_config1_fp64_2p10_batch16():
    # benchmark configuration 1: fp64, N=2^10, batch 16, U[-1,1) seed 0, single launch n=8 -- with the
    # plan shape the configuration names, and with the built-in row for this size
    x = make(16, 1024, "double2", 0)
    shaped = turbofft_amd.TurboFFT(10, "double2", param_csv=os.path.join(SHAPES_DIR, "reference_shapes_double2.csv"))
    assert shaped.launches == 1 and shaped.n == [8]
    for plan in (shaped, turbofft_amd.TurboFFT(10, "double2")):
        y = gpu_fft(plan, x)
        assert O.rel_l2(y, O.fft_ref(x)) <= 1e-13 * 10


def test_config3_and_config4_plan_shapes():
    # benchmark configuration 3 (fp64 2^15, two launches 7/8 with BS 16/8, standard normal input) and
    # config 4 (fp32 2^24, three launches 8/8/8 with BS 16): the named plan shapes on a few
    # transforms; the full 2^28-point sizes of these plans are covered by the sweeps below
    rng = np.random.default_rng(3)
    plan = turbofft_amd.TurboFFT(15, "double2", param_csv=os.path.join(SHAPES_DIR, "reference_shapes_double2.csv"))
    assert (plan.launches, plan.logNi, plan.BS) == (2, [7, 8], [16, 8])
    x = (rng.standard_normal((5, 1 << 15)) + 1j * rng.standard_normal((5, 1 << 15))).astype(np.complex128)
    assert O.rel_l2(gpu_fft(plan, x), O.fft_ref(x)) <= O.tolerance("double2", 15)
    plan = turbofft_amd.TurboFFT(24, "float2", param_csv=os.path.join(SHAPES_DIR, "reference_shapes_float2.csv"))
    assert (plan.launches, plan.logNi, plan.BS) == (3, [8, 8, 8], [16, 16, 16])
    x = make(2, 1 << 24, "float2", 4)
    assert O.rel_l2(gpu_fft(plan, x), O.fft_ref(x)) <= O.tolerance("float2", 24)


@pytest.mark.parametrize("dt", ["float2", "double2"])
@pytest.mark.parametrize("logN", list(range(1, 14)))
def test_single_launch_sizes(dt, logN):
    plan = turbofft_amd.TurboFFT(logN, dt)
    BS = plan.BS[0] if plan.launches == 1 else 1
    bs = 3 * BS + max(1, BS // 2)              # ragged last tile
    x = make(bs, 1 << logN, dt, logN)
    y = gpu_fft(plan, x)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    # every transform individually (a wrong row in a tile must not hide in the norm)
    ref = O.fft_ref(x)
    for b in range(bs):
        assert O.rel_l2(y[b], ref[b]) <= O.tolerance(dt, logN)


@pytest.mark.parametrize("dt", ["float2", "double2"])
@pytest.mark.parametrize("logN", list(range(14, 25)))
def test_multi_launch_sizes(dt, logN):
    plan = turbofft_amd.TurboFFT(logN, dt)
    bs = 3 if logN <= 20 else 1
    x = make(bs, 1 << logN, dt, logN, normal=True)
    y = gpu_fft(plan, x)
    ref = O.fft_ref(x)
    for b in range(bs):
        assert O.rel_l2(y[b], ref[b]) <= O.tolerance(dt, logN)


@pytest.mark.parametrize("dt,logN", [("float2", 13), ("double2", 15), ("float2", 24), ("double2", 20)])
def test_closed_forms(dt, logN):
    # impulse at n0 -> W^{n0 k} in natural order; constant -> N delta_0
    N = 1 << logN
    plan = turbofft_amd.TurboFFT(logN, dt)
    n0 = 12345 % N
    x = np.zeros((2, N), cdtype(dt))
    x[0, n0] = 1
    x[1, :] = 1
    y = gpu_fft(plan, x)
    k = np.arange(N)
    ref0 = np.exp(-2j * np.pi * ((n0 * k) % N) / N)
    assert O.rel_l2(y[0], ref0) <= O.tolerance(dt, logN)
    ref1 = np.zeros(N, complex); ref1[0] = N
    assert np.max(np.abs(y[1] - ref1)) <= O.tolerance(dt, logN) * N


def test_thread_bs_does_not_change_results():
    x = make(64, 1 << 12, "float2", 3)
    a = gpu_fft(turbofft_amd.TurboFFT(12, "float2", thread_bs=1), x)
    b = gpu_fft(turbofft_amd.TurboFFT(12, "float2", thread_bs=5), x)
    assert np.array_equal(a, b)


def test_exec_host_matches_device_path():
    x = make(8, 1 << 15, "double2", 4)
    plan = turbofft_amd.TurboFFT(15, "double2")
    a = plan.fft_host(x)
    b = gpu_fft(plan, x)
    assert np.array_equal(a, b)
    assert O.rel_l2(a, O.fft_ref(x)) <= O.tolerance("double2", 15)


@pytest.mark.parametrize("dt,logN,bs,piece", [("float2", 10, 1000, 96), ("double2", 15, 11, 2), ("float2", 17, 7, 3),
                                              ("float2", 23, 3, 1), ("double2", 6, 5000, 4999)])
def test_exec_host_streams_the_batch_in_pieces(dt, logN, bs, piece, monkeypatch):
    """Host buffers larger than one piece go through three device slots on three streams; the
    result is that of the device path, bit for bit, for pageable and for page-locked buffers,
    with a ragged last piece and with more pieces than slots."""
    torch = _torch()
    x = make(bs, 1 << logN, dt, 40 + logN)
    plan = turbofft_amd.TurboFFT(logN, dt)
    want = gpu_fft(plan, x)
    monkeypatch.setenv("TURBOFFT_HOST_PIECE_BYTES", str(piece * x.shape[1] * x.itemsize))
    assert np.array_equal(plan.fft_host(x), want)
    tdt = torch.complex64 if dt == "float2" else torch.complex128
    xin = torch.empty(x.shape, dtype=tdt, pin_memory=True)
    xin.copy_(torch.from_numpy(x))
    out = torch.zeros(x.shape, dtype=tdt, pin_memory=True)
    for _ in range(2):                                   # the second call reuses nothing of the first
        plan.exec_host(xin.data_ptr(), out.data_ptr(), bs)
        assert np.array_equal(out.numpy(), want)
        out.zero_()
    # a fault-tolerant plan is transformed in one piece: its groups and flagged tiles refer to the whole batch
    if logN == 10:
        ft = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=4)
        assert np.array_equal(ft.fft_host(x), gpu_fft(ft, x))
        c = ft.ft_counters()
        assert c["checked"] == 2 * ft.grid(0, bs) and c["detected"] == 0      # two executions of the whole batch


def test_empty_batch_and_bad_shapes():
    torch = _torch()
    plan = turbofft_amd.TurboFFT(10, "float2")
    plan.exec(0, 0, 0)                                   # bs = 0 is a no-op
    with pytest.raises(ValueError):
        plan.fft(torch.zeros((2, 512), dtype=torch.complex64, device="cuda"))
    with pytest.raises(turbofft_amd.TurboFFTError):
        turbofft_amd.TurboFFT(30, "float2")              # no plan row


def test_input_is_not_modified():
    torch = _torch()
    x = make(4, 1 << 16, "float2", 5)
    xd = torch.from_numpy(x).cuda()
    plan = turbofft_amd.TurboFFT(16, "float2")
    plan.fft(xd)
    torch.cuda.synchronize()
    assert np.array_equal(xd.cpu().numpy(), x)


def test_config2_full_size_fp32_2p13():
    # benchmark configuration 2 at full size (2^28 points): numpy default_rng(0), uniform[-1,1) drawn in
    # fp64 and cast (re then im, per chunk of 1024 transforms); 64 batches spread over the set against
    # the fp64 oracle, plus Parseval over the whole set as a size-independent property
    torch = _torch()
    logN, bs = 13, 1 << 15
    N = 1 << logN
    plan = turbofft_amd.TurboFFT(logN, "float2")
    rng = np.random.default_rng(0)
    x = torch.empty((bs, N), dtype=torch.complex64, device="cuda")
    idx = sorted(set(range(0, bs, bs // 63)) | {bs - 1})[:64]
    keep = {}
    chunk = 1024
    for c0 in range(0, bs, chunk):
        part = (rng.uniform(-1, 1, (chunk, N)) + 1j * rng.uniform(-1, 1, (chunk, N))).astype(np.complex64)
        for i in idx:
            if c0 <= i < c0 + chunk:
                keep[i] = part[i - c0].copy()
        x[c0:c0 + chunk].copy_(torch.from_numpy(part))
    y = plan.fft(x)
    torch.cuda.synchronize()
    ys = y[idx].cpu().numpy()
    ref = O.fft_ref(np.stack([keep[i] for i in idx]))
    worst = max(O.rel_l2(ys[k], ref[k]) for k in range(len(idx)))
    print(f"config 2: {len(idx)} sampled transforms, worst rel-L2 {worst:.3e} (bar {O.tolerance('float2', logN):.1e})", flush=True)
    assert worst <= O.tolerance("float2", logN)
    # Parseval over the whole set: sum |X|^2 = N sum |x|^2
    ex = float((x.real.double() ** 2 + x.imag.double() ** 2).sum())
    ey = float((y.real.double() ** 2 + y.imag.double() ** 2).sum())
    assert abs(ey / (N * ex) - 1) < 1e-5
    plan.close()


def _full_size_check(torch, plan, dt, logN, bs, normal):
    """Sampled transforms against the oracle plus two size-independent properties of the
    whole batch: Parseval, and additivity fft(x + x') = fft(x) + fft(x') on a rolled copy."""
    N = 1 << logN
    rdt = torch.float32 if dt == "float2" else torch.float64
    g = torch.Generator(device="cuda").manual_seed(0)
    if normal:
        x = torch.randn((bs, N, 2), generator=g, device="cuda", dtype=rdt)
    else:
        x = torch.rand((bs, N, 2), generator=g, device="cuda", dtype=rdt) * 2 - 1
    x = torch.view_as_complex(x)
    y = plan.fft(x).clone()
    torch.cuda.synchronize()
    idx = sorted({0, 1, bs // 3, bs // 2, bs - 1})
    ref = O.fft_ref(x[idx].cpu().numpy())
    ys = y[idx].cpu().numpy()
    for i in range(len(idx)):
        assert O.rel_l2(ys[i], ref[i]) <= O.tolerance(dt, logN)
    ex = float((x.real.double() ** 2 + x.imag.double() ** 2).sum())
    ey = float((y.real.double() ** 2 + y.imag.double() ** 2).sum())
    assert abs(ey / (N * ex) - 1) < (1e-5 if dt == "float2" else 1e-12)
    x2 = torch.roll(x, 1, dims=0)                      # transform b of x2 is transform b-1 of x
    y2 = plan.fft(x + x2)
    torch.cuda.synchronize()
    d = y2 - (y + torch.roll(y, 1, dims=0))
    rel = float(d.abs().double().pow(2).sum().sqrt() / y2.abs().double().pow(2).sum().sqrt())
    assert rel <= 2 * O.tolerance(dt, logN)


def test_config3_full_size_fp64_2p15():
    # benchmark configuration 3 at full size: fp64, N=2^15, batch 2^13, standard normal input, two launches
    plan = turbofft_amd.TurboFFT(15, "double2")
    assert plan.launches == 2
    _full_size_check(_torch(), plan, "double2", 15, 1 << 13, normal=True)


def test_config4_full_size_fp32_2p24():
    # benchmark configuration 4 at full size: fp32, N=2^24, batch 16, three launches
    plan = turbofft_amd.TurboFFT(24, "float2")
    assert plan.launches == 3
    _full_size_check(_torch(), plan, "float2", 24, 16, normal=False)


def test_cli_verify_mode():
    for dt, logN, bs in ((1, 10, 16), (0, 13, 4), (1, 15, 2)):
        r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "0", "--if_verify", "1", "--logN", str(logN),
                            "--bs", str(bs), "--bs_end", str(bs), "--datatype", str(dt)],
                           capture_output=True, text=True, timeout=120)
        print(r.stdout, r.stderr, flush=True)
        assert r.returncode == 0
        assert "Compare begin." in r.stdout and "Compare finished." in r.stdout
        assert "Error detected" not in r.stdout
        assert f"turboFFT, {logN}, " in r.stdout


@pytest.mark.parametrize("dt,logN,bs", [("double2", 10, 16), ("float2", 13, 64), ("double2", 15, 8),
                                        ("float2", 20, 4), ("float2", 24, 1)])
def test_agrees_with_the_vendor_library(dt, logN, bs):
    # the reference's own check (main.cu:98-102): its result against the vendor library's on the
    # same device input.  Both are roundings of the same transform, so they differ by at most the
    # sum of their error bounds.
    torch = _torch()
    if not turbofft_amd.vendor_available():
        pytest.skip("libhipfft.so cannot be opened")
    N = 1 << logN
    x = torch.view_as_complex(torch.rand((bs, N, 2), generator=torch.Generator(device="cuda").manual_seed(logN),
                                         device="cuda", dtype=torch.float32 if dt == "float2" else torch.float64) * 2 - 1)
    plan = turbofft_amd.TurboFFT(logN, dt)
    ours = plan.fft(x).clone()
    theirs = turbofft_amd.vendor_fft(x)
    err = (torch.linalg.vector_norm(ours - theirs) / torch.linalg.vector_norm(theirs)).item()
    tol = 2 * (1e-5 if dt == "float2" else 1e-13) * logN
    print(f"{dt} logN={logN} bs={bs}: rel L2 difference to hipFFT {err:.3e} (tol {tol:.1e})", flush=True)
    assert err <= tol
    plan.close()


@pytest.mark.parametrize("dt,logN", [(dt, logN) for dt in ("float2", "double2") for logN in range(25, 30)])
def test_plans_of_2p25_and_beyond(dt, logN):
    # row 25, the largest the reference dispatches, and rows 26-29 (the reference's fp64 table lists them, param/A100/param_double2.csv:27-30; its
    # dispatch stops at 2^25): one transform, checked with closed forms that need no second
    # transform of that size -- a unit impulse at m gives W_N^(m k), the constant gives N at k = 0 --
    # plus linearity on random data against the vendor library where that is available.
    torch = _torch()
    N = 1 << logN
    rdt = torch.float32 if dt == "float2" else torch.float64
    cdt = torch.complex64 if dt == "float2" else torch.complex128
    eps = (1e-5 if dt == "float2" else 1e-13) * logN
    plan = turbofft_amd.TurboFFT(logN, dt)
    assert plan.launches == 3
    out = torch.empty(plan.out_elems(1), dtype=cdt, device="cuda")
    x = torch.zeros((1, N), dtype=cdt, device="cuda")
    m = (N // 3) | 1
    x[0, m] = 1.0
    y = plan.fft(x, out)
    k = torch.arange(N, device="cuda", dtype=torch.int64)
    ang = ((k * m) % N).to(torch.float64) * (-2.0 * np.pi / N)
    err = max((y[0].real.double() - torch.cos(ang)).abs().max().item(), (y[0].imag.double() - torch.sin(ang)).abs().max().item())
    print(f"{dt} 2^{logN}: impulse max abs error {err:.3e}", flush=True)
    assert err <= eps
    del ang, k
    x.fill_(1.0)
    y = plan.fft(x, out)
    assert abs(y[0, 0].real.item() - N) <= eps * N and abs(y[0, 0].imag.item()) <= eps * N
    y[0, 0] = 0
    assert y.abs().max().item() <= eps * N
    if turbofft_amd.vendor_available():
        del x
        x = torch.view_as_complex(torch.rand((1, N, 2), generator=torch.Generator(device="cuda").manual_seed(logN),
                                             device="cuda", dtype=rdt) * 2 - 1)
        ours = plan.fft(x, out)
        theirs = turbofft_amd.vendor_fft(x)
        theirs -= ours
        err = (torch.linalg.vector_norm(theirs) / torch.linalg.vector_norm(ours)).item()
        print(f"{dt} 2^{logN}: rel L2 difference to hipFFT {err:.3e}", flush=True)
        assert err <= 2 * eps
    plan.close()


@pytest.mark.parametrize("dt,logN,bs", [("float2", 5, 1000), ("double2", 10, 16), ("double2", 11, 7), ("float2", 13, 33),
                                        ("double2", 14, 4), ("float2", 17, 8), ("double2", 20, 2), ("float2", 24, 1)])
def test_inverse_transform(dt, logN, bs):
    # turbofft_exec_inverse: the unnormalised inverse (N * numpy's ifft) through component-swapping
    # flavours of the forward kernels; one-, two- and three-launch plans (2^11 fp64 is the
    # cross-lane kernel), then the round trip forward -> inverse = N * x
    torch = _torch()
    N = 1 << logN
    rng = np.random.default_rng(400 + logN)
    x = (rng.uniform(-1, 1, (bs, N)) + 1j * rng.uniform(-1, 1, (bs, N))).astype(cdtype(dt))
    xd = torch.from_numpy(x).cuda()
    plan = turbofft_amd.TurboFFT(logN, dt)
    y = plan.ifft(xd).cpu().numpy()
    ref = np.fft.ifft(x.astype(np.complex128), axis=1) * N
    err = O.rel_l2(y, ref)
    print(f"{dt} logN={logN} bs={bs} launches={plan.launches}: inverse rel L2 {err:.3e}", flush=True)
    assert err <= O.tolerance(dt, logN)
    back = plan.ifft(plan.fft(xd).clone()).cpu().numpy() / N
    assert O.rel_l2(back, x.astype(np.complex128)) <= 2 * O.tolerance(dt, logN)
    plan.close()


def test_inverse_transform_is_refused_where_it_was_not_built():
    torch = _torch()
    x = torch.zeros((4, 1024), dtype=torch.complex128, device="cuda")
    plan = turbofft_amd.TurboFFT(10, "double2", if_ft=1, thread_bs=2)
    with pytest.raises(turbofft_amd.TurboFFTError, match="inverse"):
        plan.ifft(x)
    plan.close()
    shapes = os.path.join(os.path.dirname(turbofft_amd.LIB_PATH), "param", "gfx950", "reference_shapes_double2.csv")
    plan = turbofft_amd.TurboFFT(10, "double2", param_csv=shapes)          # n = 8: forward kernel only
    with pytest.raises(turbofft_amd.TurboFFTError, match="inverse"):
        plan.ifft(x)
    plan.fft(x)
    plan.close()


def test_whole_transform_threads_take_any_buffer_alignment():
    # fp32 plans whose threads hold whole transforms (2 and 4 points in the built-in table) move
    # two elements per 128-bit access when a buffer is aligned to 16 bytes and one element per
    # access otherwise: all four combinations of aligned and odd-element buffers give the same bits
    torch = _torch()
    for logN in (1, 2):
        N = 1 << logN
        xh = make(1000, N, "float2", logN)
        x = torch.from_numpy(np.append(np.complex64(0), xh.reshape(-1))).cuda()   # data from element 1
        xa = x[1:].clone()                                                      # the same data, aligned
        plan = turbofft_amd.TurboFFT(logN, "float2")
        st = torch.cuda.current_stream().cuda_stream
        results = []
        for src in (xa.data_ptr(), x.data_ptr() + 8):
            for shift in (0, 1):
                out = torch.zeros(1000 * N + 2, dtype=torch.complex64, device="cuda")
                plan.exec(src, out.data_ptr() + 8 * shift, 1000, st)
                torch.cuda.synchronize()
                got = out.cpu().numpy()
                assert got[:shift].tolist() == [0] * shift and got[shift + 1000 * N:].tolist() == [0] * (2 - shift)
                results.append(got[shift:shift + 1000 * N].reshape(1000, N))
        assert O.rel_l2(results[0], O.fft_ref(xh)) <= O.tolerance("float2", logN)
        for r in results[1:]:
            assert np.array_equal(r.view(np.uint32), results[0].view(np.uint32))
        plan.close()


def test_tuned_tiles_per_block_shrink_with_the_batch():
    # fp32 2^15 walks 16 tiles per block in the built-in table, tuned with the device full: a
    # batch with fewer tiles than that per resident block slot gets a block per tile (or as many
    # tiles per block as leave one block per slot), and the result is the same transform
    torch = _torch()
    for logN, tiles in ((15, 16),):
        N = 1 << logN
        plan = turbofft_amd.TurboFFT(logN, "float2")
        slots = plan.tb_gap(0)
        assert plan.grid(0, 7) == 7 and plan.grid(0, slots) == slots
        assert plan.grid(0, 3 * slots) == slots
        assert plan.grid(0, tiles * slots * 2) == 2 * slots
        for bs in (7, 3 * slots + 5):
            xh = make(bs, N, "float2", logN + bs)
            y = plan.fft(torch.from_numpy(xh).cuda()).cpu().numpy()
            sel = np.unique(np.linspace(0, bs - 1, 9).astype(int))
            assert O.rel_l2(y[sel], O.fft_ref(xh[sel])) <= O.tolerance("float2", logN)
        plan.close()


@pytest.mark.parametrize("dt,logN,log_bs", [("float2", 13, 19), ("float2", 20, 11), ("double2", 17, 14)])
def test_data_sets_beyond_4_gib(dt, logN, log_bs):
    # 2^31 and 2^32 points (16 and 32 GiB in): element offsets pass 2^32, byte offsets 2^35.
    # Sampled transforms (first, last, around the middle, six seeded) against the oracle, and
    # Parseval over every transform of the batch
    torch = _torch()
    N, bs = 1 << logN, 1 << log_bs
    x = torch.empty((bs, N), dtype=torch.complex64 if dt == "float2" else torch.complex128, device="cuda")
    xr = torch.view_as_real(x)
    step = bs // 64
    g = torch.Generator(device="cuda").manual_seed(logN)
    for b0 in range(0, bs, step):       # in slices, to bound the temporaries
        xr[b0:b0 + step].uniform_(-1, 1, generator=g)
    plan = turbofft_amd.TurboFFT(logN, dt)
    out = torch.empty(plan.out_elems(bs), dtype=x.dtype, device="cuda")
    plan.exec(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    y = out[: bs * N].view(bs, N)
    rows = sorted({0, 1, bs // 2 - 1, bs // 2, bs - 2, bs - 1} | {int(v) for v in np.random.default_rng(1).integers(0, bs, 6)})
    for r in rows:
        assert O.rel_l2(y[r].cpu().numpy()[None], O.fft_ref(x[r].cpu().numpy()[None])) <= O.tolerance(dt, logN), r
    num = sum(float((y[b0:b0 + step].abs().double() ** 2).sum()) for b0 in range(0, bs, step))
    den = sum(float((x[b0:b0 + step].abs().double() ** 2).sum()) for b0 in range(0, bs, step))
    assert abs(num / den / N - 1) < (1e-5 if dt == "float2" else 1e-12)
    plan.close()
    del x, xr, out, y
    torch.cuda.empty_cache()


def test_plans_on_concurrent_streams():
    # independent plans (and one plain plan shared by two streams: it owns no scratch memory)
    # queued on different streams at the same time give the results of running them one by one
    torch = _torch()
    cases = [("float2", 13, 600), ("double2", 16, 40), ("float2", 20, 6), ("double2", 9, 5000)]
    xs = [torch.from_numpy(make(bs, 1 << logN, dt, logN)).cuda() for dt, logN, bs in cases]
    plans = [turbofft_amd.TurboFFT(logN, dt) for dt, logN, bs in cases]
    outs = [torch.zeros(p.out_elems(bs), dtype=x.dtype, device="cuda") for p, x, (dt, logN, bs) in zip(plans, xs, cases)]
    ref = [p.fft(x).clone() for p, x in zip(plans, xs)]
    streams = [torch.cuda.Stream() for _ in cases]
    torch.cuda.synchronize()
    for rep in range(5):
        for p, x, o, st, (dt, logN, bs) in zip(plans, xs, outs, streams, cases):
            p.exec(x.data_ptr(), o.data_ptr(), bs, st.cuda_stream)
    torch.cuda.synchronize()
    for o, r in zip(outs, ref):
        assert torch.equal(o[: r.numel()].view_as(r), r)
    # one plain single-launch plan on two streams, different buffers
    p, x, (dt, logN, bs) = plans[0], xs[0], cases[0]
    x2 = torch.from_numpy(make(bs, 1 << logN, dt, 99)).cuda()
    r2 = p.fft(x2).clone()
    o1, o2 = torch.zeros_like(ref[0]), torch.zeros_like(r2)
    torch.cuda.synchronize()
    for rep in range(5):
        p.exec(x.data_ptr(), o1.data_ptr(), bs, streams[0].cuda_stream)
        p.exec(x2.data_ptr(), o2.data_ptr(), bs, streams[1].cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(o1, ref[0]) and torch.equal(o2, r2)
    for p in plans:
        p.close()


def test_small_batches_of_one_plan_on_several_streams():
    # fp32 2^13 is a single launch for large batches; its small-batch row runs two launches through an
    # intermediate buffer the plan owns -- one per stream, so executions of ONE plan on different
    # streams do not share it (ten streams: more than the plan keeps buffers for, the rest run the main row)
    torch = _torch()
    dt, logN = "float2", 13
    plan = turbofft_amd.TurboFFT(logN, dt)
    cap = plan.small_batch_max()
    assert cap >= 1 and plan.launches == 1
    bs = min(cap, 4)
    small_names, main_names = plan.kernel_names_for_batch(bs), plan.kernel_names_for_batch(cap + 1)
    assert len(small_names) == 2 and main_names == plan.kernel_names() and small_names != main_names
    xs = [torch.from_numpy(make(bs, 1 << logN, dt, 200 + i)).cuda() for i in range(10)]
    want = [torch.from_numpy(O.fft_ref(x.cpu().numpy())) for x in xs]
    outs = [torch.zeros_like(x) for x in xs]
    streams = [torch.cuda.Stream() for _ in xs]
    torch.cuda.synchronize()
    for rep in range(10):
        for x, o, st in zip(xs, outs, streams):
            plan.exec(x.data_ptr(), o.data_ptr(), bs, st.cuda_stream)
    torch.cuda.synchronize()
    for o, w in zip(outs, want):
        assert O.rel_l2(o.cpu().numpy(), w.numpy()) <= O.tolerance(dt, logN)
    # the same input gives the same bits on every stream that has a buffer of its own (the first eight)
    o2 = torch.zeros_like(outs[0])
    plan.exec(xs[0].data_ptr(), o2.data_ptr(), bs, streams[3].cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(o2, outs[0])
    # (the streams beyond the eighth ran the large-batch row: same transform, held to the same bar above)
    # per-launch timing describes the plan's own row (one launch), whatever the batch
    ms = plan.time_launches(xs[0].data_ptr(), outs[0].data_ptr(), bs, 1, 3)
    assert len(ms) == 1 and ms[0] > 0
    plan.close()


def test_capture_before_the_shared_group_slots_exist():
    # a fault-tolerant plan with groups of 32 tiles allocates the slots its blocks share a group through at the first
    # execution that needs them; when that first execution is a graph capture nothing can be allocated, the captured
    # launches walk whole groups instead, and the replays are still right and still counted
    torch = _torch()
    dt, logN, bs = "float2", 12, 300
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=32)
    x = torch.from_numpy(make(bs, 1 << logN, dt, 7)).cuda()
    out = torch.empty(plan.out_elems(bs), dtype=torch.complex64, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
    for rep in range(2):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert O.rel_l2(out[: bs << logN].view(bs, -1).cpu().numpy(), O.fft_ref(x.cpu().numpy())) <= O.tolerance(dt, logN)
    eager = plan.fft(x).clone()            # allocates the slots and shares the groups
    torch.cuda.synchronize()
    assert torch.equal(eager, out[: bs << logN].view(bs, -1))
    c = plan.ft_counters()
    assert c["detected"] == 0 and c["checked"] == 3 * plan.grid(0, bs)
    plan.close()


def test_cli_vendor_modes():
    # --if_bench 12: the vendor library alone, same line format (cufft.h:45); --if_verify adds the
    # comparison with its result after the one with the host FFT
    if not turbofft_amd.vendor_available():
        pytest.skip("libhipfft.so cannot be opened")
    r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "12", "--datatype", "0", "--param_1", "22",
                        "--logN_begin", "9", "--logN_end", "12"], capture_output=True, text=True, timeout=300)
    print(r.stdout[-2000:], r.stderr[-500:], flush=True)
    assert r.returncode == 0
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("hipFFT, ")]
    assert [int(ln.split(",")[1]) for ln in lines] == [9, 10, 11, 12]
    assert not [ln for ln in r.stdout.splitlines() if ln.startswith("turboFFT, ")]
    r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "0", "--if_verify", "1", "--if_profile", "1", "--logN", "12",
                        "--bs", "8", "--bs_end", "8", "--datatype", "1"], capture_output=True, text=True, timeout=300)
    print(r.stdout[-2000:], r.stderr[-500:], flush=True)
    assert r.returncode == 0 and "Error detected" not in r.stdout
    assert r.stdout.count("Compare finished.") == 2
    assert r.stdout.count("hipFFT, 12, 3,") == 2 and r.stdout.count("turboFFT, 12, 3,") == 2


def test_cli_bench_modes():
    # the reference's run scripts (compile.sh:12-29): --if_bench 2 prints one line per logN at
    # logBS + logN = param_1; with FT the counters follow.  Restricted here to a few sizes.
    for extra in ([], ["--if_ft", "1", "--if_err", "1", "--thread_bs", "4"]):
        r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "2", "--datatype", "0", "--param_1", "22",
                            "--logN_begin", "8", "--logN_end", "17"] + extra,
                           capture_output=True, text=True, timeout=120)
        print(r.stdout[-2000:], r.stderr[-500:], flush=True)
        assert r.returncode == 0
        lines = [ln for ln in r.stdout.splitlines() if ln.startswith("turboFFT, ")]
        assert [int(ln.split(",")[1]) for ln in lines] == list(range(8, 18))
        for ln in lines:                       # turboFFT, logN, logBS, ms, GFLOPS, GB/s
            f = [v.strip() for v in ln.split(",")]
            assert int(f[1]) + int(f[2]) == 22 and float(f[3]) > 0 and float(f[4]) > 0 and float(f[5]) > 0


@pytest.mark.parametrize("extra", [[], ["--if_ft", "1", "--thread_bs", "4"], ["--if_ft", "1", "--if_err", "1", "--thread_bs", "2"]])
def test_cli_all_batch_sizes_sweep(extra):
    # --if_bench 1 (main.cu:114-128): for every logN all batch sizes 1, 2, 4 ... 2^(param_1 - logN),
    # one metric line each, plain and fault tolerant
    p1 = 14
    r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "1", "--datatype", "1", "--param_1", str(p1),
                        "--logN_begin", "9", "--logN_end", "11"] + extra, capture_output=True, text=True, timeout=300)
    print(r.stdout[-3000:], r.stderr[-500:], flush=True)
    assert r.returncode == 0
    lines = [[v.strip() for v in ln.split(",")] for ln in r.stdout.splitlines() if ln.startswith("turboFFT, ")]
    want = [(logN, lb) for logN in (9, 10, 11) for lb in range(0, p1 - logN + 1)]
    assert [(int(f[1]), int(f[2])) for f in lines] == want          # batch column doubles from 1 up to the cap
    for f in lines:
        ms, gflops, gbs = float(f[3]), float(f[4]), float(f[5])
        N, bs = 1 << int(f[1]), 1 << int(f[2])
        assert ms > 0
        # the metric columns are the reference's formulas of the time column (main.cu:68-69),
        # which is printed with three decimals
        lo, hi = max(ms - 6e-4, 1e-7), ms + 6e-4
        assert 5.0 * N * int(f[1]) * bs / hi / 1e6 - 2e-3 <= gflops <= 5.0 * N * int(f[1]) * bs / lo / 1e6 + 2e-3
        assert 2.0 * N * bs * 16 / hi / 1e6 - 2e-3 <= gbs <= 2.0 * N * bs * 16 / lo / 1e6 + 2e-3
    ft = [ln for ln in r.stdout.splitlines() if ln.startswith("turboFFT_ft, ")]
    assert len(ft) == (len(want) if extra else 0)
    if "--if_err" not in extra:
        assert all("detected=0," in ln for ln in ft)


def test_cli_gpu_flag_selects_the_plan_table(tmp_path):
    # CommandLineParser.h:93-109: --gpu <name> reads param/<name>/param_<T>.csv and T4 lowers the
    # sweep to logBS + logN = 26; a name without tables is reported, not ignored
    pdir = os.path.join(os.path.dirname(turbofft_amd.LIB_PATH), "param")
    name = "unit_test_gpu_%d" % os.getpid()
    os.makedirs(os.path.join(pdir, name))
    try:
        src = os.path.join(pdir, "gfx950", "reference_shapes_double2.csv")
        with open(src) as f, open(os.path.join(pdir, name, "param_double2.csv"), "w") as g:
            g.write(f.read())
        common = ["--if_bench", "0", "--if_verify", "1", "--logN", "15", "--bs", "2", "--bs_end", "2", "--datatype", "1"]
        r = subprocess.run([turbofft_amd.CLI_PATH] + common + ["--gpu", name], capture_output=True, text=True, timeout=120)
        print(r.stdout[-1500:], r.stderr[-300:], flush=True)
        assert r.returncode == 0 and f"param/{name}/param_double2.csv" in r.stdout
        assert "Compare finished." in r.stdout and "Error detected" not in r.stdout
        r = subprocess.run([turbofft_amd.CLI_PATH] + common + ["--gpu", "no_such_gpu"], capture_output=True, text=True, timeout=120)
        assert r.returncode != 0 and "Failed to open file." in r.stdout
        r = subprocess.run([turbofft_amd.CLI_PATH] + common + ["--gpu", "MI355X"], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0 and "<built-in gfx950>" in r.stdout
    finally:
        import shutil
        shutil.rmtree(os.path.join(pdir, name))
    r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "2", "--gpu", "T4", "--param", os.path.join(pdir, "gfx950", "param_float2.csv"),
                        "--logN_begin", "12", "--logN_end", "12"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "param_1: 26" in r.stdout and "turboFFT, 12, 14," in r.stdout


def test_cli_sync_timing_line():
    # --if_sync 1 adds the figure the reference's loop measures (a host wait after every launch,
    # main.cu:53-62) beside the default one; it can only be slower
    r = subprocess.run([turbofft_amd.CLI_PATH, "--if_bench", "2", "--datatype", "0", "--param_1", "24", "--if_sync", "1",
                        "--logN_begin", "16", "--logN_end", "17"], capture_output=True, text=True, timeout=120)
    print(r.stdout[-1500:], r.stderr[-300:], flush=True)
    assert r.returncode == 0
    a = [float(ln.split(",")[3]) for ln in r.stdout.splitlines() if ln.startswith("turboFFT, ")]
    b = [float(ln.split(",")[3]) for ln in r.stdout.splitlines() if ln.startswith("turboFFT_sync, ")]
    assert len(a) == len(b) == 2 and all(y > 0.9 * x for x, y in zip(a, b))


SMALL = [(dt, r) for dt in ("float2", "double2")
         for r in __import__("turbofft_amd.codegen.plan", fromlist=["load_plan_csv"]).load_plan_csv(
             os.path.join(os.path.dirname(turbofft_amd.LIB_PATH), "param", "gfx950", f"param_{dt}_small.csv"))]


@pytest.mark.parametrize("dt,row", SMALL, ids=[f"{dt}-{r.logN}" for dt, r in SMALL])
def test_small_batch_rows(dt, row):
    # batches of a few transforms run the narrow-tile row of param_<T>_small.csv (two launches that
    # spread one transform over many CUs); the first batch above its cap runs the large-batch row.
    # Same accuracy bar on both sides of the switch, and through the entry point without allocation.
    torch = _torch()
    logN, cap = row.logN, row.tiles
    plan = turbofft_amd.TurboFFT(logN, dt)
    assert plan.small_batch_max() == cap
    cdt = torch.complex64 if dt == "float2" else torch.complex128
    st = torch.cuda.current_stream().cuda_stream
    for bs in sorted({1, 2, 3, cap, cap + 1}):
        x = make(bs, 1 << logN, dt, 7 * logN + bs)
        xd = torch.from_numpy(x).cuda()
        ref = O.fft_ref(x)
        guard = 1024
        out = torch.full((plan.out_elems(bs) + guard,), 5.0 - 2.0j, dtype=cdt, device="cuda")
        plan.exec(xd.data_ptr(), out.data_ptr(), bs, st)
        torch.cuda.synchronize()
        y = out[: bs << logN].view(bs, -1).cpu().numpy()
        assert max(O.rel_l2(y[b], ref[b]) for b in range(bs)) <= O.tolerance(dt, logN), (bs, "small" if bs <= cap else "large")
        assert bool((out[plan.out_elems(bs):] == 5.0 - 2.0j).all()), "wrote past the output buffer"
        # without workspace from the caller
        out2 = torch.full(((bs << logN) + guard,), 5.0 - 2.0j, dtype=cdt, device="cuda")
        plan.exec_static(xd.data_ptr(), out2.data_ptr(), bs, st)
        torch.cuda.synchronize()
        assert torch.equal(out2[: bs << logN], out[: bs << logN])
        assert bool((out2[bs << logN:] == 5.0 - 2.0j).all())
    # switched off: the large-batch row serves every batch
    plan.set_small_batch(False)
    assert plan.small_batch_max() == 0
    x = make(2, 1 << logN, dt, 3)
    y = gpu_fft(plan, x)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    # fault-tolerant plans and caller-supplied tables keep their one row
    ft = turbofft_amd.TurboFFT(logN, dt, if_ft=1)
    assert ft.small_batch_max() == 0
    ft.close()
    plan.close()


def test_overlapping_buffers_are_rejected():
    torch = _torch()
    for logN, dt in ((10, "float2"), (16, "float2")):
        plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1)
        N, bs = 1 << logN, 4
        buf = torch.zeros(4 * N * bs, dtype=torch.complex64, device="cuda")
        st = torch.cuda.current_stream().cuda_stream
        for in_off, out_off in ((0, 0), (0, N * bs // 2), (N * bs // 2, 0)):
            with pytest.raises(turbofft_amd.TurboFFTError, match="overlaps"):
                plan.exec(buf.data_ptr() + 8 * in_off, buf.data_ptr() + 8 * out_off, bs, st)
        if plan.launches > 1:                  # `in` inside the workspace half of `out`
            with pytest.raises(turbofft_amd.TurboFFTError, match="overlaps"):
                plan.exec(buf.data_ptr() + 8 * N * bs, buf.data_ptr(), bs, st)
        plan.exec(buf.data_ptr() + 8 * plan.out_elems(bs), buf.data_ptr(), bs, st)      # adjacent is fine
        torch.cuda.synchronize()
        plan.close()


VARIANTS_DIR = os.path.join(os.path.dirname(turbofft_amd.LIB_PATH), "param", "gfx950")


def _variant_rows(dt):
    from turbofft_amd.codegen.plan import load_plan_csv
    return [r for r in load_plan_csv(os.path.join(VARIANTS_DIR, f"variants_{dt}.csv")) if r.launches]


@pytest.mark.parametrize("dt", ["float2", "double2"])
def test_optional_kernel_variants(dt):
    # rows of variants_<T>.csv: split exchange, next-tile prefetch and cross-lane last pass
    # kernels that the default table does not use; every one must meet the same accuracy bar
    path = os.path.join(VARIANTS_DIR, f"variants_{dt}.csv")
    rows = _variant_rows(dt)
    assert rows
    for r in rows:
        plan = turbofft_amd.TurboFFT(r.logN, dt, param_csv=path)
        BS = plan.BS[0] if plan.launches == 1 else 1
        bs = 70 * BS + max(1, BS // 2) if r.logN <= 13 else 5      # many tiles: the prefetch loop must iterate
        x = make(bs, 1 << r.logN, dt, 100 + r.logN)
        y = gpu_fft(plan, x)
        ref = O.fft_ref(x)
        for b in range(bs):
            assert O.rel_l2(y[b], ref[b]) <= O.tolerance(dt, r.logN), (r, b)
        # the same rows with fault tolerance (cross-lane rows fall back to the LDS kernel)
        # (tight detection rule: with the default one the error's own share of the checksum
        # magnitude keeps the ratio of an 8192-point tile next to the threshold)
        planf = turbofft_amd.TurboFFT(r.logN, dt, if_err=1, thread_bs=3, param_csv=path)
        planf.set_ft_params(0.0, 1e-4 if dt == "float2" else 1e-9, correct=True)
        planf.set_injection(1, mag=1e3)
        yf = gpu_fft(planf, x)
        c = planf.ft_counters()
        assert c["detected"] == c["corrected"] > 0 and c["uncorrectable"] == 0
        for b in range(bs):
            assert O.rel_l2(yf[b], ref[b]) <= O.tolerance(dt, r.logN), (r, b, "ft")


def test_seeded_random_shapes():
    """Forty seeded draws of (type, logN, batch, tiles per block, fault tolerance): ragged
    batches, every plan depth, plain and checksummed kernels, against the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        dt = ["float2", "double2"][int(rng.integers(2))]
        logN = int(rng.integers(1, 21))
        bs = int(rng.integers(1, max(2, min(200, (1 << 22) >> logN))))
        tbs = int(rng.choice([1, 1, 2, 3, 5, 8]))
        ft = int(rng.integers(2))
        plan = turbofft_amd.TurboFFT(logN, dt, if_ft=ft, thread_bs=tbs)
        print(f"[random case {case}] ft={ft} thread_bs={tbs}", flush=True)
        x = make(bs, 1 << logN, dt, 1000 + case, normal=bool(rng.integers(2)))
        y = gpu_fft(plan, x)
        ref = O.fft_ref(x)
        assert O.rel_l2(y, ref) <= O.tolerance(dt, logN)
        worst = max(O.rel_l2(y[b], ref[b]) for b in range(bs))
        assert worst <= O.tolerance(dt, logN)
        if ft:
            c = plan.ft_counters()
            assert c["detected"] == 0 and c["checked"] == sum(plan.grid(i, bs) for i in range(plan.launches))
        plan.close()


@pytest.mark.parametrize("dt,logN,bs,ft", [("float2", 10, 7, 0), ("double2", 16, 3, 0), ("float2", 24, 1, 0), ("float2", 12, 9, 1),
                                           ("double2", 10, 200, 16), ("float2", 17, 20, 32)])
def test_exec_inside_a_hip_graph(dt, logN, bs, ft):
    """turbofft_exec allocates nothing and records no memset, so a plan can be captured into
    a HIP graph; every replay (with new input written in between) must equal the eager result."""
    torch = _torch()
    # ft > 1: checksum groups of that many tiles, shared by several blocks, with injected errors
    # that the follow-up launch corrects -- all of it inside the graph
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=ft, thread_bs=ft if ft > 1 else (2 if ft else 1))
    if ft > 1:
        assert plan.ft_part_len(plan.launches - 1) == 8
        plan.set_ft_params(1000.0, 1e-3, correct=1)
        plan.set_injection(2, every=3 * ft * plan.tb_gap(plan.launches - 1) + 1, tile_phase=1, s=0, m=0, mag=1.0e7)
    cdt = torch.complex64 if dt == "float2" else torch.complex128
    x = torch.from_numpy(make(bs, 1 << logN, dt, 50)).cuda()
    out = torch.empty(plan.out_elems(bs), dtype=cdt, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, stream.cuda_stream)        # warm-up outside the capture
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        x.copy_(torch.from_numpy(make(bs, 1 << logN, dt, 60 + rep)).cuda())
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out[: bs * (1 << logN)].view(bs, 1 << logN).clone()
        eager = plan.fft(x).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {rep} differs from the eager run"
        assert O.rel_l2(got.cpu().numpy(), O.fft_ref(x.cpu().numpy())) <= O.tolerance(dt, logN)
    if ft:
        # the groups-checked counter lives on the device: replays count like eager executions
        # (1 warm-up + 3 replays + 3 eager runs; the capture itself executes nothing)
        c = plan.ft_counters()
        assert c["checked"] == 7 * sum(plan.grid(i, bs) for i in range(plan.launches))
        if ft > 1:
            assert c["detected"] > 0 and c["detected"] % 7 == 0 and c["corrected"] == c["detected"] and c["uncorrectable"] == 0
        else:
            assert c["detected"] == 0
    plan.close()


def test_streaming_yardsticks_run():
    # the measurement kernels of known traffic (nothing of a transform): every flavour moves what it says,
    # the fused two-pass copy through the per-XCD ring copies right and never runs into its time limit
    torch = _torch()
    nbytes = 256 << 20
    src = torch.rand(nbytes // 4, device="cuda", dtype=torch.float32)
    dst = torch.zeros(nbytes // 4, device="cuda", dtype=torch.float32)
    st = torch.cuda.current_stream().cuda_stream
    for mode in (0, 1, 4, 5, 12, 13, 12 + 48):
        dst.zero_()
        assert turbofft_amd.membench(mode, src.data_ptr(), dst.data_ptr(), nbytes, 1, 2, st) > 0
        assert torch.equal(src, dst)
    assert turbofft_amd.membench(2 + 12, src.data_ptr(), dst.data_ptr(), nbytes, 1, 2, st) > 0
    assert turbofft_amd.membench(3 + 12, src.data_ptr(), dst.data_ptr(), nbytes, 1, 2, st) > 0
    for lane in (8, 16):
        for run in (128, 256, 512):
            for ls in (12, 19):
                keep = src.clone()
                assert turbofft_amd.membench_strided(False, lane, run, ls, 16, src.data_ptr(), dst.data_ptr(), nbytes, 1, 2, st) > 0
                assert torch.equal(src, keep)
                dst.zero_()
                assert turbofft_amd.membench_strided(True, lane, run, ls, 4, src.data_ptr(), dst.data_ptr(), nbytes, 1, 2, st) > 0
                v = dst.view(-1, 2)
                assert bool((v[:, 1] == 1).all())              # every 8-byte element of the buffer was written
    with pytest.raises(turbofft_amd.TurboFFTError):
        turbofft_amd.membench_strided(True, 8, 100, 12, 4, src.data_ptr(), dst.data_ptr(), nbytes, 1, 2, st)
    scratch = torch.empty((8 * 3 * 2 * 512 * 1024) // 4, device="cuda", dtype=torch.float32)
    for G, R, bpc in ((1, 2, 2), (2, 3, 3), (1, 3, 8)):
        dst.zero_()
        ms, stats = turbofft_amd.membench_fused(G, R, bpc, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes, 200, 1, 2, st)
        assert ms > 0 and stats["timed_out"] == 0 and sum(stats["blocks_per_xcd"]) == stats["blocks"]
        assert torch.equal(src, dst)
    with pytest.raises(turbofft_amd.TurboFFTError):           # the ring does not fit the scratch buffer
        turbofft_amd.membench_fused(4, 3, 2, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes)
    with pytest.raises(turbofft_amd.TurboFFTError):           # one slot: a first pass would wait for a later ticket
        turbofft_amd.membench_fused(1, 1, 2, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes)
    # the same copy with teams of blocks that share one slot: right for every team size and piece, never out of time
    scratch = torch.empty((64 << 20) // 4, device="cuda", dtype=torch.float32)
    for T, piece, bpc in ((8, 512, 1), (4, 256, 2), (16, 1024, 1), (32, 128, 4)):
        dst.zero_()
        ms, stats = turbofft_amd.membench_team(T, bpc, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes, 200, 1, 2, st, piece_kib=piece)
        assert ms > 0 and stats["timed_out"] == 0 and stats["rounds_per_block"] > 0
        assert torch.equal(src, dst)
    with pytest.raises(turbofft_amd.TurboFFTError):           # a member's share of the piece would not fit its registers
        turbofft_amd.membench_team(4, 1, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes, piece_kib=1024)


FUSED = [("float2", 16), ("double2", 15), ("double2", 16)]


@pytest.mark.parametrize("dt,logN", FUSED)
def test_fused_pair_matches_the_dft_and_the_two_launches(dt, logN, monkeypatch):
    # a plan created with TURBOFFT_FUSED=1 holds ONE kernel for both launches of these sizes (teams of blocks pass the
    # intermediate through a slot in their XCD's L2); it runs for batches that give every team a piece
    torch = _torch()
    monkeypatch.setenv("TURBOFFT_FUSED", "1")
    plan = turbofft_amd.TurboFFT(logN, dt)
    info = plan.fused_info()
    assert info is not None and info["grid_blocks"] == 8 * info["teams_per_xcd"] * info["team_blocks"]
    teams = 8 * info["teams_per_xcd"] * info["transforms_per_piece"]
    assert plan.launches == 2 and len(plan.kernel_names_for_batch(teams)) == 1 and "_pair_" in plan.kernel_names_for_batch(teams)[0]
    assert plan.kernel_names_for_batch(teams - 1) == plan.kernel_names()           # too few pieces: the two launches
    for bs, seed in ((teams, 1), (3 * teams + 5, 2), (teams - 1, 3)):
        x = make(bs, 1 << logN, dt, seed)
        y = gpu_fft(plan, x)
        assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    # against the plan's two launches on the same input: the same transform to rounding, on an output of N*bs elements only
    bs = 2 * teams + 1
    x = torch.from_numpy(make(bs, 1 << logN, dt, 9)).cuda()
    out = torch.zeros(2 * bs << logN, dtype=x.dtype, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for rep in range(3):                                                        # the control block is left clean for the next launch
        out.zero_()
        plan.exec(x.data_ptr(), out.data_ptr(), bs, st)
    torch.cuda.synchronize()
    assert not bool(out[bs << logN:].any())                                     # no intermediate in the caller's buffer
    out = out[: bs << logN]
    plan.set_fused(False)
    assert plan.fused_info() is None and len(plan.kernel_names_for_batch(bs)) == 2
    two = plan.fft(x)
    torch.cuda.synchronize()
    assert O.rel_l2(out.view(bs, -1).cpu().numpy(), two.cpu().numpy()) <= O.tolerance(dt, logN)
    plan.set_fused(True)
    plan.close()
    # without the variable a plan holds no fused kernel and says so
    monkeypatch.delenv("TURBOFFT_FUSED")
    plain = turbofft_amd.TurboFFT(logN, dt)
    assert plain.fused_info() is None
    with pytest.raises(turbofft_amd.TurboFFTError):
        plain.set_fused(True)
    plain.close()


def test_fused_pair_on_several_streams_and_in_a_graph(monkeypatch):
    # every stream that runs the fused kernel owns its slots and control block (eight sets per plan, later streams
    # run the two launches); a stream that first shows up while it is being captured gets none and records the two launches
    torch = _torch()
    monkeypatch.setenv("TURBOFFT_FUSED", "1")
    dt, logN = "float2", 16
    plan = turbofft_amd.TurboFFT(logN, dt)
    info = plan.fused_info()
    bs = 8 * info["teams_per_xcd"] + 3
    xs = [torch.from_numpy(make(bs, 1 << logN, dt, 300 + i)).cuda() for i in range(10)]
    want = [O.fft_ref(x.cpu().numpy()) for x in xs]
    outs = [torch.zeros(plan.out_elems(bs), dtype=x.dtype, device="cuda") for x in xs]
    streams = [torch.cuda.Stream() for _ in xs]
    torch.cuda.synchronize()
    for rep in range(4):
        for x, o, s in zip(xs, outs, streams):
            plan.exec(x.data_ptr(), o.data_ptr(), bs, s.cuda_stream)
    torch.cuda.synchronize()
    for o, w in zip(outs, want):
        assert O.rel_l2(o[: bs << logN].view(bs, -1).cpu().numpy(), w) <= O.tolerance(dt, logN)
    plan.close()
    # capture on a stream the plan has not seen (its first set belongs to the default stream by then)
    plan = turbofft_amd.TurboFFT(logN, dt)
    x = xs[0]
    eager = plan.fft(x).clone()
    out = torch.zeros(plan.out_elems(bs), dtype=x.dtype, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
    for rep in range(2):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert O.rel_l2(out[: bs << logN].view(bs, -1).cpu().numpy(), want[0]) <= O.tolerance(dt, logN)
    # and on a stream that owns a set: the fused kernel itself is captured (it clears its own control block)
    with torch.cuda.stream(stream):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, stream.cuda_stream)
    stream.synchronize()
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2, stream=stream):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out[: bs << logN].view(bs, -1), eager)
    plan.close()


def test_fused_pair_that_gives_up_is_reported_and_replaced(monkeypatch):
    # every wait of the fused kernel is bounded; with no time at all (a negative limit, set by the host) every block gives
    # up as it starts and leaves.  The execution after that one reports it, and the plan runs its two launches from then on
    torch = _torch()
    monkeypatch.setenv("TURBOFFT_FUSED", "1")
    monkeypatch.setenv("TURBOFFT_FUSED_LIMIT_MS", "-1")
    dt, logN = "double2", 15
    plan = turbofft_amd.TurboFFT(logN, dt)
    info = plan.fused_info()
    assert info is not None
    bs = 8 * info["teams_per_xcd"] + 1
    x = torch.from_numpy(make(bs, 1 << logN, dt, 4)).cuda()
    out = torch.zeros(plan.out_elems(bs), dtype=x.dtype, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    plan.exec(x.data_ptr(), out.data_ptr(), bs, st)                 # launches; the kernel writes nothing
    torch.cuda.synchronize()
    assert not bool(out.any())
    with pytest.raises(turbofft_amd.TurboFFTError, match="incomplete"):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, st)
    assert plan.fused_info() is None and len(plan.kernel_names_for_batch(bs)) == 2
    y = plan.fft(x)
    torch.cuda.synchronize()
    assert O.rel_l2(y.cpu().numpy(), O.fft_ref(x.cpu().numpy())) <= O.tolerance(dt, logN)
    plan.close()
