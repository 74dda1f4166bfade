"""turbofft_exec_static: the entry point that allocates nothing and brings its own workspace.
Through the C ABI, against turbofft_exec on the same input (same kernels: bit-identical),
two calls in a row per plan, the second with a smaller batch."""
import numpy as np
import pytest

import turbofft_amd
from oracle import turbofft_oracle as O

pytestmark = pytest.mark.gpu

GUARD = 4096          # elements after out[N*bs) that must stay untouched


def _torch():
    import torch
    assert torch.cuda.is_available()
    return torch


def _input(torch, bs, N, dt, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    rdt = torch.float32 if dt == "float2" else torch.float64
    return torch.view_as_complex(torch.rand((bs, N, 2), generator=g, device="cuda", dtype=rdt) * 2 - 1)


CASES = [("float2", 16, 64, 5, 0), ("double2", 15, 16, 3, 0), ("float2", 23, 1, 1, 0), ("double2", 16, 8, 2, 1),
         ("float2", 10, 300, 7, 0), ("float2", 19, 16, 1, 1)]


@pytest.mark.parametrize("dt,logN,bs1,bs2,ft", CASES)
def test_exec_static_equals_exec(dt, logN, bs1, bs2, ft):
    torch = _torch()
    N = 1 << logN
    cdt = torch.complex64 if dt == "float2" else torch.complex128
    esize = 8 if dt == "float2" else 16
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=ft, thread_bs=2 if ft else 1)
    if plan.launches > 1:
        assert N * bs1 * esize <= turbofft_amd.STATIC_WORKSPACE_BYTES
    st = torch.cuda.current_stream().cuda_stream
    for call, bs in enumerate((bs1, bs2)):
        print(f"[exec_static] {dt} logN={logN} bs={bs} launches={plan.launches} ft={ft} call={call}", flush=True)
        x = _input(torch, bs, N, dt, 10 * logN + call)
        want = torch.empty(plan.out_elems(bs), dtype=cdt, device="cuda")
        plan.exec(x.data_ptr(), want.data_ptr(), bs, st)
        got = torch.full((N * bs + GUARD,), 7.0 + 3.0j, dtype=cdt, device="cuda")      # result + guard, no workspace half
        plan.exec_static(x.data_ptr(), got.data_ptr(), bs, st)
        torch.cuda.synchronize()
        assert torch.equal(got[: N * bs], want[: N * bs])
        assert bool((got[N * bs:] == 7.0 + 3.0j).all()), "wrote past out[N*bs)"
        xs = x[: min(bs, 2)].cpu().numpy()
        assert O.rel_l2(got[: xs.shape[0] * N].view(-1, N).cpu().numpy(), O.fft_ref(xs)) <= O.tolerance(dt, logN)
    if ft:
        c = plan.ft_counters()
        assert c["detected"] == 0 and c["checked"] == 2 * sum(plan.grid(i, b) for b in (bs1, bs2) for i in range(plan.launches))
    plan.close()


def test_exec_static_rejects_what_does_not_fit():
    torch = _torch()
    plan = turbofft_amd.TurboFFT(16, "float2")
    assert plan.launches == 2
    N = 1 << 16
    fit = turbofft_amd.STATIC_WORKSPACE_BYTES // (8 * N)            # 128 transforms
    x = _input(torch, fit + 1, N, "float2", 3)
    out = torch.empty((fit + 1) * N, dtype=torch.complex64, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    with pytest.raises(turbofft_amd.TurboFFTError, match="static workspace"):
        plan.exec_static(x.data_ptr(), out.data_ptr(), fit + 1, st)
    with pytest.raises(turbofft_amd.TurboFFTError, match="negative"):
        plan.exec_static(x.data_ptr(), out.data_ptr(), -1, st)
    with pytest.raises(turbofft_amd.TurboFFTError, match="overlaps"):
        plan.exec_static(x.data_ptr(), x.data_ptr(), 2, st)
    plan.exec_static(x.data_ptr(), out.data_ptr(), fit, st)        # the largest batch that fits
    ref = torch.empty(plan.out_elems(fit), dtype=torch.complex64, device="cuda")
    plan.exec(x.data_ptr(), ref.data_ptr(), fit, st)
    torch.cuda.synchronize()
    assert torch.equal(out[: fit * N], ref[: fit * N])
    plan.close()
    one = turbofft_amd.TurboFFT(12, "double2")                      # single launch: no workspace, no limit
    bs = 3 * turbofft_amd.STATIC_WORKSPACE_BYTES // (16 << 12)
    x = _input(torch, bs, 1 << 12, "double2", 4)
    a = torch.empty(bs << 12, dtype=torch.complex128, device="cuda")
    b = torch.empty(bs << 12, dtype=torch.complex128, device="cuda")
    one.exec_static(x.data_ptr(), a.data_ptr(), bs, st)
    one.exec(x.data_ptr(), b.data_ptr(), bs, st)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    one.close()


def test_exec_static_inside_a_hip_graph():
    # what the entry point is for: captured once, replayed with new input
    torch = _torch()
    logN, bs = 17, 6
    N = 1 << logN
    plan = turbofft_amd.TurboFFT(logN, "float2")
    x = _input(torch, bs, N, "float2", 1)
    out = torch.empty(bs * N, dtype=torch.complex64, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        plan.exec_static(x.data_ptr(), out.data_ptr(), bs, stream.cuda_stream)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        plan.exec_static(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        x.copy_(_input(torch, bs, N, "float2", 20 + rep))
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.empty(plan.out_elems(bs), dtype=torch.complex64, device="cuda")
        plan.exec(x.data_ptr(), eager.data_ptr(), bs, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(out, eager[: bs * N]), f"replay {rep} differs from the eager run"
    plan.close()
