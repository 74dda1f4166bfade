#!/usr/bin/env python3
"""Benchmark of the batched FFT hot path on one MI355X.

Default workload: benchmark configuration 2 -- forward C2C FFT, fp32 complex, N=2^13,
batch 2^15 (logBS+logN=28, 2 GiB in, 2 GiB out), synthetic uniform[-1,1) data
resident in HBM before the timed region.  A "step" is one transform of the
whole batch.  Prints ONE JSON line:
  metric/value : algorithmic HBM GB/s = 2*N*bs*sizeof(T)/t  (the reference's
                 figure, main.cu:69), plus "gflops" = 5*N*log2N*bs/t (main.cu:68)
  roofline     : dominant kernel against the 8 TB/s HBM peak, timed with HIP
                 events on the launch stream over the timed region
  cpu_baseline : scipy.fft (pocketfft) on the host cores for a bounded sample
                 of the same workload, scaled to the same unit; "single_thread" inside it
                 is numpy.fft.fft, the routine of the accuracy oracle, on one core
  ft_overhead  : run time of the same workload with the fused checksums over the
                 plain plan, measured after the timed region in alternating blocks
                 (plain, checksummed, plain, ...) so that both see the same device state;
                 the ratio of the two medians (--no_ft_overhead skips it);
                 "offline" inside it is the same comparison for separate checksum passes
                 before and after the plain plan (the reference's cufft_ft.h baseline),
                 "groups_of_32" the same with the reference's published group size,
                 "thread_level" the same for thread-level verification (if_ft = 2)
                 "full_table" the same with the reference's own complex checksum table in place of
                 this build's compact (reduced-precision cotangent) form, for the sizes whose
                 fault-tolerant kernels read the compact form by default
  sweep        : the whole metric after the timed region: logN 7..24 x {fp32, fp64} at
                 logBS+logN=28 (main.cu:114-128, compile.sh:12-29), per case launches, median ms
                 of >= 10 steps, algorithmic GB/s, fraction of the 8 TB/s peak and the overhead
                 of the fused checksums at groups of 4 tiles (--no_sweep skips it)
  prewarm_s    : untimed executions before the warm-up steps, by time rather than by count:
                 a device that has been idle clocks up over its first tenths of a second
  vendor_baseline : hipFFT (rocFFT) on the same buffers and workload, after the timed
                 region, the side-by-side the reference runs against cuFFT
                 (main.cu:105,121); --no_vendor skips it

Other workloads for tuning: --logN/--datatype/--bs, --sweep (logN 7..24 at
logBS+logN=28 for both types, one JSON line per case to --out; with --vendor
every case is followed by hipFFT on the same buffers).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by
# what the same counter reads for a plain 2 GiB copy (2.000 and 1.000 KiB per count); the runs are
# listed in profiles/.  Keyed by (datatype, logN, bs, fault tolerant); other workloads report null.
MEASURED_TRAFFIC = {
    (0, 13, 1 << 15, 0): 4295993261,     # tfft_f32_row1_N13_b1_n32_s_w3_t3: 1.0002 x algorithmic
    (0, 16, 1 << 12, 0): 4296477780,     # tfft_f32_rowT_N9_b16_n32_w3_t3 (tfft_f32_col_N7_b32_n32_t3: 4295227240)
}


def make_input(torch, bs, N, datatype, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    rdt = torch.float32 if datatype == 0 else torch.float64
    x = torch.rand((bs, N, 2), generator=g, device="cuda", dtype=rdt) * 2 - 1
    return torch.view_as_complex(x)


def prewarm(torch, plan, x, out, bs, seconds):
    """Keep the device busy with the workload for `seconds` (untimed, not part of the steps)."""
    stream = torch.cuda.current_stream().cuda_stream
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            plan.exec(x.data_ptr(), out.data_ptr(), bs, stream)
        n += 8
        torch.cuda.synchronize()
    return time.perf_counter() - t0, n


def stats(v):
    v = sorted(v)
    return {"mean": sum(v) / len(v), "min": v[0], "median": v[len(v) // 2] if len(v) % 2 else 0.5 * (v[len(v) // 2 - 1] + v[len(v) // 2]),
            "max": v[-1]}


def run_case(torch, turbofft_amd, logN, datatype, bs, steps, warmup, if_ft=0, if_err=0, thread_bs=1, param=None,
             x=None, out=None, prewarm_s=0.0, correct=None, inj_every=0, inj_mag=100.0):
    N = 1 << logN
    plan = turbofft_amd.TurboFFT(logN, datatype, if_ft=if_ft, if_err=if_err, thread_bs=thread_bs, param_csv=param)
    if correct is not None:
        plan.set_ft_params(1000.0, 1e-3, correct)
    if inj_every > 0:
        # host-chosen cadence: one tile in every `inj_every` of the last launch gets `inj_mag` added to an element
        plan.set_ft_params(1000.0, 1e-3, 1 if correct is None else correct)
        plan.set_injection(2, every=inj_every, tile_phase=min(123, inj_every - 1), s=0, m=0, mag=inj_mag)
    cdt = torch.complex64 if datatype == 0 else torch.complex128
    if x is None:
        x = make_input(torch, bs, N, datatype)
    if out is None:
        out = torch.empty(plan.out_elems(bs), dtype=cdt, device="cuda")
    if out.numel() < plan.out_elems(bs) or x.numel() < bs * N:
        raise ValueError(f"buffers too small for logN={logN} bs={bs}: out holds {out.numel()} elements, "
                         f"the plan needs {plan.out_elems(bs)}")
    stream = torch.cuda.current_stream().cuda_stream
    pre_s, pre_n = prewarm(torch, plan, x, out, bs, prewarm_s) if prewarm_s > 0 else (0.0, 0)
    for _ in range(warmup):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, stream)
    torch.cuda.synchronize()
    # one event between every two steps (on the stream the kernels are launched on): the whole
    # region gives the mean, the intervals its spread
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        plan.exec(x.data_ptr(), out.data_ptr(), bs, stream)
        ev[i + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1000.0 / steps
    ev_ms = ev[0].elapsed_time(ev[steps]) / steps
    per_step = [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]
    res = {
        "logN": logN, "datatype": datatype, "bs": bs, "launches": plan.launches,
        "plan": {"logNi": plan.logNi, "BS": plan.BS, "n": plan.n, "threads": plan.threads, "lds_bytes": plan.lds_bytes},
        "wall_ms": wall_ms, "event_ms": ev_ms, "step_ms": stats(per_step),
        "gbs": plan.gbs(bs, wall_ms), "gflops": plan.gflops(bs, wall_ms),
        "alg_bytes": plan.algorithmic_bytes(bs), "prewarm_s": pre_s, "prewarm_execs": pre_n,
    }
    if if_ft or if_err:
        # counters accumulate over every execution of the plan (warm-up included)
        res["ft"] = {k: v for k, v in plan.ft_counters().items() if k not in ("flagged", "flagged_truncated")}
        res["ft"]["execs"] = pre_n + warmup + steps
    plan.close()
    return res, x, out


def make_ft_plan(turbofft_amd, logN, datatype, thread_bs, param, compact=True, scheme=1):
    """Fault-tolerant plan; compact=False keeps the full (complex) checksum table for every
    launch (the library reads TURBOFFT_COMPACT_CHECKSUM when a plan is created); scheme 2 is
    thread-level verification."""
    if compact:
        return turbofft_amd.TurboFFT(logN, datatype, if_ft=scheme, thread_bs=thread_bs, param_csv=param)
    old = os.environ.get("TURBOFFT_COMPACT_CHECKSUM")
    os.environ["TURBOFFT_COMPACT_CHECKSUM"] = "0"
    try:
        return turbofft_amd.TurboFFT(logN, datatype, if_ft=1, thread_bs=thread_bs, param_csv=param)
    finally:
        if old is None:
            del os.environ["TURBOFFT_COMPACT_CHECKSUM"]
        else:
            os.environ["TURBOFFT_COMPACT_CHECKSUM"] = old


def interleaved_overhead(torch, turbofft_amd, logN, datatype, bs, x, out, param, thread_bs=4, rounds=7, block=10, compact=True, scheme=1):
    """Plain and checksummed plan of the same workload in alternating blocks of `block`
    executions (plain first and last), each block between two events; the overhead is the
    ratio of the median block times, so neither plan is measured on a colder device."""
    plain = turbofft_amd.TurboFFT(logN, datatype, param_csv=param)
    ft = make_ft_plan(turbofft_amd, logN, datatype, thread_bs, param, compact, scheme)
    stream = torch.cuda.current_stream().cuda_stream
    for pl in (plain, ft):
        for _ in range(3):
            pl.exec(x.data_ptr(), out.data_ptr(), bs, stream)
    torch.cuda.synchronize()
    times = {0: [], 1: []}
    marks = []
    for r in range(2 * rounds + 1):
        which = r % 2
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(block):
            (ft if which else plain).exec(x.data_ptr(), out.data_ptr(), bs, stream)
        e1.record()
        marks.append((which, e0, e1))
    torch.cuda.synchronize()
    for which, e0, e1 in marks:
        times[which].append(e0.elapsed_time(e1) / block)
    counters = {k: v for k, v in ft.ft_counters().items() if k not in ("flagged", "flagged_truncated")}
    info = {"logNi": ft.logNi, "BS": ft.BS, "n": ft.n, "threads": ft.threads, "lds_bytes": ft.lds_bytes, "kernels": ft.kernel_names()}
    plain.close()
    ft.close()
    p, f = stats(times[0]), stats(times[1])
    return {"overhead_pct": 100.0 * (f["median"] / p["median"] - 1.0), "plain_ms": p, "ft_ms": f, "ms_per_step": f["median"],
            "thread_bs": thread_bs, "order": "plain/ft alternating, %d blocks of %d executions each" % (2 * rounds + 1, block),
            "plan": info, "counters": counters}


def vendor_case(torch, turbofft_amd, logN, datatype, bs, x, out, reps=20, warmup=2):
    """hipFFT on the same device buffers; reported beside the result, never part of it."""
    if not turbofft_amd.vendor_available():
        return {"library": "hipFFT", "error": "libhipfft.so could not be opened"}
    esize = 8 if datatype == 0 else 16
    try:
        ms = turbofft_amd.vendor_time(logN, datatype, x.data_ptr(), out.data_ptr(), bs, warmup, reps,
                                      torch.cuda.current_stream().cuda_stream)
    except turbofft_amd.TurboFFTError as e:
        return {"library": "hipFFT", "error": str(e)}
    pts = bs * (1 << logN)
    return {"library": "hipFFT", "value": 2 * pts * esize / ms / 1e6, "unit": "GB/s", "ms_per_step": ms,
            "gflops": 5.0 * pts * logN / ms / 1e6, "reps": reps}


def sweep_rows(torch, turbofft_amd, lo=7, hi=24, steps=10, ft_rounds=2, ft_block=5, log=None):
    """The metric's whole range on this device: for each type and logN in [lo, hi] at
    logBS+logN=28 the plain plan (median of `steps` event-timed steps after a short pre-warm) and
    the overhead of the fused checksums at groups of 4 tiles (plain and checksummed in
    alternating blocks).  One input of 2^28 points and one output of 2 x 2^28 per type serve
    every size."""
    rows = []
    stream = torch.cuda.current_stream().cuda_stream
    for dt in (0, 1):
        cdt = torch.complex64 if dt == 0 else torch.complex128
        x = make_input(torch, 1 << (28 - lo), 1 << lo, dt)
        out = torch.empty(2 << 28, dtype=cdt, device="cuda")
        for logN in range(lo, hi + 1):
            bs = 1 << (28 - logN)
            plan = turbofft_amd.TurboFFT(logN, dt)
            prewarm(torch, plan, x, out, bs, 0.1)
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
            ev[0].record()
            for i in range(steps):
                plan.exec(x.data_ptr(), out.data_ptr(), bs, stream)
                ev[i + 1].record()
            torch.cuda.synchronize()
            st = stats([ev[i].elapsed_time(ev[i + 1]) for i in range(steps)])
            ms = st["median"]
            row = {"logN": logN, "dtype": "f32" if dt == 0 else "f64", "launches": plan.launches, "ms": ms, "ms_min": st["min"],
                   "gbs": plan.gbs(bs, ms), "gflops": plan.gflops(bs, ms), "frac": plan.gbs(bs, ms) / HBM_PEAK_GBS,
                   "frac_per_launch": plan.launches * plan.gbs(bs, ms) / HBM_PEAK_GBS, "steps": steps}
            plan.close()
            if ft_rounds > 0:
                f = interleaved_overhead(torch, turbofft_amd, logN, dt, bs, x, out, None, thread_bs=4, rounds=ft_rounds, block=ft_block)
                row["ft_pct"] = f["overhead_pct"]
                row["ft_false_alarms"] = f["counters"]["detected"]
                # thread-level verification (every tile checked on its own, by its threads)
                f = interleaved_overhead(torch, turbofft_amd, logN, dt, bs, x, out, None, thread_bs=1, rounds=ft_rounds, block=ft_block, scheme=2)
                row["ft_thread_level_pct"] = f["overhead_pct"]
                row["ft_false_alarms"] += f["counters"]["detected"]
            rows.append(row)
            if log:
                log(row)
        del x, out
        torch.cuda.empty_cache()
    return rows


def fused_pair_rows(torch, turbofft_amd, steps=10, rounds=4, log=None):
    """The sizes whose two launches also exist as one kernel (plans created with TURBOFFT_FUSED=1 hold it): that kernel
    against the plan's two launches at logBS+logN=28, in alternating blocks of `steps` event-timed executions."""
    rows = []
    stream = torch.cuda.current_stream().cuda_stream
    before = os.environ.get("TURBOFFT_FUSED")
    os.environ["TURBOFFT_FUSED"] = "1"
    try:
        for dt, logN in ((0, 16), (1, 15), (1, 16)):
            plan = turbofft_amd.TurboFFT(logN, dt)
            if plan.fused_info() is None:
                plan.close()
                continue
            bs = 1 << (28 - logN)
            x = make_input(torch, bs, 1 << logN, dt)
            out = torch.empty(2 << 28, dtype=torch.complex64 if dt == 0 else torch.complex128, device="cuda")
            ms = {True: [], False: []}
            names = {}
            for rnd in range(rounds):
                for fused in (True, False):
                    plan.set_fused(fused)
                    names[fused] = plan.kernel_names_for_batch(bs)
                    for _ in range(3):
                        plan.exec(x.data_ptr(), out.data_ptr(), bs, stream)
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(steps):
                        plan.exec(x.data_ptr(), out.data_ptr(), bs, stream)
                    e1.record()
                    torch.cuda.synchronize()
                    ms[fused].append(e0.elapsed_time(e1) / steps)
            f, t = stats(ms[True])["median"], stats(ms[False])["median"]
            row = {"logN": logN, "dtype": "f32" if dt == 0 else "f64", "bs": bs, "fused_kernel": names[True][0], "ms_fused": f, "ms_two_launches": t,
                   "two_launches_over_fused": t / f, "gbs_fused": plan.gbs(bs, f), "team": plan.fused_info() or None}
            plan.set_fused(True)
            row["team"] = plan.fused_info()
            plan.close()
            rows.append(row)
            if log:
                log(row)
            del x, out
            torch.cuda.empty_cache()
    finally:
        if before is None:
            del os.environ["TURBOFFT_FUSED"]
        else:
            os.environ["TURBOFFT_FUSED"] = before
    return rows


def cpu_baseline(logN, datatype, target_s=10.0):
    """Reference CPU path: pocketfft via scipy.fft on all host cores the box
    gives one GPU (16), on a bounded sample of the workload."""
    import numpy as np
    import scipy.fft
    from oracle import turbofft_oracle as O  # noqa: F401  (the oracle's FFT is numpy/pocketfft itself)
    N = 1 << logN
    cores = max(1, min(16, os.cpu_count() or 1))
    cdt = np.complex64 if datatype == 0 else np.complex128
    rng = np.random.default_rng(0)
    nb = max(1, (1 << 22) // N)                   # 4M points per call
    x = (rng.uniform(-1, 1, (nb, N)) + 1j * rng.uniform(-1, 1, (nb, N))).astype(cdt)
    scipy.fft.fft(x, axis=-1, workers=cores)      # warm-up
    t0 = time.perf_counter()
    calls = 0
    while True:
        scipy.fft.fft(x, axis=-1, workers=cores)
        calls += 1
        el = time.perf_counter() - t0
        if el >= target_s or calls >= 1000000:
            break
    pts = calls * nb * N
    esize = 8 if datatype == 0 else 16
    gbs = 2 * pts * esize / el / 1e9
    # the routine the accuracy oracle itself calls (numpy's pocketfft, one thread), for ~3 s
    np.fft.fft(x, axis=-1)
    t1 = time.perf_counter()
    calls1 = 0
    while True:
        np.fft.fft(x, axis=-1)
        calls1 += 1
        el1 = time.perf_counter() - t1
        if el1 >= min(3.0, target_s) or calls1 >= 1000000:
            break
    pts1 = calls1 * nb * N
    return {"value": gbs, "unit": "GB/s", "cores": cores, "kind": "port",
            "gflops": 5.0 * pts * logN / el / 1e9,
            "sample": f"scipy.fft.fft (pocketfft, workers={cores}) on {calls} x ({nb} x 2^{logN}) "
                      f"{'complex64' if datatype == 0 else 'complex128'} transforms, {el:.1f} s",
            "single_thread": {"value": 2 * pts1 * esize / el1 / 1e9, "unit": "GB/s", "cores": 1,
                              "gflops": 5.0 * pts1 * logN / el1 / 1e9,
                              "sample": f"numpy.fft.fft on {calls1} x ({nb} x 2^{logN}) transforms, {el1:.1f} s"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--logN", type=int, default=13)
    ap.add_argument("--datatype", type=int, default=0)
    ap.add_argument("--bs", type=int, default=0, help="default 2^(28-logN)")
    ap.add_argument("--if_ft", type=int, default=0)
    ap.add_argument("--if_err", type=int, default=0)
    ap.add_argument("--thread_bs", type=int, default=1)
    ap.add_argument("--param", type=str, default=None)
    ap.add_argument("--prewarm_s", type=float, default=1.0,
                    help="seconds of untimed executions before the warm-up steps (reported as prewarm_s)")
    ap.add_argument("--correct", type=int, default=None, help="with --if_err: 1 recompute, 2 delayed batch correction")
    ap.add_argument("--inj_every", type=int, default=0,
                    help="with --if_ft 1: inject into one tile of every N of the last launch (host-chosen cadence) and correct")
    ap.add_argument("--inj_mag", type=float, default=100.0, help="magnitude of the --inj_every injections")
    ap.add_argument("--no_cpu", action="store_true")
    ap.add_argument("--cpu_seconds", type=float, default=10.0)
    ap.add_argument("--sweep", action="store_true")
    ap.add_argument("--sweep_lo", type=int, default=7)
    ap.add_argument("--sweep_hi", type=int, default=24)
    ap.add_argument("--out", type=str, default=None)
    ap.add_argument("--no_ft_overhead", action="store_true",
                    help="skip the extra fault-tolerant run that reports the FT overhead of the workload")
    ap.add_argument("--no_vendor", action="store_true", help="skip the hipFFT side-by-side of the default line")
    ap.add_argument("--no_sweep", action="store_true", help="skip the logN 7..24 x {fp32, fp64} sweep of the default line")
    ap.add_argument("--sweep_steps", type=int, default=10, help="timed steps per case of the default line's sweep")
    ap.add_argument("--vendor", action="store_true", help="--sweep: run hipFFT after every case")
    ap.add_argument("--offline", action="store_true", help="--sweep: time the offline checksum scheme after every case")
    ap.add_argument("--membench", action="store_true",
                    help="time the streaming yardsticks (copy with 8- and 16-byte lanes, read only, write only) "
                         "on 2 GiB and print one JSON line")
    ap.add_argument("--membench_fused", type=str, default=None, metavar="G:R:B",
                    help="--membench: only the two-pass copy through a per-XCD ring of R slots of G 512 KiB pieces with B blocks per CU "
                         "(for counter runs of one configuration)")
    ap.add_argument("--membench_team", type=str, default=None, metavar="T:P:B",
                    help="--membench: only the two-pass copy with teams of T blocks that share a slot of P KiB, B blocks per CU")
    ap.add_argument("--fused_pairs", action="store_true", help="only the fused-pair comparison (one JSON line)")
    ap.add_argument("--calib_copy", type=int, default=0,
                    help="also run this many plain device copies of the input (a kernel of known traffic, "
                         "for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (batches shard trivially across "
              "GPUs by splitting the batch, no exchange needed). Run with --gpus 1.", file=sys.stderr)
        return 2
    import torch
    import turbofft_amd
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 1
    if a.membench:
        nbytes = 2 << 30
        src = torch.rand(nbytes // 4, device="cuda", dtype=torch.float32)
        dst = torch.empty(nbytes // 4, device="cuda", dtype=torch.float32)
        st = torch.cuda.current_stream().cuda_stream
        for _ in range(20):
            turbofft_amd.membench(0, src.data_ptr(), dst.data_ptr(), nbytes, 0, 10, st)      # clock the device up
        res = {}
        only_fused = [tuple(int(t) for t in a.membench_fused.split(":"))] if a.membench_fused else None
        only_team = [tuple(int(t) for t in a.membench_team.split(":"))] if a.membench_team else None
        if only_team:
            only_fused = []
        # every kernel plain, then with what the FFT kernels use: non-temporal accesses (+4), XCD-aware
        # tile order (+8) and a bound on the blocks resident per CU (+16*k; the exchange buffer of an
        # FFT kernel bounds it to 2-4)
        flavours = (("", 0), ("_nt", 4), ("_nt_xcd", 12), ("_nt_xcd_2percu", 12 + 32), ("_nt_xcd_3percu", 12 + 48), ("_nt_xcd_4percu", 12 + 64), ("_nt_xcd_6percu", 12 + 96))
        for kind, name, moved in ((0, "copy_8B_lanes", 2), (1, "copy_16B_lanes", 2), (2, "read_only", 1), (3, "write_only", 1)):
            if only_fused is not None:
                break
            for sfx, bits in flavours:
                ms = sorted(turbofft_amd.membench(kind + bits, src.data_ptr(), dst.data_ptr(), nbytes, 3, 20, st) for _ in range(5))
                res[name + sfx] = {"ms_per_pass_median": ms[2], "ms_min": ms[0], "ms_max": ms[4], "GB/s": moved * nbytes / ms[2] / 1e6}
                print(f"{name + sfx:32s} {ms[2]:.4f} ms  {moved * nbytes / ms[2] / 1e6:7.0f} GB/s", file=sys.stderr, flush=True)
        # the access patterns of the column kernels and of the transposed store: runs of 128-512 bytes at a large stride
        strided = {}
        for ls in (() if only_fused is not None else (12, 14, 16, 19)):
            for run in (128, 256, 512):
                for lane in (8, 16):
                    for write in (0, 1):
                        best = None
                        for xc in (4, 16, 64):
                            ms = sorted(turbofft_amd.membench_strided(write, lane, run, ls, xc, src.data_ptr(), dst.data_ptr(), nbytes, 3, 10, st) for _ in range(3))[1]
                            if best is None or ms < best[0]:
                                best = (ms, xc)
                        name = f"{'write' if write else 'read'}_run{run}_stride2^{ls}_{lane}B_lanes"
                        strided[name] = {"ms_per_pass": best[0], "GB/s": nbytes / best[0] / 1e6, "tiles_per_xcd_run": best[1]}
                        print(f"{name:40s} {best[0]:.4f} ms  {nbytes / best[0] / 1e6:7.0f} GB/s  (runs of {best[1]} tiles per XCD)", file=sys.stderr, flush=True)
        res["strided"] = strided
        # two passes through a ring meant to stay in the XCD's L2, against two whole passes
        scratch = torch.empty((8 * 3 * 8 * 512 * 1024) // 4, device="cuda", dtype=torch.float32)
        fused = {}
        two = sorted(turbofft_amd.membench(12, src.data_ptr(), dst.data_ptr(), nbytes, 3, 20, st) for _ in range(5))[2] * 2
        fused["two_whole_passes_ms"] = two
        for G, R, bpc in (only_fused if only_fused is not None else ((1, 3, 2), (2, 3, 2), (4, 2, 2), (4, 3, 2), (8, 3, 2), (8, 3, 3))):
            dst.zero_()
            ms, stt = turbofft_amd.membench_fused(G, R, bpc, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes, 50, 1, 5, st)
            ok = bool(torch.equal(src, dst))
            fused[f"group{G}_slots{R}_blocks{bpc}"] = {"ms": ms, "ring_KiB_per_xcd": G * R * 512, "copied_right": ok, **stt}
            print(f"fused copy: {G} x 512 KiB per group, {R} slots ({G * R * 512} KiB ring per XCD), {bpc} blocks per CU: {ms:.3f} ms "
                  f"(two whole passes {two:.3f} ms), right {ok}, {stt}", file=sys.stderr, flush=True)
        res["fused_two_pass_copy"] = fused
        # the same two passes with teams of blocks that share ONE slot each (the form the fused FFT kernels use)
        team = {}
        scratch = torch.empty((8 * 64 * 1024 * 1024) // 4, device="cuda", dtype=torch.float32)
        for T, P, bpc in (only_team or ((() if a.membench_fused else ((4, 256, 1), (4, 256, 2), (8, 512, 1), (8, 512, 2), (16, 512, 2), (8, 1024, 1), (16, 1024, 1), (16, 1024, 2))))):
            dst.zero_()
            ms, stt = turbofft_amd.membench_team(T, bpc, src.data_ptr(), scratch.data_ptr(), scratch.numel() * 4, dst.data_ptr(), nbytes, 50, 1, 5, st, piece_kib=P)
            ok = bool(torch.equal(src, dst))
            slots = (stt["blocks"] // 8) // T
            team[f"team{T}_piece{P}KiB_blocks{bpc}"] = {"ms": ms, "slots_KiB_per_xcd": slots * P, "copied_right": ok, **stt}
            print(f"team copy: teams of {T}, pieces of {P} KiB, {bpc} blocks per CU ({slots * P} KiB of slots per XCD): {ms:.3f} ms "
                  f"(two whole passes {two:.3f} ms), right {ok}, us per round {stt['us_per_round']}", file=sys.stderr, flush=True)
        res["team_two_pass_copy"] = team
        print(json.dumps({"membench": res, "bytes": nbytes, "tile_bytes": 65536, "threads": 256}), flush=True)
        return 0
    if a.fused_pairs:
        print(json.dumps({"fused_pairs": fused_pair_rows(torch, turbofft_amd, max(10, a.sweep_steps))}), flush=True)
        return 0
    if a.sweep:
        lines = []
        for dt in (0, 1):
            # one input of 2^28 points and one output of 2*2^28 (result + workspace of the
            # multi-launch plans) serve every logN of the sweep
            cdt = torch.complex64 if dt == 0 else torch.complex128
            x = make_input(torch, 1 << (28 - a.sweep_lo), 1 << a.sweep_lo, dt)
            out = torch.empty(2 << 28, dtype=cdt, device="cuda")
            for logN in range(a.sweep_lo, a.sweep_hi + 1):
                bs = 1 << (28 - logN)
                if x is not None:
                    x = x.view(-1).view(bs, 1 << logN)
                try:
                    r, x, out = run_case(torch, turbofft_amd, logN, dt, bs, a.steps, a.warmup, a.if_ft, a.if_err,
                                         a.thread_bs, a.param, x, out, prewarm_s=min(a.prewarm_s, 0.2), correct=a.correct)
                except turbofft_amd.TurboFFTError as e:
                    # a plan row without a compiled kernel must not stop the sweep; anything
                    # that comes from the device does
                    if "no compiled kernel" not in str(e) and "no plan row" not in str(e):
                        raise
                    r = {"logN": logN, "datatype": dt, "error": str(e)}
                if "gbs" in r:
                    r["frac_hbm"] = r["gbs"] / HBM_PEAK_GBS
                    print(f"{'fp32' if dt == 0 else 'fp64'} logN={logN:2d} L={r['launches']} "
                          f"{r['wall_ms']:8.3f} ms (min {r['step_ms']['min']:.3f}) {r['gflops']:9.1f} GFLOPS {r['gbs']:8.1f} GB/s  "
                          f"{100 * r['frac_hbm']:5.1f}% of HBM peak  {r['plan']}"
                          + (f"  ft per exec: " + " ".join(f"{k} {v // r['ft']['execs']}" for k, v in r["ft"].items() if k != "execs")
                             if "ft" in r else ""), flush=True)
                else:
                    print(r, flush=True)
                if a.offline and "gbs" in r:
                    oms, oflag = turbofft_amd.offline_ft_time(logN, dt, x.data_ptr(), out.data_ptr(), bs, 2, max(5, a.steps // 4),
                                                              torch.cuda.current_stream().cuda_stream)
                    r["offline_ft"] = {"ms_per_step": oms, "flagged": oflag, "overhead_pct": 100.0 * (oms / r["event_ms"] - 1.0)}
                    print(f"     offline FT  {oms:8.3f} ms  +{r['offline_ft']['overhead_pct']:.1f} % over the plain plan, {oflag} flagged", flush=True)
                if a.vendor and "gbs" in r:
                    v = vendor_case(torch, turbofft_amd, logN, dt, bs, x, out, reps=max(5, a.steps // 4))
                    r["vendor"] = v
                    if "value" in v:
                        print(f"     hipFFT      {v['ms_per_step']:8.3f} ms {v['gflops']:9.1f} GFLOPS {v['value']:8.1f} GB/s  "
                              f"this library / hipFFT = {r['gbs'] / v['value']:.2f}", flush=True)
                    else:
                        print(f"     hipFFT      {v['error']}", flush=True)
                lines.append(r)
            del x, out
            torch.cuda.empty_cache()
        if a.out:
            with open(a.out, "w") as f:
                for r in lines:
                    f.write(json.dumps(r) + "\n")
        return 0

    logN, dt = a.logN, a.datatype
    bs = a.bs or (1 << (28 - logN))
    r, x, out = run_case(torch, turbofft_amd, logN, dt, bs, a.steps, a.warmup, a.if_ft, a.if_err, a.thread_bs, a.param,
                         prewarm_s=a.prewarm_s, correct=a.correct, inj_every=a.inj_every, inj_mag=a.inj_mag)
    for _ in range(a.calib_copy):
        out.view(-1)[: x.numel()].copy_(x.view(-1))          # reads and writes x.numel()*sizeof(T) bytes
    torch.cuda.synchronize()
    ft_line = None
    if not (a.if_ft or a.if_err) and not a.no_ft_overhead:
        # the second half of the headline metric: the same workload with the fused checksums
        # (4 tiles per checksum group, no error injected), outside the timed region above
        ft_line = interleaved_overhead(torch, turbofft_amd, logN, dt, bs, x, out, a.param)
        # the same with the group size of the reference's published runs (compile.sh:13): 32 tiles,
        # which this library walks with several blocks per group
        g32 = interleaved_overhead(torch, turbofft_amd, logN, dt, bs, x, out, a.param, thread_bs=32, rounds=4)
        ft_line["groups_of_32"] = {"overhead_pct": g32["overhead_pct"], "ms_per_step": g32["ms_per_step"], "order": g32["order"]}
        # the same groups of 4 with the reference's complex checksum table in every launch (this build's
        # compact form switched off): what the fused scheme costs on the reference's own arithmetic
        if any(n.endswith(("_h_ft", "_h2_ft", "_h3_ft")) for n in ft_line["plan"]["kernels"]):
            full = interleaved_overhead(torch, turbofft_amd, logN, dt, bs, x, out, a.param, thread_bs=4, rounds=4, compact=False)
            ft_line["full_table"] = {"overhead_pct": full["overhead_pct"], "ms_per_step": full["ms_per_step"], "order": full["order"],
                                     "kernels": full["plan"]["kernels"]}
        else:
            ft_line["full_table"] = {"overhead_pct": ft_line["overhead_pct"], "ms_per_step": ft_line["ms_per_step"],
                                     "note": "this size's fault-tolerant kernels read the full table by default"}
        ft_line["table"] = "compact" if "kernels" in ft_line["full_table"] else "full"
        # thread-level verification of the same workload: every thread checks its own register-level DFTs,
        # every tile is decided before it is stored (no groups)
        tl = interleaved_overhead(torch, turbofft_amd, logN, dt, bs, x, out, a.param, thread_bs=1, rounds=4, scheme=2)
        ft_line["thread_level"] = {"overhead_pct": tl["overhead_pct"], "ms_per_step": tl["ms_per_step"], "order": tl["order"],
                                   "kernels": tl["plan"]["kernels"], "counters": tl["counters"]}
        # the offline scheme on the same workload: checksum pass, plain plan, checksum pass, compare
        try:
            oms, oflag = turbofft_amd.offline_ft_time(logN, dt, x.data_ptr(), out.data_ptr(), bs, 2, max(10, a.steps // 10),
                                                      torch.cuda.current_stream().cuda_stream)
            ft_line["offline"] = {"overhead_pct": 100.0 * (oms / ft_line["plain_ms"]["median"] - 1.0), "ms_per_step": oms, "flagged": oflag}
        except turbofft_amd.TurboFFTError as e:
            ft_line["offline"] = {"error": str(e)}
    sync_ms = None
    if not (a.if_ft or a.if_err):
        # the reference's own timing protocol beside the default one: a host wait after every launch
        pl = turbofft_amd.TurboFFT(logN, dt, param_csv=a.param)
        sync_ms = pl.time_sync(x.data_ptr(), out.data_ptr(), bs, 2, max(10, a.steps // 4), torch.cuda.current_stream().cuda_stream)
        pl.close()
    vendor_line = None
    if not a.no_vendor:
        vendor_line = vendor_case(torch, turbofft_amd, logN, dt, bs, x, out, reps=max(10, a.steps // 10))
    del x, out
    torch.cuda.empty_cache()
    sweep = None
    fused_pairs = None
    if not a.no_sweep and not (a.if_ft or a.if_err):
        t_sw = time.perf_counter()
        sweep = sweep_rows(torch, turbofft_amd, a.sweep_lo, a.sweep_hi, max(10, a.sweep_steps))
        fused_pairs = fused_pair_rows(torch, turbofft_amd, max(10, a.sweep_steps))
        sweep_s = time.perf_counter() - t_sw
    tname = "fp32" if dt == 0 else "fp64"
    launches = r["launches"]
    # dominant kernel: with one launch it is the whole step; with several, the launches are
    # equal-traffic passes and the per-launch average is event time / launches
    kernel_ms = r["event_ms"] / launches
    achieved = r["alg_bytes"] / (kernel_ms * 1e-3) / 1e9
    line = {
        "metric": "batched C2C FFT algorithmic HBM GB/s (2*N*bs*sizeof(T)/t) at logBS+logN=28",
        "value": r["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": r["wall_ms"], "step_ms": r["step_ms"], "prewarm_s": r["prewarm_s"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if dt == 0 else "f64", "data": "synthetic",
        "gflops": r["gflops"],
        "config": {"workload": f"forward C2C FFT {tname} N=2^{logN} batch=2^{int(math.log2(bs))} "
                               f"({launches}-launch plan {r['plan']['logNi']}, BS {r['plan']['BS']}, n {r['plan']['n']})"
                               + (", fault tolerant" if (a.if_ft or a.if_err) else ""),
                   "logN": logN, "bs": bs, "if_ft": a.if_ft, "if_err": a.if_err, "thread_bs": a.thread_bs,
                   "inj_every": a.inj_every, "inj_mag": a.inj_mag if a.inj_every else None},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC.get((dt, logN, bs, int(bool(a.if_ft or a.if_err)))),
                     "traffic_source": "constant from the rocprofv3 FETCH_SIZE/WRITE_SIZE runs listed in profiles/, not measured in this run",
                     "kernel_ms": kernel_ms, "alg_bytes_per_launch": r["alg_bytes"]},
    }
    if sweep is not None:
        line["sweep"] = sweep
        line["fused_pairs"] = fused_pairs         # opt-in kernels (TURBOFFT_FUSED=1): both launches of a two-launch plan in one
        line["sweep_s"] = sweep_s
    if sync_ms is not None:
        line["ms_per_step_sync_each_launch"] = sync_ms          # main.cu:53-62 protocol, reported only
    if a.if_ft or a.if_err:
        line["ft"] = r.get("ft")
    if ft_line is not None:
        line["ft_overhead"] = ft_line
    if vendor_line is not None:
        line["vendor_baseline"] = vendor_line
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(logN, dt, a.cpu_seconds)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
