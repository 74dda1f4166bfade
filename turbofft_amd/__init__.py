"""turbofft_amd -- ctypes binding of libturbofft_hip.so (MI355X / gfx950).

The reference has no Python binding (its test.py only prints dispatch
tables); this module exposes the C ABI of include/turbofft.h with the
reference's vocabulary: logN, bs, datatype (0 = float2, 1 = double2), if_ft,
if_err, thread_bs -- the options of its `turbofft` command line
(include/utils/CommandLineParser.h:26-45).

There is no CPU fallback: if the HIP library is missing, importing the plan
class works but creating a plan raises, and every transform runs the
generated gfx950 kernels.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libturbofft_hip.so")
CLI_PATH = os.path.join(_HERE, "bin", "turbofft")

FP32, FP64 = 0, 1
STATIC_WORKSPACE_BYTES = 64 << 20      # TURBOFFT_STATIC_WORKSPACE_BYTES of include/turbofft.h
_lib = None


class TurboFFTError(RuntimeError):
    pass


def _datatype(dt) -> int:
    if dt in (0, "float2", "fp32", "f32", np.complex64):
        return FP32
    if dt in (1, "double2", "fp64", "f64", np.complex128):
        return FP64
    raise ValueError(f"datatype must be 0/float2 or 1/double2, got {dt!r}")


def lib() -> C.CDLL:
    """Load libturbofft_hip.so (built by turbofft_amd/build.py).  Fails loudly."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise TurboFFTError(f"{LIB_PATH} is missing: run `python turbofft_amd/build.py` (there is no CPU fallback)")
    try:
        # PyTorch ships its own HIP runtime; when both live in one process it has to
        # be the one that is loaded first, or torch.cuda stops seeing the device.
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    vp, ll, i = C.c_void_p, C.c_longlong, C.c_int
    L.turbofft_last_error.restype = C.c_char_p
    L.turbofft_plan_create.restype = vp
    L.turbofft_plan_create.argtypes = [i, i, i, i, i, C.c_char_p]
    L.turbofft_plan_destroy.argtypes = [vp]
    L.turbofft_plan_destroy.restype = None
    L.turbofft_exec.argtypes = [vp, vp, vp, ll, vp]
    L.turbofft_exec_inverse.argtypes = [vp, vp, vp, ll, vp]
    L.turbofft_exec_static.argtypes = [vp, vp, vp, ll, vp]
    L.turbofft_exec_host.argtypes = [vp, vp, vp, ll]
    L.turbofft_time.argtypes = [vp, vp, vp, ll, i, i, vp, C.POINTER(C.c_float)]
    L.turbofft_time_sync.argtypes = [vp, vp, vp, ll, i, i, vp, C.POINTER(C.c_float)]
    L.turbofft_set_checksum_mode.argtypes = [vp, i]
    L.turbofft_time_launches.argtypes = [vp, vp, vp, ll, i, i, vp, C.POINTER(C.c_float)]
    L.turbofft_plan_info.argtypes = [vp, C.POINTER(i), C.POINTER(i), C.POINTER(i), C.POINTER(i),
                                     C.POINTER(C.c_size_t), C.POINTER(i)]
    L.turbofft_plan_grid.argtypes = [vp, i, ll]
    L.turbofft_plan_grid.restype = ll
    L.turbofft_plan_small_batch_max.argtypes = [vp]
    L.turbofft_plan_small_batch_max.restype = ll
    L.turbofft_plan_set_small_batch.argtypes = [vp, i]
    L.turbofft_plan_set_fused.argtypes = [vp, i]
    L.turbofft_plan_fused_info.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.turbofft_plan_kernel_name.argtypes = [vp, i]
    L.turbofft_plan_kernel_name.restype = C.c_char_p
    L.turbofft_plan_launches_for_batch.argtypes = [vp, ll]
    L.turbofft_plan_kernel_name_for_batch.argtypes = [vp, i, ll]
    L.turbofft_plan_kernel_name_for_batch.restype = C.c_char_p
    L.turbofft_plan_tb_gap.argtypes = [vp, i]
    L.turbofft_plan_set_tb_gap.argtypes = [vp, i, i]
    L.turbofft_plan_set_ft_part_len.argtypes = [vp, i, i]
    L.turbofft_plan_ft_part_len.argtypes = [vp, i]
    L.turbofft_set_ft_params.argtypes = [vp, C.c_double, C.c_double, i]
    L.turbofft_set_injection.argtypes = [vp, i, i, i, ll, i, i, C.c_double]
    L.turbofft_get_ft_counters.argtypes = [vp] + [C.POINTER(C.c_ulonglong)] * 4 + [C.POINTER(ll), i, C.POINTER(i)]
    L.turbofft_reset_ft_counters.argtypes = [vp]
    L.turbofft_build_twiddle_table.argtypes = [i, ll, vp]
    L.turbofft_build_checksum_vector.argtypes = [i, ll, i, vp]
    L.turbofft_builtin_plan_row.argtypes = [i, i, C.POINTER(i)]
    L.turbofft_kernel_name.restype = C.c_char_p
    L.turbofft_kernel_name.argtypes = [i]
    L.turbofft_main.argtypes = [i, C.POINTER(C.c_char_p)]
    L.turbofft_vendor_exec.argtypes = [i, i, vp, vp, ll, vp]
    L.turbofft_vendor_time.argtypes = [i, i, vp, vp, ll, i, i, vp, C.POINTER(C.c_float)]
    L.turbofft_membench.argtypes = [i, vp, vp, C.c_size_t, i, i, vp, C.POINTER(C.c_float)]
    L.turbofft_membench_strided.argtypes = [i, i, i, i, i, vp, vp, C.c_size_t, i, i, vp, C.POINTER(C.c_float)]
    L.turbofft_membench_fused.argtypes = [i, i, i, i, vp, vp, C.c_size_t, vp, C.c_size_t, i, i, i, vp, C.POINTER(C.c_float), C.POINTER(C.c_uint)]
    L.turbofft_membench_team.argtypes = [i, i, i, i, vp, vp, C.c_size_t, vp, C.c_size_t, i, i, i, vp, C.POINTER(C.c_float), C.POINTER(C.c_uint)]
    L.turbofft_offline_checksums.argtypes = [i, i, vp, vp, ll, vp, vp, vp]
    L.turbofft_offline_ft_time.argtypes = [i, i, vp, vp, ll, i, i, vp, C.POINTER(C.c_float), C.POINTER(C.c_ulonglong)]
    _lib = L
    return L


def _check(rc: int):
    if rc != 0:
        raise TurboFFTError(lib().turbofft_last_error().decode() or f"turbofft error {rc}")


# ---- host tables (no GPU needed) ------------------------------------------
def twiddle_table(N: int, datatype) -> np.ndarray:
    dt = _datatype(datatype)
    out = np.empty(2 * N - 1, dtype=np.complex64 if dt == FP32 else np.complex128)
    _check(lib().turbofft_build_twiddle_table(dt, N, out.ctypes.data))
    return out


def checksum_vector(N: int, datatype, mode: str = "exact") -> np.ndarray:
    dt = _datatype(datatype)
    out = np.empty(N, dtype=np.complex64 if dt == FP32 else np.complex128)
    _check(lib().turbofft_build_checksum_vector(dt, N, {"exact": 0, "reference": 1}[mode], out.ctypes.data))
    return out


def builtin_plan_row(datatype, logN: int) -> List[int]:
    row = (C.c_int * 11)()
    _check(lib().turbofft_builtin_plan_row(_datatype(datatype), logN, row))
    return list(row)


def kernel_names() -> List[str]:
    L = lib()
    return [L.turbofft_kernel_name(i).decode() for i in range(L.turbofft_kernel_count())]


# ---- vendor-library side-by-side (hipFFT; the role of cufft/cufft.h in the reference) ----
def vendor_available() -> bool:
    return bool(lib().turbofft_vendor_available())


def vendor_fft(x, out=None):
    """hipFFT forward transform of a (bs, N) complex tensor on the GPU; measurement and
    cross-check only (main.cu:99-101 compares the reference's result with cuFFT's)."""
    import torch
    if x.dim() != 2 or not x.is_cuda or not x.is_contiguous() or x.dtype not in (torch.complex64, torch.complex128):
        raise ValueError("expected a contiguous complex64/complex128 tensor of shape (bs, N) on the GPU")
    bs, N = x.shape
    logN = N.bit_length() - 1
    if N != 1 << logN:
        raise ValueError("N must be a power of two")
    if out is None:
        out = torch.empty_like(x)
    _check(lib().turbofft_vendor_exec(logN, FP32 if x.dtype == torch.complex64 else FP64, x.data_ptr(), out.data_ptr(), bs,
                                      torch.cuda.current_stream(x.device).cuda_stream))
    return out


def vendor_time(logN: int, datatype, in_ptr: int, out_ptr: int, bs: int, warmup: int = 1, reps: int = 10, stream: int = 0) -> float:
    ms = C.c_float(0)
    _check(lib().turbofft_vendor_time(logN, _datatype(datatype), in_ptr, out_ptr, bs, warmup, reps, stream, C.byref(ms)))
    return ms.value


# ---- offline checksums (the baseline of cufft/cufft_ft.h: separate passes around the transform) ----
def offline_checksums(x, y):
    """Per-transform input and output checksums of x -> y (both (bs, N) complex tensors on the
    GPU), computed by two separate passes; returns two real tensors of length bs."""
    import torch
    if x.shape != y.shape or x.dim() != 2 or x.dtype != y.dtype or not (x.is_cuda and y.is_cuda) or \
            not (x.is_contiguous() and y.is_contiguous()) or x.dtype not in (torch.complex64, torch.complex128):
        raise ValueError("expected two contiguous complex tensors of the same (bs, N) shape on the GPU")
    bs, N = x.shape
    logN = N.bit_length() - 1
    if N != 1 << logN:
        raise ValueError("N must be a power of two")
    rdt = torch.float32 if x.dtype == torch.complex64 else torch.float64
    a = torch.empty(bs, dtype=rdt, device=x.device)
    b = torch.empty(bs, dtype=rdt, device=x.device)
    _check(lib().turbofft_offline_checksums(logN, FP32 if rdt == torch.float32 else FP64, x.data_ptr(), y.data_ptr(), bs,
                                            a.data_ptr(), b.data_ptr(), torch.cuda.current_stream(x.device).cuda_stream))
    return a, b


def offline_ft_time(logN: int, datatype, in_ptr: int, out_ptr: int, bs: int, warmup: int = 1, reps: int = 10, stream: int = 0):
    """(ms per execution, transforms flagged in the last one) of checksum pass + plain plan + checksum pass + compare."""
    ms = C.c_float(0)
    flagged = C.c_ulonglong(0)
    _check(lib().turbofft_offline_ft_time(logN, _datatype(datatype), in_ptr, out_ptr, bs, warmup, reps, stream,
                                          C.byref(ms), C.byref(flagged)))
    return ms.value, flagged.value


def membench_strided(write: bool, lane_bytes: int, run_bytes: int, log_stride: int, xcd_chunk: int, src_ptr: int, dst_ptr: int,
                     nbytes: int, warmup: int = 2, reps: int = 10, stream: int = 0) -> float:
    """ms per read-only or write-only pass over 64 KiB tiles made of `run_bytes` runs at a stride of 2^log_stride bytes."""
    ms = C.c_float(0)
    _check(lib().turbofft_membench_strided(int(bool(write)), lane_bytes, run_bytes, log_stride, xcd_chunk, src_ptr, dst_ptr, nbytes,
                                           warmup, reps, stream, C.byref(ms)))
    return ms.value


def membench_fused(group: int, ring_slots: int, blocks_per_cu: int, src_ptr: int, scratch_ptr: int, scratch_bytes: int, dst_ptr: int,
                   nbytes: int, limit_ms: int = 50, warmup: int = 1, reps: int = 5, stream: int = 0, lag: int = 1):
    """Two-pass copy through a per-XCD ring as one persistent kernel: (ms per launch, stats dict)."""
    ms = C.c_float(0)
    st = (C.c_uint * 12)()
    _check(lib().turbofft_membench_fused(group, ring_slots, lag, blocks_per_cu, src_ptr, scratch_ptr, scratch_bytes, dst_ptr, nbytes, limit_ms,
                                         warmup, reps, stream, C.byref(ms), st))
    return ms.value, {"timed_out": st[0], "waits": st[1], "polls": st[2], "blocks": st[3], "blocks_per_xcd": list(st)[4:12]}


def membench_team(team_blocks: int, blocks_per_cu: int, src_ptr: int, scratch_ptr: int, scratch_bytes: int, dst_ptr: int, nbytes: int,
                  limit_ms: int = 50, warmup: int = 1, reps: int = 5, stream: int = 0, piece_kib: int = 512, policy: int = 0):
    """Two-pass copy through one L2-resident slot per team of blocks: (ms per launch, stats dict).  stats["us_per_round"]
    is the mean time a block spends per round in: waiting for the piece's loads, waiting for the slot, the slot's stores,
    the team barrier, the slot's loads, the rest."""
    ms = C.c_float(0)
    st = (C.c_uint * 12)()
    _check(lib().turbofft_membench_team(team_blocks, piece_kib, policy, blocks_per_cu, src_ptr, scratch_ptr, scratch_bytes, dst_ptr, nbytes, limit_ms,
                                        warmup, reps, stream, C.byref(ms), st))
    return ms.value, {"timed_out": st[0], "waits": st[1], "polls": st[2], "blocks": st[3], "us_per_round": [v / 100.0 for v in list(st)[4:10]],
                      "rounds_per_block": st[10]}


def membench(mode: int, src_ptr: int, dst_ptr: int, nbytes: int, warmup: int = 2, reps: int = 10, stream: int = 0) -> float:
    """ms per pass of a streaming kernel of known traffic: 0 copy with 8-byte lanes, 1 copy with
    16-byte lanes, 2 read only, 3 write only; +4 non-temporal accesses, +8 XCD-aware tile order,
    +16*k at most k blocks per CU (measurement yardsticks, not part of any transform)."""
    ms = C.c_float(0)
    _check(lib().turbofft_membench(mode, src_ptr, dst_ptr, nbytes, warmup, reps, stream, C.byref(ms)))
    return ms.value


def turbofft_main(argv: List[str]) -> int:
    """Run the `turbofft` command line in-process."""
    args = [b"turbofft"] + [a.encode() for a in argv]
    arr = (C.c_char_p * len(args))(*args)
    return lib().turbofft_main(len(args), arr)


class TurboFFT:
    """A plan for `bs` forward C2C transforms of length 2^logN."""

    def __init__(self, logN: int, datatype=FP32, if_ft: int = 0, if_err: int = 0, thread_bs: int = 1,
                 param_csv: Optional[str] = None):
        self.logN = int(logN)
        self.N = 1 << self.logN
        self.datatype = _datatype(datatype)
        self.cdtype = np.complex64 if self.datatype == FP32 else np.complex128
        # if_ft: 1 checksums per group of thread_bs tiles, 2 thread-level verification (every tile on its own)
        self.if_ft = int(if_ft) if int(if_ft) in (1, 2) else int(bool(if_ft or if_err))
        self.if_err = int(bool(if_err))
        self.thread_bs = int(thread_bs)
        self._h = lib().turbofft_plan_create(self.logN, self.datatype, self.if_ft, self.if_err, self.thread_bs,
                                             param_csv.encode() if param_csv else None)
        if not self._h:
            raise TurboFFTError(lib().turbofft_last_error().decode())
        i3 = (C.c_int * 3)
        n = C.c_int()
        a, b, c, t = i3(), i3(), i3(), i3()
        lds = (C.c_size_t * 3)()
        _check(lib().turbofft_plan_info(self._h, C.byref(n), a, b, c, lds, t))
        self.launches = n.value
        self.logNi, self.BS, self.n = list(a)[:n.value], list(b)[:n.value], list(c)[:n.value]
        self.lds_bytes, self.threads = list(lds)[:n.value], list(t)[:n.value]

    def close(self):
        if getattr(self, "_h", None):
            if lib is not None:                     # (module globals are gone at interpreter shutdown)
                lib().turbofft_plan_destroy(self._h)
            self._h = None

    __del__ = close

    # ---- geometry ----
    def plan_row(self) -> List[int]:
        """The 11 reference columns of the row this plan runs (a fault-tolerant plan may use
        another built-in row than the plain plan of the same size)."""
        z = lambda v: list(v) + [0] * (3 - len(v))
        return [self.logN, self.launches] + z(self.logNi) + z(self.BS) + z(self.n)

    def out_elems(self, bs: int) -> int:
        """Elements the output buffer must hold (workspace included)."""
        return self.N * bs * (2 if self.launches > 1 else 1)

    def grid(self, launch: int, bs: int) -> int:
        return lib().turbofft_plan_grid(self._h, launch, bs)

    def small_batch_max(self) -> int:
        """Largest batch that runs the narrow-tile row of the small-batch table (0: none)."""
        return lib().turbofft_plan_small_batch_max(self._h)

    def set_small_batch(self, enable: bool):
        _check(lib().turbofft_plan_set_small_batch(self._h, int(bool(enable))))

    def set_fused(self, enable: bool):
        """Switch the plan's fused kernel (both launches of a two-launch plan in one) off or on."""
        _check(lib().turbofft_plan_set_fused(self._h, int(bool(enable))))

    def fused_info(self):
        """None when the plan holds no enabled fused kernel, else a dict with its team size, transforms per piece,
        teams per XCD and grid."""
        v = [C.c_int(0) for _ in range(4)]
        rc = lib().turbofft_plan_fused_info(self._h, *[C.byref(x) for x in v])
        if rc < 0:
            _check(rc)
        if rc == 0:
            return None
        return {"team_blocks": v[0].value, "transforms_per_piece": v[1].value, "teams_per_xcd": v[2].value, "grid_blocks": v[3].value}

    def kernel_names(self) -> List[str]:
        """Kernels the launches of a forward execution run with the current settings."""
        return [(lib().turbofft_plan_kernel_name(self._h, i) or b"").decode() for i in range(self.launches)]

    def kernel_names_for_batch(self, bs: int) -> List[str]:
        """Kernels a batch of `bs` transforms runs: the small-batch row's up to its cap, else the plan's own."""
        n = lib().turbofft_plan_launches_for_batch(self._h, bs)
        _check(min(n, 0))
        return [(lib().turbofft_plan_kernel_name_for_batch(self._h, i, bs) or b"").decode() for i in range(n)]

    def tb_gap(self, launch: int) -> int:
        return lib().turbofft_plan_tb_gap(self._h, launch)

    def set_tb_gap(self, launch: int, gap: int):
        _check(lib().turbofft_plan_set_tb_gap(self._h, launch, gap))

    def ft_part_len(self, launch: int) -> int:
        """Tiles of a checksum group one block walks (0: the whole group)."""
        return lib().turbofft_plan_ft_part_len(self._h, launch)

    def set_ft_part_len(self, launch: int, tiles: int):
        _check(lib().turbofft_plan_set_ft_part_len(self._h, launch, tiles))

    # ---- execution ----
    def exec(self, in_ptr: int, out_ptr: int, bs: int, stream: int = 0):
        _check(lib().turbofft_exec(self._h, in_ptr, out_ptr, bs, stream))

    def exec_static(self, in_ptr: int, out_ptr: int, bs: int, stream: int = 0):
        """turbofft_exec with an N*bs output buffer: the intermediate of a multi-launch plan goes to
        the library's static device workspace (STATIC_WORKSPACE_BYTES per GPU); allocates nothing."""
        _check(lib().turbofft_exec_static(self._h, in_ptr, out_ptr, bs, stream))

    def exec_inverse(self, in_ptr: int, out_ptr: int, bs: int, stream: int = 0):
        _check(lib().turbofft_exec_inverse(self._h, in_ptr, out_ptr, bs, stream))

    def ifft(self, x, out=None):
        """Unnormalised inverse transform (N times numpy's ifft); arguments as for fft()."""
        return self.fft(x, out, _inverse=True)

    def fft(self, x, out=None, _inverse=False):
        """x: torch tensor on the GPU, shape (bs, N), complex64/complex128.
        Returns a (bs, N) view of the transform (natural order)."""
        import torch
        if x.dim() != 2 or x.shape[1] != self.N:
            raise ValueError(f"expected shape (bs, {self.N}), got {tuple(x.shape)}")
        want = torch.complex64 if self.datatype == FP32 else torch.complex128
        if x.dtype != want or not x.is_cuda or not x.is_contiguous():
            raise ValueError(f"expected a contiguous {want} tensor on the GPU")
        bs = x.shape[0]
        if out is None:
            out = torch.empty(self.out_elems(bs), dtype=want, device=x.device)
        elif out.numel() < self.out_elems(bs) or out.dtype != want or not out.is_contiguous():
            raise ValueError(f"out must be contiguous {want} with >= {self.out_elems(bs)} elements")
        (self.exec_inverse if _inverse else self.exec)(x.data_ptr(), out.data_ptr(), bs, torch.cuda.current_stream(x.device).cuda_stream)
        return out.view(-1)[: bs * self.N].view(bs, self.N)

    def exec_host(self, in_ptr: int, out_ptr: int, bs: int):
        """turbofft_exec_host on raw host addresses (N*bs elements each; page-locked buffers let the
        copies in, the kernels and the copies out overlap)."""
        _check(lib().turbofft_exec_host(self._h, in_ptr, out_ptr, bs))

    def fft_host(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=self.cdtype)
        if x.ndim != 2 or x.shape[1] != self.N:
            raise ValueError(f"expected shape (bs, {self.N}), got {x.shape}")
        out = np.empty_like(x)
        self.exec_host(x.ctypes.data, out.ctypes.data, x.shape[0])
        return out

    def time(self, in_ptr: int, out_ptr: int, bs: int, warmup: int = 1, reps: int = 10, stream: int = 0) -> float:
        ms = C.c_float()
        _check(lib().turbofft_time(self._h, in_ptr, out_ptr, bs, warmup, reps, stream, C.byref(ms)))
        return ms.value

    def time_sync(self, in_ptr: int, out_ptr: int, bs: int, warmup: int = 1, reps: int = 10, stream: int = 0) -> float:
        """The reference's timing protocol: the host waits after every launch (main.cu:53-62)."""
        ms = C.c_float()
        _check(lib().turbofft_time_sync(self._h, in_ptr, out_ptr, bs, warmup, reps, stream, C.byref(ms)))
        return ms.value

    def time_launches(self, in_ptr: int, out_ptr: int, bs: int, warmup: int = 1, reps: int = 10, stream: int = 0):
        """Mean duration of every launch of the plan (HIP events around each launch)."""
        ms = (C.c_float * 3)()
        _check(lib().turbofft_time_launches(self._h, in_ptr, out_ptr, bs, warmup, reps, stream, ms))
        return list(ms)[: self.launches]

    # ---- fault tolerance ----
    def set_ft_params(self, err_smoothing: float = 1000.0, err_threshold: float = 1e-3, correct=True):
        """correct: 0/False detect only, 1/True recompute the located tile, 2 delayed batch correction."""
        _check(lib().turbofft_set_ft_params(self._h, err_smoothing, err_threshold, int(correct)))

    def set_checksum_mode(self, mode: str):
        """"exact" (default) or "reference": the reference's float-rounded-angle table (abft.h:21-61)."""
        _check(lib().turbofft_set_checksum_mode(self._h, {"exact": 0, "reference": 1}[mode]))

    def set_injection(self, mode: int, launch: int = -1, every: int = 1, tile_phase: int = 0, s: int = 0, m: int = 0,
                      mag: float = 100.0):
        _check(lib().turbofft_set_injection(self._h, mode, launch, every, tile_phase, s, m, mag))

    def reset_ft_counters(self):
        _check(lib().turbofft_reset_ft_counters(self._h))

    def ft_counters(self, cap: int = 4096) -> dict:
        v = [C.c_ulonglong() for _ in range(4)]
        fl = (C.c_longlong * (2 * cap))()
        n = C.c_int()
        _check(lib().turbofft_get_ft_counters(self._h, *[C.byref(t) for t in v], fl, cap, C.byref(n)))
        flagged = [(fl[2 * i], fl[2 * i + 1]) for i in range(n.value)]
        return {"checked": v[0].value, "detected": v[1].value, "corrected": v[2].value,
                "uncorrectable": v[3].value, "flagged": flagged, "flagged_truncated": v[1].value > n.value}

    # ---- metrics (main.cu:68-69) ----
    def gflops(self, bs: int, ms: float) -> float:
        return 5.0 * self.N * self.logN * bs / ms * 1000 / 1e9

    def algorithmic_bytes(self, bs: int) -> int:
        return 2 * self.N * bs * (8 if self.datatype == FP32 else 16)

    def gbs(self, bs: int, ms: float) -> float:
        return self.algorithmic_bytes(bs) / ms * 1000 / 1e9
