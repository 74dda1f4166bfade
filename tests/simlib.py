"""Test helper: build and run the CPU lock-step flavour of generated kernels.

The generator prints every kernel as barrier-separated phases; with
-DTFFT_SIM the same text runs on the CPU, one phase for all threads at a
time, with bounds-checked accessors.  This validates the generator's index
algebra, LDS layouts and barrier placement here, where there is no GPU.
"""
import ctypes as C
import hashlib
import os
import subprocess
import tempfile

import numpy as np

from turbofft_amd.codegen.fft_codegen import KernelSpec, generate_source
from turbofft_amd.codegen.plan import KernelKey

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_CACHE = os.path.join(tempfile.gettempdir(), "tfft_sim_cache")


class FtArgs(C.Structure):
    _fields_ = [("cksum", C.c_void_p), ("counters", C.c_void_p), ("flagged", C.c_void_p),
                ("flagged_cap", C.c_int), ("launch", C.c_int), ("correct", C.c_int),
                ("inj_mode", C.c_int), ("inj_every", C.c_int), ("inj_tile", C.c_longlong),
                ("inj_s", C.c_int), ("inj_m", C.c_int), ("inj_mag", C.c_double),
                ("err_smoothing", C.c_double), ("err_threshold", C.c_double),
                ("parts", C.c_int), ("part_len", C.c_int), ("part_sums", C.c_void_p), ("tickets", C.c_void_p),
                ("fix_list", C.c_void_p), ("fix_ctl", C.c_void_p), ("fix_mode", C.c_int)]


class KArgs(C.Structure):
    _fields_ = [("ntiles", C.c_longlong), ("nrows", C.c_longlong), ("thread_bs", C.c_int),
                ("tb_gap", C.c_int), ("log_ncols", C.c_int), ("logQ", C.c_int), ("logC", C.c_int),
                ("logN", C.c_int), ("tw_lo_bits", C.c_int), ("xcd_chunk", C.c_int),
                ("tw_hi", C.c_void_p), ("tw_lo", C.c_void_p), ("ft", FtArgs)]


FT_SUB0, FT_SUB_STRIDE, FT_COUNTER_WORDS = 16, 16, 16 + 64 * 16      # include/turbofft_kargs.h


class FtState:
    """Counter block and flagged list of a fault-tolerant launch, laid out as the kernels expect
    (64 sub-counter lines, each owning a 64th of the list), and the totals the library derives."""

    def __init__(self, kargs, cap=512):
        assert cap % 64 == 0
        self.counters = np.zeros(FT_COUNTER_WORDS, dtype=np.uint64)
        self.flagged = np.full(2 * cap, -7, dtype=np.int64)
        self.cap = cap
        kargs.ft.counters = self.counters.ctypes.data
        kargs.ft.flagged = self.flagged.ctypes.data
        kargs.ft.flagged_cap = cap

    @property
    def checked(self):
        return int(self.counters[0])

    @property
    def detected(self):
        return int(self.counters[FT_SUB0::FT_SUB_STRIDE].sum())

    @property
    def unlocatable(self):
        return int(self.counters[FT_SUB0 + 1::FT_SUB_STRIDE].sum())

    def pairs(self):
        region = self.cap // 64
        out = []
        for k in range(64):
            have = min(int(self.counters[FT_SUB0 + FT_SUB_STRIDE * k]), region)
            for j in range(have):
                i = k * region + j
                out.append((int(self.flagged[2 * i]), int(self.flagged[2 * i + 1])))
        return out


def ctype_of(dtype):
    return np.complex64 if dtype == "float2" else np.complex128


def twiddle_table(N, dtype):
    out = np.empty(2 * N - 1, dtype=np.complex128)
    c = 1
    while c <= N:
        out[c - 1:2 * c - 1] = np.exp(-2j * np.pi * np.arange(c) / c)
        c *= 2
    return out.astype(ctype_of(dtype))


def build_sim(spec: KernelSpec):
    src = generate_source([spec], True).replace(
        '#include "../tfft_device.h"', f'#include "{ROOT}/turbofft_amd/csrc/tfft_device.h"')
    src += "\ntfft_sim_bounds_t tfft_sim_bounds; long long tfft_sim_errors = 0;\n"
    src += 'extern "C" long long tfft_sim_error_count() { return tfft_sim_errors; }\n'
    h = hashlib.sha1(src.encode()).hexdigest()[:16]
    os.makedirs(_CACHE, exist_ok=True)
    so = os.path.join(_CACHE, f"{spec.name}_{h}.so")
    if not os.path.exists(so):
        # build under a private name and rename: parallel test workers may want the same library
        tmp = f"{so[:-3]}.{os.getpid()}"
        with open(tmp + ".cpp", "w") as f:
            f.write(src)
        subprocess.check_call(["g++", "-O1", "-shared", "-fPIC", "-o", tmp + ".so", tmp + ".cpp"])
        os.replace(tmp + ".so", so)
        os.remove(tmp + ".cpp")
    return C.CDLL(so)


def run_sim(spec: KernelSpec, x_in: np.ndarray, out_elems: int, kargs: KArgs, grid: int,
            tw: np.ndarray, twhi=None, twlo=None, ck=None, out=None):
    lib = build_sim(spec)
    fn = getattr(lib, spec.name + "_sim")
    ct = ctype_of(spec.T2)
    x_in = np.ascontiguousarray(x_in, dtype=ct).ravel()
    if out is None:
        out = np.full(out_elems, np.nan + 1j * np.nan, dtype=ct)
    assert out.size == out_elems and out.dtype == ct and out.flags.c_contiguous
    tw = np.ascontiguousarray(tw, dtype=ct)
    keep = [x_in, out, tw]
    lim = np.zeros(6, dtype=np.int64)
    lim[0], lim[1], lim[2] = x_in.size, out.size, tw.size
    if twhi is not None:
        twhi = np.ascontiguousarray(twhi, dtype=ct); twlo = np.ascontiguousarray(twlo, dtype=ct)
        kargs.tw_hi = twhi.ctypes.data; kargs.tw_lo = twlo.ctypes.data
        lim[3], lim[4] = twhi.size, twlo.size
        keep += [twhi, twlo]
    if ck is not None:
        ck = np.ascontiguousarray(ck, dtype=ct)
        kargs.ft.cksum = ck.ctypes.data
        lim[5] = ck.size
        keep.append(ck)
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(KArgs), C.c_longlong, C.c_void_p]
    fn.restype = None
    fn(x_in.ctypes.data, out.ctypes.data, tw.ctypes.data, C.byref(kargs), grid, lim.ctypes.data)
    lib.tfft_sim_error_count.restype = C.c_longlong
    errs = lib.tfft_sim_error_count()
    assert errs == 0, f"{errs} out-of-bounds accesses in {spec.name}"
    return out


def split_tables(logL, dtype):
    """Two-level table for W_(2^L)^e: hi[h] = W^(h << lo_bits), lo[l] = W^l."""
    lo_bits = (logL + 1) // 2
    L = 1 << logL
    hi = np.exp(-2j * np.pi * (np.arange(1 << (logL - lo_bits)) << lo_bits) / L)
    lo = np.exp(-2j * np.pi * np.arange(1 << lo_bits) / L)
    return lo_bits, hi.astype(ctype_of(dtype)), lo.astype(ctype_of(dtype))


class FuseArgs(C.Structure):
    _fields_ = [("slots", C.c_void_p), ("ctl", C.c_void_p), ("err_host", C.c_void_p), ("piece_elems", C.c_longlong),
                ("npieces", C.c_longlong), ("tiles_a", C.c_int), ("tiles_b", C.c_int), ("team", C.c_int),
                ("teams_per_xcd", C.c_int), ("limit_ms", C.c_int)]


def run_pair_sim(fs, x_in: np.ndarray, bs: int, team: int, per_piece: int):
    """The fused pair of a two-launch plan for `bs` transforms of 2^(logN1 + logN2) points, one team of
    `team` members working through pieces of `per_piece` transforms (the last piece may be ragged)."""
    from turbofft_amd.codegen.fft_codegen import generate_fused_source
    src = generate_fused_source(fs, True).replace(
        '#include "../tfft_device.h"', f'#include "{ROOT}/turbofft_amd/csrc/tfft_device.h"')
    src += "\ntfft_sim_bounds_t tfft_sim_bounds; long long tfft_sim_errors = 0;\n"
    src += 'extern "C" long long tfft_sim_error_count() { return tfft_sim_errors; }\n'
    h = hashlib.sha1(src.encode()).hexdigest()[:16]
    os.makedirs(_CACHE, exist_ok=True)
    so = os.path.join(_CACHE, f"{fs.name}_{h}.so")
    if not os.path.exists(so):
        tmp = f"{so[:-3]}.{os.getpid()}"
        with open(tmp + ".cpp", "w") as f:
            f.write(src)
        subprocess.check_call(["g++", "-O1", "-shared", "-fPIC", "-o", tmp + ".so", tmp + ".cpp"])
        os.replace(tmp + ".so", so)
        os.remove(tmp + ".cpp")
    lib = C.CDLL(so)
    dtype = fs.T2
    ct = ctype_of(dtype)
    l1, l2 = fs.a.logNi, fs.b.logNi
    N = 1 << (l1 + l2)
    x_in = np.ascontiguousarray(x_in, dtype=ct).ravel()
    assert x_in.size == bs * N
    out = np.full(bs * N, np.nan + 1j * np.nan, dtype=ct)
    slot = np.full(per_piece * N, np.nan + 1j * np.nan, dtype=ct)
    tw = twiddle_table(max(1 << l1, 1 << l2), dtype)
    lo_bits, hi, lo = split_tables(l1 + l2, dtype)
    a0, a1 = KArgs(), KArgs()
    a0.ntiles, a0.thread_bs, a0.tb_gap, a0.log_ncols, a0.tw_lo_bits = bs * ((1 << l2) // fs.a.BS), 1, 1, l2, lo_bits
    a0.tw_hi, a0.tw_lo = hi.ctypes.data, lo.ctypes.data
    a1.ntiles, a1.thread_bs, a1.tb_gap = bs * ((1 << l1) // fs.b.BS), 1, 1
    a1.logQ, a1.logC, a1.logN = 0, l1, l1 + l2
    f = FuseArgs()
    f.piece_elems, f.npieces = per_piece * N, (bs + per_piece - 1) // per_piece
    f.tiles_a, f.tiles_b = per_piece * ((1 << l2) // fs.a.BS), per_piece * ((1 << l1) // fs.b.BS)
    f.team, f.teams_per_xcd, f.limit_ms = team, 1, 1
    lim = np.zeros(6, dtype=np.int64)
    lim[0], lim[1], lim[2], lim[3], lim[4] = x_in.size, out.size, tw.size, hi.size, lo.size
    fn = getattr(lib, fs.name + "_sim")
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(KArgs), C.POINTER(KArgs), C.POINTER(FuseArgs), C.c_void_p, C.c_void_p]
    fn.restype = None
    fn(x_in.ctypes.data, out.ctypes.data, tw.ctypes.data, C.byref(a0), C.byref(a1), C.byref(f), slot.ctypes.data, lim.ctypes.data)
    lib.tfft_sim_error_count.restype = C.c_longlong
    errs = lib.tfft_sim_error_count()
    assert errs == 0, f"{errs} out-of-bounds accesses in {fs.name}"
    return out.reshape(bs, N)
