"""CPU oracle for the batched radix-2 C2C forward FFT and its fused ABFT scheme.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() as the
checker and by bench.py for the timed CPU baseline.  The product package never
imports it.

Parity status (what pins each function):
  fft_ref                 the DFT definition; checked against dft_bruteforce,
                          impulse / constant / tone closed forms, linearity and
                          Parseval in tests/test_oracle.py.
  twiddle_table           closed form exp(-2*pi*i*m/c)         (pinned).
  dft_checksum_vector     mode="exact": hand-computed N=2,4 vectors and the
                          geometric-series closed form          (pinned);
                          mode="reference": the float-rounded angle of the
                          reference table builder, pinned by an independent
                          multiprecision evaluation of the same source lines
                          (tests/mp_checksum.py: float32 angle via struct,
                          cos/sin and the sum in 40-digit arithmetic; agreement
                          to 1e-14 in fp64, to float accumulation rounding in
                          fp32; five wrong readings of the lines -- unrounded
                          angle, 2*pi rounded first, index product rounded
                          first, r started at the wrong residue, +i exponent,
                          exact sqrt(3)/2 -- are each told apart)  (pinned).
  compact_cotangents      this build's compact form of the exact vector; pinned against
                          the (pinned) exact mode element by element to float16 rounding.
  block_fft / plan_fft    restatement of the reference kernel algebra (DIF
                          passes, twiddle recurrences, four-step digit maps);
                          checked against fft_ref for every plan class.
  delayed_batch_correction  the reference's batch-sum correction (live sums, commented
                          correction lines, notebook algebra); pinned by linearity: the
                          patched tile must equal the clean transform for errors of any
                          shape on one tile, and a flipped sign, a dropped sum or a wrong
                          tile index leaves an error of the injected size.
  ft_launch_model         restatement of the reference checksum arithmetic;
                          checked against the closed-form checksum shift of an
                          injected error and the "clean data -> no detection"
                          invariant.  The reference holds no vectors for it.

  thread_level_model      the same two-sided checksum applied by each thread to its own
                          register-level DFTs (the reference keeps the per-thread sums and the
                          result tables of its thread-level scheme, not its code); pinned by the
                          checksum identity against brute-force DFTs, by the closed-form shift of
                          an injected error (one thread of one pass objects, by exactly
                          injected_delta_closed_form of the first radix) and by faults put on
                          single butterfly outputs of every pass.

The reference repository ships no golden vectors, known-answer tests or
fixtures for this path (its only check is a run-time comparison with cuFFT),
so every pin above is mathematical.

Reference files restated here (all under the reference tree):
  include/utils/initializeData.h:31-37      twiddle table
  include/utils/abft.h:21-61, main.cu:85-93 DFT checksum table
  include/code_gen/scripts/fft_codegen.py   kernel algebra and FT arithmetic
  include/utils/compareData.h:4-35          element-wise comparator
  main.cu:4-73                              launch geometry and metrics
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

# sqrt(3)/2 as the float-rounded literal the reference uses for r[1], r[2]
# (abft.h:22-28, constants.h:2-7, fft_codegen.py:219-225).
SQRT3_2_LITERAL = 0.8660253882408142

ERR_SMOOTHING_DEFAULT = 1000      # fft_codegen.py:714
ERR_INJ_DEFAULT = 100             # fft_codegen.py:716
ERR_THRESHOLD_DEFAULT = 1e-3      # fft_codegen.py:718


# --------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------
def _ctype(dtype) -> np.dtype:
    """complex dtype for 'float2'/'double2'/0/1/np dtypes."""
    if dtype in (0, "float2", "fp32", "f32", np.float32, np.complex64):
        return np.dtype(np.complex64)
    if dtype in (1, "double2", "fp64", "f64", np.float64, np.complex128):
        return np.dtype(np.complex128)
    return np.dtype(dtype)


def _rtype(dtype) -> np.dtype:
    return np.dtype(np.float32) if _ctype(dtype) == np.complex64 else np.dtype(np.float64)


# --------------------------------------------------------------------------
# the accuracy oracle
# --------------------------------------------------------------------------
def fft_ref(x: np.ndarray) -> np.ndarray:
    """fp64 forward DFT along the last axis: X[k] = sum_n x[n] exp(-2 pi i n k / N)."""
    return np.fft.fft(np.asarray(x).astype(np.complex128), axis=-1)


def dft_bruteforce(x: np.ndarray) -> np.ndarray:
    """O(N^2) DFT with exact integer angle reduction (for N <= ~4096)."""
    x = np.asarray(x).astype(np.complex128)
    n = x.shape[-1]
    idx = (np.arange(n)[:, None] * np.arange(n)[None, :]) % n
    w = np.exp(-2j * np.pi * idx / n)
    return x @ w.T


def rel_l2(a: np.ndarray, ref: np.ndarray) -> float:
    a = np.asarray(a).astype(np.complex128).ravel()
    ref = np.asarray(ref).astype(np.complex128).ravel()
    den = np.linalg.norm(ref)
    return float(np.linalg.norm(a - ref) / (den if den > 0 else 1.0))


def tolerance(dtype, logN: int) -> float:
    """Accuracy bar: rel-L2 <= 1e-5*log2N (fp32), 1e-13*log2N (fp64)."""
    base = 1e-5 if _ctype(dtype) == np.complex64 else 1e-13
    return base * max(1, logN)


def compare_data(res: np.ndarray, ref: np.ndarray, error_bound: float = 1e-4) -> int:
    """The reference's element-wise comparator (compareData.h:4-35).

    Scans re then im of each element; a component fails if
    |res-ref|/(1+|ref|) > bound or res is NaN.  Returns the flat index of the
    first failing element, or -1 if the scan finishes.
    """
    res = np.asarray(res).ravel()
    ref = np.asarray(ref).ravel()
    bad = np.zeros(res.shape, dtype=bool)
    for part in (np.real, np.imag):
        a = part(res).astype(np.float64)
        b = part(ref).astype(np.float64)
        bad |= (np.abs((a - b) / (1 + np.abs(b))) > error_bound) | np.isnan(a)
    hit = np.flatnonzero(bad)
    return int(hit[0]) if hit.size else -1


# --------------------------------------------------------------------------
# host tables
# --------------------------------------------------------------------------
def twiddle_table(N: int, dtype) -> np.ndarray:
    """Concatenated twiddle table of 2N-1 entries (initializeData.h:31-37).

    For c = 1, 2, 4, ..., N:  tw[c-1+m] = exp(-2 pi i m / c), m < c, with the
    angle evaluated in double and the result stored as T.
    """
    out = np.empty(2 * N - 1, dtype=np.complex128)
    c = 1
    while c <= N:
        m = np.arange(c, dtype=np.float64)
        ang = (-2.0 * math.pi * m) / float(c)
        out[c - 1:2 * c - 1] = np.cos(ang) + 1j * np.sin(ang)
        c *= 2
    return out.astype(_ctype(dtype))


def checksum_r(dtype=np.complex128) -> np.ndarray:
    """The 3-periodic output encoding vector r (abft.h:22-28)."""
    r = np.array([1.0 + 0.0j,
                  -0.5 - 1j * SQRT3_2_LITERAL,
                  -0.5 + 1j * SQRT3_2_LITERAL], dtype=np.complex128)
    return r.astype(_ctype(dtype))


def dft_checksum_vector(N: int, dtype, mode: str = "exact") -> np.ndarray:
    """c_N[i] = sum_{j<N} W_N^{ij} r[j%3]   (abft.h:21-61).

    mode="exact":     angles reduced exactly, accumulated in fp64, cast to T.
    mode="compact":   this build's half-precision cotangent form of the exact vector (no
                      counterpart in the reference): see compact_cotangents.
    mode="reference": the reference's arithmetic -- the angle 2*pi*i*j is
                      rounded to float *before* the division by float(N)
                      (abft.h:34-35, 55-56), cos/sin in T, accumulation over j
                      in T, in order.
    """
    ct = _ctype(dtype)
    if mode == "exact":
        rvec = checksum_r(np.complex128)[np.arange(N) % 3]
        return np.fft.fft(rvec).astype(ct)        # c[i] = sum_j r[j%3] W^{ij}
    if mode == "compact":
        # what the kernels that read the compact table multiply with: kappa (1 - i t[m]), t in
        # half precision for fp32 kernels and in single precision for fp64 kernels
        return (compact_kappa(N) * (1.0 - 1j * compact_cotangents(N, dtype).astype(np.float64))).astype(ct)
    if mode != "reference":
        raise ValueError(mode)
    rt = _rtype(dtype)
    r = checksum_r(ct)
    i = np.arange(N, dtype=np.float64)
    accx = np.zeros(N, dtype=rt)
    accy = np.zeros(N, dtype=rt)
    two_pi = 2 * math.pi
    fN = np.float32(N)
    for j in range(N):
        ang = -(((two_pi * i) * float(j)).astype(np.float32)) / fN     # float32
        if rt == np.float32:
            x = np.cos(ang)                       # cosf on float
            y = np.sin(ang)
        else:
            x = np.cos(ang.astype(np.float64))    # cos on the promoted float
            y = np.sin(ang.astype(np.float64))
        rx = rt.type(r[j % 3].real)
        ry = rt.type(r[j % 3].imag)
        accx = (accx + (x * rx - y * ry)).astype(rt)
        accy = (accy + (x * ry + y * rx)).astype(rt)
    return (accx.astype(np.float64) + 1j * accy.astype(np.float64)).astype(ct)


def compact_kappa(N: int) -> complex:
    """(1 - rho^N) / 2 for the exact cube root rho = exp(-2 pi i / 3)."""
    return (1.0 - np.exp(-2j * np.pi * (N % 3) / 3.0)) / 2.0


def compact_cotangents(N: int, dtype="float2") -> np.ndarray:
    """The compact checksum table (a design of this build, not reference behaviour).

    With r[j%3] = rho^j for the exact cube root rho, c_N[m] = sum_j (rho W^m)^j is a geometric
    series: c_N[m] = (1 - rho^N) / (1 - rho W^m), and 1 / (1 - e^{-i theta}) = 1/2 - (i/2) cot(theta/2)
    makes it kappa (1 - i t[m]) with kappa = (1 - rho^N)/2 and the single real number
    t[m] = cot(pi (m/N + 1/3)) per element.  Stored in half precision for fp32 kernels and in
    single precision for fp64 kernels, which bounds the usable detection threshold from below
    (the library switches to the full table under 5e-4 and 1e-6).
    The reference's r uses a float-rounded sqrt(3)/2, 1.6e-8 away from rho: far below float16."""
    m = np.arange(N, dtype=np.float64)
    a = np.pi * (3.0 * m + N) / (3.0 * N)
    return (np.cos(a) / np.sin(a)).astype(np.float16 if _ctype(dtype) == np.complex64 else np.float32)


def compact_table_words(N: int, n: int, dtype="float2") -> np.ndarray:
    """Device layout of the compact table for a kernel whose threads hold n elements x + Tr*e
    (Tr = N/n).  fp32 kernels: 32-bit word [x + Tr*q] = (t[x + Tr*2q] low half, t[x + Tr*(2q+1)]
    high half); fp64 kernels: word [m] = t[m] in single precision."""
    if _ctype(dtype) == np.complex128:
        return compact_cotangents(N, dtype).view(np.uint32).copy()
    Tr = N // n
    bits = compact_cotangents(N).view(np.uint16).astype(np.uint32)
    x = np.arange(Tr)[None, :]
    q = np.arange(n // 2)[:, None]
    return (bits[x + Tr * 2 * q] | (bits[x + Tr * (2 * q + 1)] << 16)).reshape(-1).astype(np.uint32)


def dft_checksum_table(dtype, mode: str = "exact", max_log: int = 13) -> np.ndarray:
    """Concatenated c_N for N = 2, 4, ..., 2^max_log; c_N at offset N-2.

    Buffer length 16384*2 elements as in the reference (main.cu:85-93).
    """
    buf = np.zeros(16384 * 2, dtype=_ctype(dtype))
    N = 2
    while N <= (1 << max_log):
        buf[N - 2:2 * N - 2] = dft_checksum_vector(N, dtype, mode)
        N *= 2
    return buf


def checksum_closed_form(N: int) -> np.ndarray:
    """Geometric-series closed form of the exact c_N with r[j%3] = rho^j,
    where rho is the exact primitive cube root exp(-2 pi i/3).

    c_N[i] = (1 - q^N)/(1 - q),  q = exp(-2 pi i (i/N + 1/3)).
    Used only as an independent pin (agrees with the literal-based table to
    ~1.6e-8*N because the literal sqrt(3)/2 is float-rounded).
    """
    i = np.arange(N)
    th = -2 * np.pi * (i / N + 1.0 / 3.0)
    q = np.exp(1j * th)
    return (1 - np.exp(1j * th * N)) / (1 - q)


# --------------------------------------------------------------------------
# plan rows
# --------------------------------------------------------------------------
@dataclass
class PlanRow:
    """One row of a plan CSV: logN, launches, logN1..3, BS1..3, n1..3
    (readme.md:48-60; consumed at fft_codegen.py:745-752, main.cu:8-9,16,22-24).
    Launch i transforms a digit of size 2^logNi; launch 0 owns the most-strided
    digit, the last launch the contiguous one."""
    logN: int
    launches: int
    logNi: Tuple[int, ...]
    BS: Tuple[int, ...]
    n: Tuple[int, ...]

    @staticmethod
    def from_list(row: Sequence[int]) -> "PlanRow":
        row = [int(v) for v in row]
        L = row[1]
        return PlanRow(row[0], L, tuple(row[2:2 + L]), tuple(row[5:5 + L]), tuple(row[8:8 + L]))

    @property
    def N(self) -> int:
        return 1 << self.logN


def load_plan_csv(path: str) -> List[PlanRow]:
    """Row index == logN (main.cu:99,123); readCSV.h:3-33 splits on ','."""
    rows = []
    with open(path) as f:
        for line in f:
            line = line.strip()
            if not line:
                continue
            rows.append(PlanRow.from_list([int(t) for t in line.split(",")[:11]]))
    return rows


def radix_passes(Ni: int, n: int) -> List[int]:
    """In-block pass radices [n, n, ..., rest], rest last (fft_codegen.py:36-43
    builds the list, :127-138 rotates it so the partial radix runs last)."""
    out = []
    m = Ni
    while m > 1:
        out.append(n if m >= n else m)
        m //= n
    # the generator appends (n if N_tmp >= n else N_tmp) and divides by n each
    # time, so the final entry is the leftover factor
    prod = 1
    for r in out[:-1]:
        prod *= r
    out[-1] = Ni // prod
    return out


# --------------------------------------------------------------------------
# kernel algebra, restated on the CPU
# --------------------------------------------------------------------------
def _zmul(a, b, ct):
    """turboFFT_ZMUL (macro_ops.h:16): 4-op complex multiply in T."""
    return (a * b).astype(ct)


def _reg_fft(v: np.ndarray, R: int, ct) -> np.ndarray:
    """Radix-R DIF on axis 0 by log2(R) radix-2 stages (fft_codegen.py:647-705);
    returns outputs in natural order o = 0..R-1 (the generator's dict_output
    undoes the bit reversal, :560-572)."""
    if R == 1:
        return v
    half = R // 2
    a = v[:half]
    b = v[half:]
    s = (a + b).astype(ct)
    d = (a - b).astype(ct)
    k = np.arange(half)
    w = np.exp(-2j * np.pi * k / R).astype(ct)
    d = (d * w.reshape((half,) + (1,) * (v.ndim - 1))).astype(ct)
    even = _reg_fft(s, half, ct)     # X[2k]
    odd = _reg_fft(d, half, ct)      # X[2k+1]
    out = np.empty_like(v)
    out[0::2] = even
    out[1::2] = odd
    return out


def block_fft(x: np.ndarray, n: int, dtype, tw: Optional[np.ndarray] = None) -> np.ndarray:
    """The in-block multi-pass DIF Stockham FFT along the last axis, natural
    order out, computed in T with the reference's twiddle scheme: base
    W_M^j looked up in the concatenated table at [M-1+j], powers by the
    recurrence angle <- angle*delta (fft_codegen.py:574-645)."""
    ct = _ctype(dtype)
    x = np.asarray(x).astype(ct)
    Ni = x.shape[-1]
    if tw is None:
        tw = twiddle_table(Ni, dtype)
    lead = x.shape[:-1]
    P, M = 1, Ni
    data = x.reshape(lead + (M, P))                 # [m, low] <-> low + P*m
    passes = radix_passes(Ni, n)
    for q, R in enumerate(passes):
        J = M // R
        d = data.reshape(lead + (R, J, P))          # m = j + J*i
        d = np.moveaxis(d, len(lead), 0)            # [i, ..., j, low]
        y = _reg_fft(d, R, ct)                      # [o, ..., j, low]
        if q != len(passes) - 1:
            delta = tw[M - 1 + np.arange(J)].astype(ct)            # W_M^j
            angle = np.ones(J, dtype=ct)
            for o in range(1, R):
                angle = _zmul(angle, delta, ct)
                y[o] = (y[o] * angle.reshape((1,) * len(lead) + (J, 1))).astype(ct)
        # new position: low' = low + P*o, m' = j
        y = np.moveaxis(y, 0, len(lead) + 1)        # [..., j, o, low]
        data = y.reshape(lead + (J, R * P))
        P *= R
        M = J
    return data.reshape(lead + (Ni,))


def _interkernel_twiddle(y: np.ndarray, cols: np.ndarray, Ni: int, n: int, modulus: int,
                         tw: np.ndarray, ct) -> np.ndarray:
    """Multiply y[..., k, col] by W_modulus^{col*k} the way the kernels do
    (fft_codegen.py:385-400): a thread owns outputs k = k0 + (Ni/n)*i; it looks up
    angle = tw[modulus-1 + col*k0], delta = tw[modulus-1 + col*(Ni/n)] and
    advances angle <- angle*delta for i = 1..n-1."""
    T = Ni // n
    k0 = np.arange(T)
    out = np.empty_like(y)
    base = modulus - 1
    angle = tw[base + (cols[None, :] * k0[:, None]) % modulus].astype(ct)      # [k0, col]
    delta = tw[base + (cols * T) % modulus].astype(ct)[None, :]
    for i in range(n):
        if i:
            angle = _zmul(angle, delta, ct)
        out[..., k0 + T * i, :] = (y[..., k0 + T * i, :] * angle).astype(ct)
    return out


def plan_fft(x: np.ndarray, row: PlanRow, dtype, return_stages: bool = False):
    """The 1/2/3-launch decomposition (index algebra derived from the
    generated kernels, e.g. generated/double2/fft_radix_2_logN_15_upload_{0,1}.cuh
    and generated/float2/fft_radix_2_logN_24_upload_{0,1,2}.cuh):

      n = a + A*b + A*B*c, A = 2^logN_last (contiguous digit).
      L=2: launch 0  Y[a,kb] = W_N^{a kb} sum_b x[a+A b] W_B^{b kb}  (stored at a + A kb)
           launch 1  X[kb + B ka] = sum_a Y[a,kb] W_A^{a ka}
      L=3: launch 0  digit c, twiddle W_N^{(a+A b) kc}
           launch 1  digit b, twiddle W_{AB}^{a kb}
           launch 2  digit a, output X[kc + C kb + C B ka]

    x: (bs, N).  Returns X (bs, N) in natural order, computed in T.
    With return_stages also returns the list of per-launch (input, pre-twiddle
    output) arrays in launch memory layout, for the FT model.
    """
    ct = _ctype(dtype)
    x = np.asarray(x).astype(ct)
    bs, N = x.shape
    assert N == row.N
    tw = twiddle_table(N, dtype)
    stages = []
    L = row.launches
    if L == 1:
        out = block_fft(x, row.n[0], dtype, tw)
        stages.append((x, out))
        return (out, stages) if return_stages else out
    if L == 2:
        B, A = 1 << row.logNi[0], 1 << row.logNi[1]
        v = x.reshape(bs, B, A)
        y = np.moveaxis(block_fft(np.moveaxis(v, 1, 2), row.n[0], dtype, tw), 2, 1)   # [bs, kb, a]
        stages.append((v.reshape(bs, N), y.reshape(bs, N).copy()))
        y = _interkernel_twiddle(y, np.arange(A), B, row.n[0], N, tw, ct)
        z = block_fft(y, row.n[1], dtype, tw)                                           # [bs, kb, ka]
        stages.append((y.reshape(bs, N), z.reshape(bs, N)))
        out = np.moveaxis(z, 1, 2).reshape(bs, N)                                       # kb + B*ka
        return (out, stages) if return_stages else out
    if L == 3:
        C, B, A = (1 << row.logNi[0]), (1 << row.logNi[1]), (1 << row.logNi[2])
        v = x.reshape(bs, C, A * B)
        y = np.moveaxis(block_fft(np.moveaxis(v, 1, 2), row.n[0], dtype, tw), 2, 1)   # [bs, kc, m]
        stages.append((x, y.reshape(bs, N).copy()))
        y = _interkernel_twiddle(y, np.arange(A * B), C, row.n[0], N, tw, ct)
        v1 = y.reshape(bs, C, B, A)
        y1 = np.moveaxis(block_fft(np.moveaxis(v1, 2, 3), row.n[1], dtype, tw), 3, 2)  # [bs,kc,kb,a]
        stages.append((y.reshape(bs, N), y1.reshape(bs, N).copy()))
        y1 = _interkernel_twiddle(y1, np.arange(A), B, row.n[1], A * B, tw, ct)
        z = block_fft(y1, row.n[2], dtype, tw)                                           # [bs,kc,kb,ka]
        stages.append((y1.reshape(bs, N), z.reshape(bs, N)))
        out = np.transpose(z, (0, 3, 2, 1)).reshape(bs, N)                              # kc + C kb + CB ka
        return (out, stages) if return_stages else out
    raise ValueError("launches must be 1..3")


# --------------------------------------------------------------------------
# launch geometry (tiles) -- used by the FT model
# --------------------------------------------------------------------------
@dataclass
class LaunchGeom:
    """Tile geometry of one launch.

    A tile is BS sub-FFTs of length Ni.  `gather(arr)` returns the launch's
    data as [tile, s, m] (m = index along the transformed digit) from an array
    in launch memory layout (bs, N).  The tile enumeration is the gfx950
    plan's (a design choice of this build, not reference behaviour):
      column launches: tile -> (outer block, BS adjacent columns), columns fastest;
      final launch of L>=2: tile -> BS rows adjacent along the most-strided
        digit (kc for L=3, kb for L=2), then the middle digit, then batch;
      single launch: tile -> BS consecutive transforms.
    The reference enumerates contiguous digits first (fft_codegen.py:303-344);
    the checksum arithmetic per tile group does not depend on that order.
    """
    Ni: int
    BS: int
    n: int
    ntiles: int
    kind: str              # "col", "row1", "rowT"
    shape: Tuple[int, ...]

    def gather(self, arr: np.ndarray) -> np.ndarray:
        bs = arr.shape[0]
        Ni, BS = self.Ni, self.BS
        if self.kind == "row1":
            pad = (-bs) % BS
            if pad:
                arr = np.concatenate([arr, np.zeros((pad, Ni), arr.dtype)], 0)
            return arr.reshape(-1, BS, Ni)
        if self.kind == "col":
            outer, ncols = self.shape            # per transform
            v = arr.reshape(bs * outer, Ni, ncols // BS, BS)      # [o, m, ct, s]
            return np.transpose(v, (0, 2, 3, 1)).reshape(-1, BS, Ni)
        if self.kind == "rowT":
            C, Q = self.shape                    # rows = q + Q*s', s' in [0,C)
            v = arr.reshape(bs, C // BS, BS, Q, Ni)               # [b, ct, s, q, a]
            return np.transpose(v, (0, 3, 1, 2, 4)).reshape(-1, BS, Ni)
        raise ValueError(self.kind)


def launch_geometry(row: PlanRow, bs: int) -> List[LaunchGeom]:
    N = row.N
    L = row.launches
    g = []
    if L == 1:
        BS = row.BS[0]
        g.append(LaunchGeom(N, BS, row.n[0], (bs + BS - 1) // BS, "row1", ()))
    elif L == 2:
        B, A = 1 << row.logNi[0], 1 << row.logNi[1]
        g.append(LaunchGeom(B, row.BS[0], row.n[0], bs * A // row.BS[0], "col", (1, A)))
        g.append(LaunchGeom(A, row.BS[1], row.n[1], bs * B // row.BS[1], "rowT", (B, 1)))
    else:
        C, B, A = (1 << row.logNi[0]), (1 << row.logNi[1]), (1 << row.logNi[2])
        g.append(LaunchGeom(C, row.BS[0], row.n[0], bs * A * B // row.BS[0], "col", (1, A * B)))
        g.append(LaunchGeom(B, row.BS[1], row.n[1], bs * C * A // row.BS[1], "col", (C, A)))
        g.append(LaunchGeom(A, row.BS[2], row.n[2], bs * B * C // row.BS[2], "rowT", (C, B)))
    return g


def tile_groups(ntiles: int, thread_bs: int, tb_gap: int) -> List[List[int]]:
    """Tiles handled by each block, in processing order (cnt = 1, 2, ...).

    Restates the reference loop (fft_codegen.py:218,260-261) with the grid
    size rounded up instead of down (main.cu:32 truncates and would drop the
    remainder tiles):
      bid0  = (bx / tb_gap) * tb_gap * thread_bs + bx % tb_gap
      delta = tb_gap, or gridDim % tb_gap in the last partial chunk
      tiles = bid0 + cnt*delta while cnt < thread_bs and tile < ntiles
    """
    grid = (ntiles + thread_bs - 1) // thread_bs
    groups = []
    for bx in range(grid):
        chunk = bx // tb_gap
        delta = tb_gap if (chunk + 1) * tb_gap <= grid else grid - chunk * tb_gap
        t = chunk * tb_gap * thread_bs + bx % tb_gap
        tiles = []
        while len(tiles) < thread_bs and t < ntiles:
            tiles.append(t)
            t += delta
        groups.append(tiles)
    return groups


# --------------------------------------------------------------------------
# FT model
# --------------------------------------------------------------------------
@dataclass
class Injection:
    """Compute-side soft error: `mag` added to re of element m of sub-FFT s of
    `tile`, after the input checksum (fft_codegen.py:412-415 uses s=0, m=0,
    tile cnt == blockIdx % thread_bs + 1 of every block, last launch only)."""
    tile: int
    s: int = 0
    m: int = 0
    mag: float = float(ERR_INJ_DEFAULT)


def reference_injections(groups: List[List[int]], thread_bs: int, mag: float = ERR_INJ_DEFAULT,
                         every: int = 1) -> List[Injection]:
    """The reference cadence: in block bx the tile with cnt == bx % thread_bs + 1."""
    out = []
    for bx, tiles in enumerate(groups):
        if bx % every:
            continue
        c = bx % thread_bs
        if c < len(tiles):
            out.append(Injection(tiles[c], 0, 0, float(mag)))
    return out


@dataclass
class GroupDecision:
    delta: float
    delta2: float
    mag: float
    detected: bool
    k: int                 # 1-based tile counter of the flagged tile, -1 if none
    tile: int              # flagged tile id, -1 if none / out of range


def _round_half_away(v: float) -> int:
    return int(math.floor(abs(v) + 0.5)) * (1 if v >= 0 else -1)


def ft_launch_model(xin: np.ndarray, yout: np.ndarray, n: int, groups: List[List[int]], dtype,
                    c_vec: np.ndarray, err_smoothing: float = ERR_SMOOTHING_DEFAULT,
                    err_threshold: float = ERR_THRESHOLD_DEFAULT) -> List[GroupDecision]:
    """The per-block checksum test of one launch (fft_codegen.py:354-384, 432-503).

    xin[tile, s, m]   : launch inputs;  yout[tile, s, k] : the outputs the kernel
    produced (including any injected error), before the inter-launch twiddle.
    A thread owns elements {txr + (Ni/n)*e, e<n} of one sub-FFT on both sides.
      in1  += s_in,  in2  += cnt*s_in,   s_in  = re+im of x*c[m]
      out1 -= s_out, out2 -= cnt*s_out,  s_out = re+im of y*r[k%3]
      delta = sum_thr(in1+out1); mag = sum_thr(|in1|+|out1|); delta2 = sum_thr(in2+out2)
      detected = |delta|/(err_smoothing+|mag|) > err_threshold
      k = round(|delta2|/|delta|)
    Accumulation is done in T per thread, then summed over threads (the order
    of the cross-thread sum is not part of the scheme).
    """
    ct = _ctype(dtype)
    rt = _rtype(dtype)
    ntile, BS, Ni = xin.shape
    T = Ni // n
    r = checksum_r(ct)
    tin = (xin.astype(ct) * c_vec.astype(ct)[None, None, :]).astype(ct)
    sin = (tin.real + tin.imag).astype(rt)                         # [tile, s, m]
    tout = (yout.astype(ct) * r[np.arange(Ni) % 3][None, None, :]).astype(ct)
    sout = (tout.real + tout.imag).astype(rt)
    # per-thread partial sums per tile: thread (s, txr) owns m = txr + T*e
    sin_t = sin.reshape(ntile, BS, n, T).sum(axis=2, dtype=rt)     # [tile, s, txr]
    sout_t = sout.reshape(ntile, BS, n, T).sum(axis=2, dtype=rt)
    out = []
    for tiles in groups:
        in1 = np.zeros((BS, T), rt); in2 = np.zeros((BS, T), rt)
        o1 = np.zeros((BS, T), rt); o2 = np.zeros((BS, T), rt)
        for cnt, t in enumerate(tiles, start=1):
            in1 = (in1 + sin_t[t]).astype(rt)
            in2 = (in2 + rt.type(cnt) * sin_t[t]).astype(rt)
            o1 = (o1 - sout_t[t]).astype(rt)
            o2 = (o2 - rt.type(cnt) * sout_t[t]).astype(rt)
        delta = float((in1 + o1).astype(rt).sum(dtype=np.float64))
        mag = float((np.abs(in1) + np.abs(o1)).astype(rt).sum(dtype=np.float64))
        delta2 = float((in2 + o2).astype(rt).sum(dtype=np.float64))
        det = abs(delta) / (err_smoothing + abs(mag)) > err_threshold
        k = -1
        tile = -1
        if det:
            k = _round_half_away(abs(delta2) / abs(delta)) if delta != 0 else -1
            if 1 <= k <= len(tiles):
                tile = tiles[k - 1]
        out.append(GroupDecision(delta, delta2, mag, bool(det), k, tile))
    return out


def delayed_batch_correction(x_tiles: np.ndarray, y_tiles: np.ndarray, k: int, n: int, dtype) -> np.ndarray:
    """Delayed batch correction of one checksum group (fft_codegen.py:355-357 per-thread input
    sums, :421-423 output sums, the correction lines commented at :401-404 and :427-429, and
    the algebra of test.ipynb cell 0 with unit weights):

        y_k  <-  y_k + FFT(sum_t x_t) - sum_t y_t

    x_tiles[t, s, m] are the inputs of the group's tiles in processing order, y_tiles[t, s, j]
    the outputs as the kernel produced them (tile k, 0-based, carrying the error), both before
    any inter-launch twiddle.  Sums run over t in order, in T; the transform of the summed
    input is the in-block FFT in T.  By linearity the patched tile equals the clean
    transform of x_k when no other tile of the group is corrupted; unlike a recompute it is
    not bit-identical to it (its rounding error grows with the group size).
    Returns the patched y_tiles[k]."""
    ct = _ctype(dtype)
    sx = np.zeros(x_tiles.shape[1:], ct)
    sy = np.zeros(y_tiles.shape[1:], ct)
    for t in range(x_tiles.shape[0]):
        sx = (sx + x_tiles[t].astype(ct)).astype(ct)
        sy = (sy + y_tiles[t].astype(ct)).astype(ct)
    corr = (block_fft(sx, n, dtype) - sy).astype(ct)
    return (y_tiles[k].astype(ct) + corr).astype(ct)


def injected_delta_closed_form(Ni: int, mag: float) -> float:
    """Checksum shift caused by adding `mag` to re(x[0]) of one sub-FFT after
    the input checksum: every output of that sub-FFT moves by mag, so
    delta = -mag * sum_{k<Ni} (re r[k%3] + im r[k%3])."""
    r = checksum_r(np.complex128)
    rv = r[np.arange(Ni) % 3]
    return -mag * float((rv.real + rv.imag).sum())


def ft_plan_model(x: np.ndarray, row: PlanRow, dtype, thread_bs: int, tb_gap: Sequence[int],
                  injections: Optional[Sequence[Injection]] = None, inj_launch: int = -1,
                  table_mode: str = "exact", err_smoothing: float = ERR_SMOOTHING_DEFAULT,
                  err_threshold: float = ERR_THRESHOLD_DEFAULT):
    """Run every launch's checksum test on clean data plus injected errors.

    Returns (decisions per launch, corrected output).  With recompute
    correction every flagged tile is recomputed from the launch input without
    the error, so the corrected result equals the clean transform.
    """
    ct = _ctype(dtype)
    out, stages = plan_fft(x, row, dtype, return_stages=True)
    geoms = launch_geometry(row, x.shape[0])
    inj_launch = inj_launch % row.launches
    decisions = []
    for li, (geom, (lin, lout)) in enumerate(zip(geoms, stages)):
        xin = geom.gather(lin)
        if geom.kind == "col":
            yout = geom.gather(lout)
        else:
            # row launches: `lout` is [.., rows, k] in the same row order as the input
            yout = geom.gather(lout)
        yout = yout.copy()
        if injections and li == inj_launch:
            for inj in injections:
                # x[m] += mag  ==>  y[k] += mag * W^{m k}
                k = np.arange(geom.Ni)
                yout[inj.tile, inj.s, :] += (inj.mag * np.exp(-2j * np.pi * ((inj.m * k) % geom.Ni) / geom.Ni)).astype(ct)
        groups = tile_groups(geom.ntiles, thread_bs, tb_gap[li])
        c_vec = dft_checksum_vector(geom.Ni, dtype, table_mode)
        decisions.append(ft_launch_model(xin, yout, geom.n, groups, dtype, c_vec,
                                         err_smoothing, err_threshold))
    return decisions, out


# --------------------------------------------------------------------------
# thread-level verification
# --------------------------------------------------------------------------
def thread_level_vectors(R: int, dtype) -> Tuple[np.ndarray, np.ndarray]:
    """Checksum vectors of one register-level radix-R DFT: the output-side r[o % 3]
    (abft.h:22-28) and the input-side c_R = W_R^T r (abft.h:45-60 for N = R, exact angles)."""
    ct = _ctype(dtype)
    rv = checksum_r(np.complex128)[np.arange(R) % 3]
    return np.fft.fft(rv).astype(ct), rv.astype(ct)


@dataclass
class ThreadVerdict:
    tile: int
    s: int          # sub-FFT of the tile
    q: int          # pass
    thread: int     # thread of the sub-FFT (x = 0 .. Ni/n - 1)
    delta: float    # in - out of the thread's two sums
    mag: float      # |in| + |out|
    ratio: float    # |delta| / (err_smoothing + mag)


def thread_level_model(xin: np.ndarray, n: int, dtype, injections: Optional[Sequence[Injection]] = None,
                       out_faults: Optional[Sequence[Tuple[int, int, int, int, int, complex]]] = None,
                       err_smoothing: float = ERR_SMOOTHING_DEFAULT, err_threshold: float = ERR_THRESHOLD_DEFAULT):
    """Thread-level verification of one launch (the scheme behind the reference's
    data_ft/ft_scheme_thread_bs=1_* tables, of which its generator keeps only the per-thread
    sums, fft_codegen.py:354-384): the two-sided checksum of abft.h applied by every thread to
    the radix-R DFTs it computes in registers, pass by pass.

    xin[tile, s, m]: launch inputs.  In pass q a thread x of sub-FFT s owns the U = n/R DFTs
    `rest = x + (Ni/n) u` (rest = low + P j: inputs m = j + J i of the length-M sub-problem `low`).
      in  = sum over its DFTs and their inputs  of re+im(x_i c_R[i])
      out = sum over its DFTs and their outputs of re+im(y_o r[o % 3])   (before the pass's twiddles)
      the thread objects iff |in - out| / (err_smoothing + |in| + |out|) > err_threshold
    A tile is flagged when any of its threads objects in any pass; it is then recomputed, so the
    corrected result is the clean transform.  `injections` add `mag` to re of input element m
    (m < Ni/n: register 0 of thread m) of sub-FFT s after the first pass's input sums
    (fft_codegen.py:412-415); `out_faults` (tile, s, q, rest, o, value) add `value` to output o of one
    register-level DFT of pass q before the output sums (a fault inside that butterfly network).
    Returns (flagged[tile] bool array, list of ThreadVerdict for the objecting threads, worst ratio
    among the threads that did not object)."""
    ct = _ctype(dtype)
    rt = _rtype(dtype)
    xin = np.asarray(xin).astype(ct)
    ntile, BS, Ni = xin.shape
    Tr = Ni // n
    tw = twiddle_table(Ni, dtype)
    P, M = 1, Ni
    data = xin.reshape(ntile, BS, M, P)
    passes = radix_passes(Ni, n)
    flagged = np.zeros(ntile, dtype=bool)
    verdicts: List[ThreadVerdict] = []
    worst_quiet = 0.0
    for q, R in enumerate(passes):
        J = M // R
        U = n // R
        cR, rR = thread_level_vectors(R, dtype)
        d = np.moveaxis(data.reshape(ntile, BS, R, J, P), 2, 0).copy()        # [i, tile, s, j, low]
        t = (d * cR.reshape(R, 1, 1, 1, 1)).astype(ct)
        sin = (t.real + t.imag).astype(rt).sum(axis=0, dtype=rt)                # [tile, s, j, low]
        if q == 0 and injections:
            for inj in injections:
                assert 0 <= inj.m < Tr, "the injected element is one of the first Ni/n of its sub-FFT"
                d[0, inj.tile, inj.s, inj.m, 0] += rt.type(inj.mag)
        y = _reg_fft(d, R, ct)                                                  # [o, tile, s, j, low]
        if out_faults:
            for (ft_tile, ft_s, ft_q, ft_rest, ft_o, ft_val) in out_faults:
                if ft_q == q:
                    y[ft_o, ft_tile, ft_s, ft_rest // P, ft_rest % P] += ct.type(ft_val)
        t = (y * rR.reshape(R, 1, 1, 1, 1)).astype(ct)
        sout = (t.real + t.imag).astype(rt).sum(axis=0, dtype=rt)
        # DFT (j, low) is `rest = low + P j` = x + Tr u of thread x
        tin = sin.reshape(ntile, BS, U, Tr).sum(axis=2, dtype=rt)
        tout = sout.reshape(ntile, BS, U, Tr).sum(axis=2, dtype=rt)
        delta = (tin - tout).astype(np.float64)
        mag = (np.abs(tin) + np.abs(tout)).astype(np.float64)
        ratio = np.abs(delta) / (err_smoothing + mag)
        bad = ratio > err_threshold
        for (ti, si, xi) in zip(*np.nonzero(bad)):
            verdicts.append(ThreadVerdict(int(ti), int(si), q, int(xi), float(delta[ti, si, xi]), float(mag[ti, si, xi]),
                                          float(ratio[ti, si, xi])))
        flagged |= bad.any(axis=(1, 2))
        if (~bad).any():
            worst_quiet = max(worst_quiet, float(ratio[~bad].max()))
        if q != len(passes) - 1:
            delta_w = tw[M - 1 + np.arange(J)].astype(ct)
            angle = np.ones(J, dtype=ct)
            for o in range(1, R):
                angle = _zmul(angle, delta_w, ct)
                y[o] = (y[o] * angle.reshape(1, 1, J, 1)).astype(ct)
        data = np.moveaxis(y, 0, 3).reshape(ntile, BS, J, R * P)               # [tile, s, j, o, low] -> low' = low + P o
        P *= R
        M = J
    return flagged, verdicts, worst_quiet


def thread_level_plan_model(x: np.ndarray, row: PlanRow, dtype, injections: Optional[Sequence[Injection]] = None,
                            inj_launch: int = -1, err_smoothing: float = ERR_SMOOTHING_DEFAULT,
                            err_threshold: float = ERR_THRESHOLD_DEFAULT):
    """thread_level_model for every launch of a plan on clean data plus injected errors (in launch
    `inj_launch`).  Returns (per launch: flagged[tile], verdicts, worst quiet ratio) and the corrected
    output (every flagged tile is recomputed, so it is the clean transform)."""
    out, stages = plan_fft(x, row, dtype, return_stages=True)
    geoms = launch_geometry(row, x.shape[0])
    inj_launch = inj_launch % row.launches
    res = []
    for li, (geom, (lin, _)) in enumerate(zip(geoms, stages)):
        res.append(thread_level_model(geom.gather(lin), geom.n, dtype, injections if li == inj_launch else None,
                                      None, err_smoothing, err_threshold))
    return res, out


# --------------------------------------------------------------------------
# metrics (main.cu:68-69)
# --------------------------------------------------------------------------
def gflops(N: int, bs: int, ms: float) -> float:
    return 5.0 * N * math.log2(N) * bs / ms * 1000 / 1e9


def algorithmic_gbs(N: int, bs: int, ms: float, dtype) -> float:
    return float(N * bs * _ctype(dtype).itemsize * 2) / ms * 1000.0 / 1e9
