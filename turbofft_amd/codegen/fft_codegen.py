#!/usr/bin/env python3
"""gfx950 kernel generator for the batched radix-2 C2C FFT.

Plays the role of the reference generator
(include/code_gen/scripts/fft_codegen.py, class TurboFFT + __main__): it reads
a plan CSV in the reference's 11-column format (logN, launches, logN1..3,
BS1..3, n1..3; readme.md:48-60) and prints fully unrolled kernels, with the
same command-line flags (--if_ft, --if_err_injection, --err_smoothing,
--err_inj, --err_threshold, --datatype, --gpu; fft_codegen.py:709-723).

It is not a translation of that generator.  The differences that matter:
  * three kernel kinds with run-time geometry -- `row1` (whole transforms,
    contiguous axis), `col` (strided digit + inter-launch twiddle) and `rowT`
    (contiguous digit, transposed natural-order store) -- so one kernel per
    (type, kind, Ni, BS, n) serves every logN with that tile shape;
  * wave64 thread maps chosen per pass: loads of contiguous rows are
    row-major (a wavefront reads whole 128-byte lines), the last pass of
    `rowT` is re-mapped column-major through the final LDS exchange so the
    transposed store writes BS-element runs;
  * LDS exchanges with computed padding (see lds_model.py) instead of the
    rotation swizzle; twiddles W_M^(j*2^b) are fetched exactly from the
    concatenated table and combined with log-depth products instead of a
    linear recurrence; inter-launch twiddles use a two-level (hi/lo) table
    instead of a 2N-entry one;
  * the fault-tolerance variant keeps the reference's checksum arithmetic
    (fft_codegen.py:354-384, 432-503) but takes thresholds, the injection
    descriptor and the correction switch at run time, reports counters, and
    re-runs the located tile through the same loop body.

Every kernel is emitted as a list of phases separated by block barriers.  The
same phase text compiles for gfx950 (hipcc) and, with -DTFFT_SIM, as a
lock-step CPU execution with bounds-checked accessors that the CPU test-suite
uses to validate index algebra without a GPU.
"""
from __future__ import annotations

import argparse
import math
import os
import sys
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

if __package__ in (None, ""):
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from turbofft_amd.codegen import lds_model
from turbofft_amd.codegen.plan import PlanRow, KernelKey, load_plan_csv, kernels_for_row, radix_passes

WAVE = 64


def ilog2(v: int) -> int:
    l = v.bit_length() - 1
    if v <= 0 or (1 << l) != v:
        raise ValueError(f"{v} is not a power of two")
    return l


def bitrev(x: int, bits: int) -> int:
    y = 0
    for _ in range(bits):
        y = (y << 1) | (x & 1)
        x >>= 1
    return y


class Code:
    def __init__(self):
        self.lines: List[str] = []
        self.ind = 0

    def __call__(self, s: str = ""):
        for ln in s.split("\n"):
            self.lines.append(("    " * self.ind + ln) if ln else "")

    def text(self) -> str:
        return "\n".join(self.lines) + "\n"


@dataclass
class KernelSpec:
    key: KernelKey
    pad_override: Optional[Dict[int, Tuple[int, int]]] = None

    def __post_init__(self):
        k = self.key
        self.T2 = k.dtype                       # float2 / double2
        self.R = "float" if k.dtype == "float2" else "double"
        self.esize = 8 if k.dtype == "float2" else 16
        self.Ni = 1 << k.logNi
        self.BS = k.BS
        self.n = k.n
        self.kind = k.kind
        self.ft = int(k.ft) in (1, 2)   # block-level two-sided checksums over a group of tiles
        self.dc = int(k.ft) == 2    # delayed batch correction: sums of the group's inputs and outputs per thread
        # thread-level verification: every thread checks each register-level radix-R DFT it computes
        # (sum_o y_o r[o%3] against sum_i x_i c_R[i], the two-sided checksum of abft.h:21-61 applied to
        # the thread's own butterflies) pass by pass; no sums leave the thread, the block only agrees on
        # whether any thread objected, and a tile that one did object to is recomputed before it is stored
        self.tl = int(k.ft) == 3
        if self.tl and (k.pf or k.xl or k.ck or k.inv):
            raise ValueError(f"{k}: thread-level verification has no prefetching, cross-lane, compact-table or inverse flavour")
        self.ck16 = bool(k.ck)      # compact checksum table: one cotangent per element (half precision for fp32, single for fp64)
        if self.ck16 and (int(k.ft) != 1 or k.n % 2 or k.pf):
            raise ValueError(f"{k}: the compact checksum table is for recompute-correcting kernels without prefetch")
        if self.ck16 and k.dtype == "float2" and k.logNi > 16:
            # the largest entry, cot(pi/3 + pi m/Ni) next to its pole, is about 3 Ni / pi: over 65504 from Ni = 2^17
            raise ValueError(f"{k}: half-precision cotangents overflow for sub-FFTs of more than 2^16 points")
        self.split = bool(k.split)
        self.pf = bool(k.pf)        # software prefetch of the next tile into a second register set
        # pf > 1: only the first pf elements of a thread are fetched ahead, and only from the start
        # of the tile's last pass on (for 1024-thread blocks, which have no room for a whole set)
        self.pfk = int(k.pf) if int(k.pf) > 1 else 0
        if self.pfk and (int(k.ft) or k.xl or self.pfk >= k.n):
            raise ValueError(f"{k}: partial prefetch is for plain kernels, fewer elements than n")
        self.xl = bool(k.xl)        # last (radix 2/4/8) pass across lanes instead of through LDS
        self.lds_esize = self.esize // 2 if self.split else self.esize   # bytes per LDS access
        self.passes = radix_passes(self.Ni, self.n)
        self.npass = len(self.passes)
        self.Tr = self.Ni // self.n              # threads per sub-FFT
        self.threads = self.Tr * self.BS
        self.E = self.Ni * self.BS
        if self.dc and self.pf:
            raise ValueError(f"{k}: delayed batch correction has no prefetching flavour")
        if self.threads % WAVE or self.threads > 1024:
            raise ValueError(f"{k}: {self.threads} threads per block (need a multiple of 64, <= 1024)")
        # thread map per pass: 'major' (s = tx / Tr) or 'minor' (s = tx % BS)
        if self.kind == "col":
            self.maps = ["minor"] * self.npass
        elif self.kind == "row1":
            self.maps = ["major"] * self.npass
        else:  # rowT: row-major loads, column-major transposed store
            self.maps = ["major"] * (self.npass - 1) + ["minor"]
            if self.npass == 1:
                self.maps = ["minor"]
        # P_q: product of the radices before pass q
        self.P = [1]
        for R in self.passes:
            self.P.append(self.P[-1] * R)
        # passes that end with an LDS exchange or the global store; with a cross-lane last
        # pass the final radix is folded into the pass before it
        self.npass_lds = self.npass
        if self.xl:
            self.RL = self.passes[-1]
            if (self.kind != "row1" or self.ft or self.npass < 3 or self.RL not in (2, 4, 8)
                    or self.passes[-2] != self.n or self.Tr % self.RL):
                raise ValueError(f"{k}: the cross-lane last pass needs a row1 non-FT kernel with >= 3 passes "
                                 f"ending in radix 2, 4 or 8 (passes {self.passes})")
            self.npass_lds = self.npass - 1
        # padding per exchange x (between pass x and x+1)
        self.pads: List[Tuple[int, int]] = []
        for x in range(self.npass_lds - 1):
            if self.pad_override and x in self.pad_override:
                self.pads.append(self.pad_override[x])
            else:
                self.pads.append(lds_model.choose_padding(self, x))
        self.lds_elems = max([self.phys_const(self.E - 1, p) + 1 for p in self.pads] + [1])
        self.red_off_bytes = (self.lds_elems * self.lds_esize + 15) // 16 * 16
        self.lds_bytes = self.red_off_bytes + (3 * (self.threads // WAVE) * 8 if self.ft else 0) + (16 * 4 if self.tl else 0)
        # compact checksum words parked in LDS (ck = 3): W words per thread behind the reduction
        # slots, four to an access, access g of thread tx at [g * threads + tx]
        self.ck_lds = int(k.ck) == 3
        self.ck_words = (self.n // 2 if self.R == "float" else self.n) if self.ck16 else 0
        self.cw_off_bytes = (self.lds_bytes + 15) // 16 * 16
        if self.ck_lds:
            if self.ck_words % 4:
                raise ValueError(f"{k}: parking the compact table in LDS needs a multiple of 4 words per thread")
            self.lds_bytes = self.cw_off_bytes + self.ck_words * self.threads * 4

    # ---- address helpers (python side) ----
    @staticmethod
    def phys_const(a: int, pad: Tuple[int, int]) -> int:
        ps, pl = pad
        return a if ps < 0 else a + ((a >> ps) << pl)

    def logical_write_addr(self, x: int, tx: int, u: int, o: int) -> int:
        """Logical LDS element address written by thread tx after pass x for
        butterfly u, output digit o (layout = thread map of pass x+1)."""
        s, xr = self.thread_sx(x, tx)
        R = self.passes[x]
        P = self.P[x]
        rest = xr + self.Tr * u
        low, j = rest % P, rest // P
        pos = low + P * o + P * R * j
        return self.layout_addr(self.maps[x + 1], s, pos)

    def logical_read_addr(self, q: int, tx: int, e: int) -> int:
        s, xr = self.thread_sx(q, tx)
        return self.layout_addr(self.maps[q], s, xr + self.Tr * e)

    def thread_sx(self, q: int, tx: int) -> Tuple[int, int]:
        if self.maps[q] == "major":
            s, x = tx // self.Tr, tx % self.Tr
        else:
            s, x = tx % self.BS, tx // self.BS
        if self.xl and q == self.npass_lds - 1:
            # partners of the cross-lane pass sit in adjacent lanes: j in the low bits
            x = (x // self.RL) + (x % self.RL) * self.P[q]
        return s, x

    def layout_addr(self, kind: str, s: int, pos: int) -> int:
        return s * self.Ni + pos if kind == "major" else s + self.BS * pos

    @property
    def name(self) -> str:
        return self.key.name


class KernelEmitter:
    def __init__(self, spec: KernelSpec, err_smoothing=1000, err_inj=100, err_threshold=1e-3, role: Optional[str] = None,
                 block_threads: Optional[int] = None):
        self.s = spec
        self.T2 = spec.T2
        self.R = spec.R
        # Half of a fused pair (one kernel runs both launches of a two-launch plan, the intermediate
        # staying in a slot that the XCD's L2 holds): "A" writes its tiles into the slot, "B" reads its
        # tiles from it.  Slot addresses are relative to the first element of the piece the team works
        # on; `block_threads` is the block size of the fused kernel (a half with fewer threads leaves the
        # other wavefronts idle between barriers).
        self.role = role
        self.block_threads = block_threads or spec.threads
        self.prefetched = False     # half "A": a member's first tile of a piece arrives in rn[] (fetched during the piece before)
        # Single-launch kernels address global memory through buffer instructions (uniform base
        # in SGPRs, one shared 32-bit lane offset): fewer address registers and no per-access
        # vector arithmetic, +4-5 % on the large tiles.  The strided accesses of the column and
        # transposing kernels measured 1-9 % slower that way and keep plain global pointers.
        buf = spec.kind == "row1"
        self.GLD, self.GST = ("GLDU", "GSTU") if buf else ("GLDG", "GSTG")
        self.GLDC = self.GLD            # cached load of the same form (re-reads of a tile just stored)
        # Non-temporal variants for the tile data only (it is touched once); twiddles and the
        # checksum table are re-read by every tile and stay on the cached path.
        nt = int(spec.key.nt)
        if nt & 1:
            self.GLD += "N"
        if nt & 2:
            self.GST += "N"
        if role == "A":
            self.GST = "GSTG"       # the slot is meant to stay in the L2: default policy
        if role == "B":
            self.GLD = "GLDUS"      # agent-scope loads: a CU's L1 may still hold the slot's previous contents
        self.TWL, self.TWLU = ("TWLD", "TWLDU") if buf else ("TWLG", "TWLGU")

    def pair_access(self) -> bool:
        """Whether a thread reads and writes its elements two at a time (one 128-bit access)
        when the buffer is aligned to 16 bytes: fp32 kernels whose threads hold whole
        transforms, where a lane's elements are contiguous in memory.  fp64 elements already
        fill a 128-bit access."""
        sp = self.s
        return sp.kind == "row1" and sp.Tr == 1 and self.T2 == "float2" and sp.n % 2 == 0

    # ---------- literals ----------
    def lit(self, v: float) -> str:
        if self.R == "float":
            t = "%.9g" % v
            if "." not in t and "e" not in t and "n" not in t:
                t += ".0"
            return t + "f"
        t = "%.17g" % v
        if "." not in t and "e" not in t and "n" not in t:
            t += ".0"
        return t

    # ---------- thread map ----------
    def map_vars(self, c: Code, q: int):
        sp = self.s
        xn = "x"
        if sp.xl and q == sp.npass_lds - 1:
            xn = "xraw"
        t = "tx"
        if sp.threads >= 1024 or sp.n * (2 if self.R == "float" else 4) >= 128:
            # Everything derived from the thread index (LDS addresses, table indices, lane
            # offsets) is the same for every tile, and LLVM hoists it all out of the tile loop:
            # dozens of registers live across the whole kernel, 20-60 of them spilled under the
            # 128-register cap of a 1024-thread block.  An opaque copy per phase makes each phase
            # recompute its few shifts and masks instead (kernels with room for the hoisted
            # values measured 2-6 % slower that way and keep the plain index).  Kernels whose
            # elements alone fill 128 registers per lane get the same treatment.
            c("unsigned txq = tx; OPAQUE(txq);")
            t = "txq"
        if sp.maps[q] == "major":
            c(f"const unsigned s = {t} >> {ilog2(sp.Tr)}, {xn} = {t} & {sp.Tr - 1}u;")
        else:
            c(f"const unsigned s = {t} & {sp.BS - 1}u, {xn} = {t} >> {ilog2(sp.BS)};")
        if xn == "xraw":
            # the RL partners of the cross-lane pass are adjacent lanes: sub-index j = xraw % RL,
            # completed digits low = xraw / RL; x is the row position low + P*j the pass works on
            c(f"const unsigned x = (xraw >> {ilog2(sp.RL)}) + ((xraw & {sp.RL - 1}u) << {ilog2(sp.P[q])});")

    def lds_index(self, expr: str, pad: Tuple[int, int]) -> str:
        ps, pl = pad
        if ps < 0:
            return expr
        return f"(({expr}) + ((({expr}) >> {ps}) << {pl}))"

    def lds_index_at(self, base: str, base_phys: str, off: int, pad: Tuple[int, int]) -> str:
        """Padded index of base + off, where base_phys names the padded index of base.  An offset
        that is a multiple of the padding period moves the padded index by a constant (the shift
        drops none of its bits), which the compiler cannot see for itself in a 1024-thread block
        and otherwise recomputes per element (four integer instructions per LDS access)."""
        ps, pl = pad
        if ps < 0 or off % (1 << ps):
            return self.lds_index(f"{base} + {off}u", pad)
        return f"({base_phys} + {off + ((off >> ps) << pl)}u)"

    # ---------- radix-R DIF in registers ----------
    def emit_radix(self, c: Code, regs: Sequence[int]):
        R = len(regs)
        length = R
        while length >= 2:
            half = length // 2
            for b0 in range(0, R, length):
                for k in range(half):
                    a, b = regs[b0 + k], regs[b0 + k + half]
                    c(f"t = r[{a}]; r[{a}] = cadd(t, r[{b}]); t = csub(t, r[{b}]);")
                    # multiply the difference by W_length^k = exp(-2 pi i k/length)
                    if k == 0:
                        c(f"r[{b}] = t;")
                    elif 4 * k == length:
                        c(f"r[{b}] = cmul_mi(t);")
                    else:
                        ang = -2.0 * math.pi * k / length
                        c(f"r[{b}] = cmulc(t, {self.lit(math.cos(ang))}, {self.lit(math.sin(ang))});")
            length = half

    # ---------- twiddle powers ----------
    def emit_apply_powers(self, c: Code, count: int, pow2: Dict[int, str], targets: Sequence[Optional[int]],
                          base: Optional[str] = None):
        """Multiply r[targets[e]] by base * w^e for e < count, where pow2[b]
        names w^(2^b).  Products have depth <= log2(count)."""
        lo_n = min(count, 8)
        lo_bits = ilog2(lo_n)
        wl: Dict[int, Optional[str]] = {0: base}
        c("{")
        c.ind += 1
        for l in range(1, lo_n):
            hb = l.bit_length() - 1
            rest = l - (1 << hb)
            prev = wl[rest]
            nm = f"wl{l}"
            if prev is None:
                c(f"const {self.T2} {nm} = {pow2[hb]};")
            else:
                c(f"const {self.T2} {nm} = cmul({prev}, {pow2[hb]});")
            wl[l] = nm
        for h in range(count // lo_n):
            wh = None
            if h:
                bits = [b for b in range(8) if (h >> b) & 1]
                terms = [pow2[lo_bits + b] for b in bits]
                if len(terms) == 1:
                    wh = terms[0]
                else:
                    c(f"const {self.T2} wh{h} = cmul({terms[0]}, {terms[1]});" if len(terms) == 2 else
                      f"const {self.T2} wh{h} = cmul(cmul({terms[0]}, {terms[1]}), {terms[2]});")
                    wh = f"wh{h}"
            for l in range(lo_n):
                e = h * lo_n + l
                tgt = targets[e]
                if tgt is None:
                    continue
                a, b = wl[l], wh
                if a is None and b is None:
                    continue
                if a is None:
                    w = b
                elif b is None:
                    w = a
                else:
                    w = f"cmul({a}, {b})"
                c(f"r[{tgt}] = cmul(r[{tgt}], {w});")
        c.ind -= 1
        c("}")

    # ---------- one FFT pass (butterflies + block twiddle) ----------
    def emit_pass_compute(self, c: Code, q: int):
        sp = self.s
        R = sp.passes[q]
        U = sp.n // R
        lR = ilog2(R)
        last = q == sp.npass - 1
        M = sp.Ni // sp.P[q]
        c(f"// pass {q}: radix {R}, {U} butterfl{'y' if U == 1 else 'ies'} per thread, sub-FFT length {M}")
        if sp.tl:
            self.emit_tl_input(c, q)
        for u in range(U):
            self.emit_radix(c, [u + U * i for i in range(R)])
        if sp.tl:
            self.emit_tl_output(c, q)
        if last:
            return
        lP = ilog2(sp.P[q])
        for u in range(U):
            c("{")
            c.ind += 1
            # j does not depend on the tile, so the compiler would hoist the twiddle loads and
            # every product below out of the tile loop and keep them all in registers
            # (measured: +70 VGPRs on the 8192-point kernel); OPAQUE pins them inside the loop
            c(f"unsigned j = (x + {sp.Tr * u}u) >> {lP};")
            c("OPAQUE(j);")
            pow2 = {}
            for b in range(lR):
                Mb = M >> b
                c(f"const {self.T2} w{1 << b} = {self.TWLU}(tw, {Mb - 1}u, j);   // W_{M}^(j*{1 << b})")
                pow2[b] = f"w{1 << b}"
            targets = [u + U * bitrev(o, lR) for o in range(R)]
            targets[0] = None
            self.emit_apply_powers(c, R, pow2, targets)
            c.ind -= 1
            c("}")

    # ---------- thread-level verification ----------
    @staticmethod
    def tl_vectors(R: int):
        """Checksum vectors of a radix-R DFT: output side r[o % 3] (abft.h:22-28, with its float-rounded
        sqrt(3)/2) and input side c_R[i] = sum_o r[o % 3] W_R^(i o) (abft.h:45-60 with exact angles), each
        as the pair (re + im, re - im) that makes re+im of a product two multiply-adds."""
        s3 = 0.8660253882408142
        r = [complex(1.0, 0.0), complex(-0.5, -s3), complex(-0.5, s3)]
        cin = []
        for i in range(R):
            acc = 0j
            for o in range(R):
                ang = -2.0 * math.pi * ((i * o) % R) / R
                acc += r[o % 3] * complex(math.cos(ang), math.sin(ang))
            cin.append((acc.real + acc.imag, acc.real - acc.imag))
        rout = [(v.real + v.imag, v.real - v.imag) for v in r]
        return cin, rout

    def emit_tl_input(self, c: Code, q: int):
        """Before the butterflies of pass q: the thread's input-side sum over its U radix-R DFTs, then
        (first pass only) the compute-side error injection of fft_codegen.py:412-415."""
        sp = self.s
        R = sp.passes[q]
        U = sp.n // R
        cin, _ = self.tl_vectors(R)
        c(f"{self.R} tin = 0, tiy = 0, tout = 0, toy = 0;")
        c("if (!is_redo) {")
        c.ind += 1
        for u in range(U):
            for i in range(R):
                reg = u + U * i
                c(f"tin += r[{reg}].x * {self.lit(cin[i][0])}; tiy += r[{reg}].y * {self.lit(cin[i][1])};")
        if q == 0:
            # the injected element is one of the first Ni/n of its sub-FFT (register 0 of thread x = m;
            # the reference injects at m = 0), after the input-side sum has been taken
            c(f"r[0].x += (inj_hit && s == (unsigned)a.ft.inj_s && x == (unsigned)a.ft.inj_m) ? ({self.R})a.ft.inj_mag : ({self.R})0;")
        c.ind -= 1
        c("}")

    def emit_tl_output(self, c: Code, q: int):
        """After the butterflies of pass q and before its twiddles: the output-side sum and the thread's
        own verdict, |in - out| / (err_smoothing + |in| + |out|) > err_threshold (the rule of
        fft_codegen.py:495 on this thread's two sums)."""
        sp = self.s
        R = sp.passes[q]
        U = sp.n // R
        lR = ilog2(R)
        _, rout = self.tl_vectors(R)
        c("if (!is_redo) {")
        c.ind += 1
        for u in range(U):
            for o in range(R):
                reg = u + U * bitrev(o, lR)
                c(f"tout += r[{reg}].x * {self.lit(rout[o % 3][0])}; toy += r[{reg}].y * {self.lit(rout[o % 3][1])};")
        c(f"const {self.R} ti = tin + tiy, to = tout + toy;")
        c(f"if (fabs(ti - to) / (({self.R})a.ft.err_smoothing + fabs(ti) + fabs(to)) > ({self.R})a.ft.err_threshold) tbad = true;")
        c.ind -= 1
        c("}")
        c("(void)tin; (void)tiy; (void)tout; (void)toy;")

    def emit_lds_write(self, c: Code, q: int, part: str = ""):
        """Store the outputs of pass q in the layout pass q+1 reads
        (part = ".x" / ".y" for one round of a split exchange)."""
        sp = self.s
        R = sp.passes[q]
        U = sp.n // R
        lR = ilog2(R)
        P = sp.P[q]
        lP = ilog2(P)
        pad = sp.pads[q]
        nxt = sp.maps[q + 1]
        for u in range(U):
            c("{")
            c.ind += 1
            c(f"const unsigned rest = x + {sp.Tr * u}u;")
            c(f"const unsigned pos0 = (rest & {P - 1}u) + ((rest >> {lP}) << {lP + lR});")
            if nxt == "major":
                c(f"const unsigned a0 = (s << {ilog2(sp.Ni)}) + pos0;")
                step = P
            else:
                c(f"const unsigned a0 = s + (pos0 << {ilog2(sp.BS)});")
                step = P * sp.BS
            if pad[0] >= 0:
                c(f"const unsigned a0p = {self.lds_index('a0', pad)};")
            for o in range(R):
                reg = u + U * bitrev(o, lR)
                c(f"LST({self.lds_index_at('a0', 'a0p', step * o, pad)}, r[{reg}]{part});")
            c.ind -= 1
            c("}")

    def emit_lds_read(self, c: Code, q: int, part: str = ""):
        sp = self.s
        pad = sp.pads[q - 1]
        if sp.maps[q] == "major":
            c(f"const unsigned b0 = (s << {ilog2(sp.Ni)}) + x;")
            step = sp.Tr
        else:
            c("const unsigned b0 = tx;")
            step = sp.threads
        if pad[0] >= 0:
            c(f"const unsigned b0p = {self.lds_index('b0', pad)};")
        for e in range(sp.n):
            c(f"r[{e}]{part} = LLD({self.lds_index_at('b0', 'b0p', step * e, pad)});")

    # ---------- global addressing ----------
    def emit_tile_decode(self, c: Code, tile: str = "tile", sfx: str = ""):
        """Wave-uniform part of the tile's addresses (64-bit, lives in SGPRs)."""
        sp = self.s
        lBS = ilog2(sp.BS)
        lNi = ilog2(sp.Ni)
        if sp.kind == "row1":
            c(f"const long long row0{sfx} = ({tile}) << {lBS};")
            c(f"const long long ubase{sfx} = row0{sfx} << {lNi};")
        elif sp.kind == "col":
            c(f"const unsigned tpl{sfx} = (unsigned)a.log_ncols - {lBS}u;")
            c(f"const unsigned ct{sfx} = (unsigned)(({tile}) & ((1ll << tpl{sfx}) - 1));")
            c(f"const long long outer{sfx} = ({tile}) >> tpl{sfx};")
            c(f"const long long ubase{sfx} = (outer{sfx} << ({lNi} + a.log_ncols)) + ((long long)ct{sfx} << {lBS});")
            c(f"const long long gstep{sfx} = {sp.Tr}ll << a.log_ncols;")
            if self.role == "A":
                c(f"const long long ubase_st{sfx} = ubase{sfx} - piece_base;")
        else:
            c(f"const unsigned ctl{sfx} = (unsigned)a.logC - {lBS}u;")
            c(f"const unsigned ct{sfx} = (unsigned)(({tile}) & ((1ll << ctl{sfx}) - 1));")
            c(f"const unsigned qd{sfx} = (unsigned)((({tile}) >> ctl{sfx}) & ((1ll << a.logQ) - 1));")
            c(f"const long long tb{sfx} = (({tile}) >> (ctl{sfx} + a.logQ)) << a.logN;")
            c(f"const long long ubase_in{sfx} = tb{sfx} + ((long long)(qd{sfx} + ((ct{sfx} << {lBS}) << a.logQ)) << {lNi});")
            c(f"const unsigned ls{sfx} = (unsigned)a.logN - {lNi}u;")
            c(f"const long long ubase_out{sfx} = tb{sfx} + (ct{sfx} << {lBS}) + ((long long)qd{sfx} << a.logC);")
            c(f"const long long gstep{sfx} = {sp.Tr}ll << ls{sfx};")
            if self.role == "B":
                c(f"const long long ubase_ld{sfx} = ubase_in{sfx} - piece_base;")
        names = {"row1": ["row0", "ubase"], "col": ["tpl", "ct", "outer", "ubase", "gstep"],
                 "rowT": ["ctl", "ct", "qd", "tb", "ubase_in", "ls", "ubase_out", "gstep"]}[sp.kind]
        c(" ".join(f"(void){n}{sfx};" for n in names))

    def emit_load(self, c: Code, dst: str = "r", sfx: str = "", elems: Optional[Sequence[int]] = None):
        """Loads of a tile's elements into dst[e]; `elems` restricts them to some of a thread's
        elements (one element per access, forward kernels)."""
        sp = self.s
        lNi = ilog2(sp.Ni)
        pairs = self.pair_access() and elems is None
        if elems is not None:
            assert not self.pair_access() and not int(sp.key.inv)
        es = list(elems) if elems is not None else list(range(sp.n))
        if sp.kind == "row1":
            c(f"const unsigned gi{sfx} = (s << {lNi}) + x;")
            if sp.BS > 1:
                c(f"if ((row0{sfx} + s) < a.nrows) {{")
                c.ind += 1
            if pairs:
                # a buffer that starts on an odd element takes the one-element accesses (uniform branch)
                c("if (((unsigned long long)in & 15ull) == 0ull) {")
                c.ind += 1
                for e in range(0, sp.n, 2):
                    c(f"{self.GLD}2(in, ubase{sfx}, {e}, gi{sfx}, {dst}[{e}], {dst}[{e + 1}]);")
                c.ind -= 1
                c("} else {")
                c.ind += 1
            for e in es:
                c(f"{dst}[{e}] = {self.GLD}(in, ubase{sfx}, {sp.Tr * e}, gi{sfx});")
            if pairs:
                c.ind -= 1
                c("}")
            if sp.BS > 1:
                c.ind -= 1
                c("} else {")
                c.ind += 1
                for e in es:
                    c(f"{dst}[{e}] = czero({dst}[0]);")
                c.ind -= 1
                c("}")
        elif sp.kind == "col":
            c(f"const unsigned gi{sfx} = s + (x << a.log_ncols);")
            for e in es:
                c(f"{dst}[{e}] = {self.GLD}(in, ubase{sfx}, {e} * gstep{sfx}, gi{sfx});")
        else:
            c(f"const unsigned gi{sfx} = ((s << a.logQ) << {lNi}) + x;")
            for e in es:
                c(f"{dst}[{e}] = {self.GLD}(in, {'ubase_ld' if self.role == 'B' else 'ubase_in'}{sfx}, {sp.Tr * e}, gi{sfx});")
        if int(sp.key.inv) and sp.kind in ("row1", "col"):
            # inverse plan, first launch: a forward transform of (im, re) is (im, re) of the
            # inverse one.  A compile-time exchange costs nothing (the loaded register pair is
            # simply read the other way round); as a run-time branch in the forward kernels it
            # measured 2-25 % slower.
            for e in range(sp.n):
                c(f"{dst}[{e}] = cswap({dst}[{e}]);")

    def out_reg(self, e: int) -> int:
        """Register that holds output k = x + Tr*e after the last pass."""
        sp = self.s
        R = sp.passes[-1]
        U = sp.n // R
        u, o = e % U, e // U
        return u + U * bitrev(o, ilog2(R))

    def emit_swap_out(self, c: Code):
        """Inverse plan, last launch: exchange the components of the results."""
        sp = self.s
        if int(sp.key.inv) and sp.kind in ("row1", "rowT"):
            for e in range(sp.n):
                c(f"r[{e}] = cswap(r[{e}]);")

    def emit_store(self, c: Code):
        sp = self.s
        lNi = ilog2(sp.Ni)
        self.emit_swap_out(c)
        if sp.kind == "row1":
            c(f"const unsigned go = (s << {lNi}) + x;")
            if sp.BS > 1:
                c("if ((row0 + s) < a.nrows) {")
                c.ind += 1
            if sp.dc:
                self.emit_patch_load(c, [f"{self.GLDC}(out, ubase, {sp.Tr * e}, go)" for e in range(sp.n)])
            if self.pair_access():
                c("if (((unsigned long long)out & 15ull) == 0ull) {")
                c.ind += 1
                for e in range(0, sp.n, 2):
                    c(f"{self.GST}2(out, ubase, {e}, go, r[{self.out_reg(e)}], r[{self.out_reg(e + 1)}]);")
                c.ind -= 1
                c("} else {")
                c.ind += 1
            for e in range(sp.n):
                c(f"{self.GST}(out, ubase, {sp.Tr * e}, go, r[{self.out_reg(e)}]);")
            if self.pair_access():
                c.ind -= 1
                c("}")
            if sp.BS > 1:
                c.ind -= 1
                c("}")
        elif sp.kind == "col":
            c("const unsigned col = (ct << %d) + s;" % ilog2(sp.BS))
            self.emit_interlaunch_twiddle(c)
            c("const unsigned go = s + (x << a.log_ncols);")
            if sp.dc:
                self.emit_patch_load(c, [f"{self.GLDC}(out, ubase, {e} * gstep, go)" for e in range(sp.n)])
            for e in range(sp.n):
                c(f"{self.GST}(out, {'ubase_st' if self.role == 'A' else 'ubase'}, {e} * gstep, go, r[{self.out_reg(e)}]);")
        else:
            c("const unsigned go = s + (x << ls);")
            if sp.dc:
                self.emit_patch_load(c, [f"{self.GLDC}(out, ubase_out, {e} * gstep, go)" for e in range(sp.n)])
            for e in range(sp.n):
                c(f"{self.GST}(out, ubase_out, {e} * gstep, go, r[{self.out_reg(e)}]);")

    def emit_patch_load(self, c: Code, loads: Sequence[str]):
        """Extra trip of a delayed-correction kernel: the registers hold the correction term
        of the located tile; add what the tile's earlier trip stored, so that the stores that
        follow write the patched result."""
        sp = self.s
        c("if (is_redo && !hold) {")
        c.ind += 1
        c(f"{self.T2} pv[{sp.n}];")
        for e, ld in enumerate(loads):
            c(f"pv[{e}] = {ld};")
        for e in range(sp.n):
            c(f"r[{self.out_reg(e)}] = cadd(r[{self.out_reg(e)}], pv[{e}]);")
        c.ind -= 1
        c("}")

    def emit_interlaunch_twiddle(self, c: Code):
        """r[k] *= W_(Ni*ncols)^(col*k), k = x + Tr*e: base and step come from the
        two-level table, powers of the step by squaring."""
        sp = self.s
        n = sp.n
        c("{")
        c.ind += 1
        c(f"const unsigned L = {ilog2(sp.Ni)}u + (unsigned)a.log_ncols;")
        c("const unsigned emask = (L >= 32u) ? 0xffffffffu : ((1u << L) - 1u);")
        c("const unsigned lomask = (1u << a.tw_lo_bits) - 1u;")
        c("const unsigned e0 = (col * x) & emask;")
        c(f"const unsigned e1 = (col * {sp.Tr}u) & emask;")
        c(f"const {self.T2} wb = cmul({self.TWL}(twhi, e0 >> a.tw_lo_bits), {self.TWL}(twlo, e0 & lomask));")
        pow2 = {}
        if n > 1:
            c(f"const {self.T2} d1 = cmul({self.TWL}(twhi, e1 >> a.tw_lo_bits), {self.TWL}(twlo, e1 & lomask));")
            pow2[0] = "d1"
            for b in range(1, ilog2(n)):
                c(f"const {self.T2} d{1 << b} = cmul(d{1 << (b - 1)}, d{1 << (b - 1)});")
                pow2[b] = f"d{1 << b}"
        targets = [self.out_reg(e) for e in range(n)]
        self.emit_apply_powers(c, n, pow2, targets, base="wb")
        c.ind -= 1
        c("}")

    # ---------- fault tolerance ----------
    def ft_table_resident(self) -> bool:
        """Whether a thread keeps its n checksum-table entries in registers for all the tiles
        of its block: they are the same for every tile, so the table is read once per block
        instead of once per tile (-5..6 % run time).  Not under the 128-register cap of a
        1024-thread block, where the extra registers spill, nor when the entries alone would
        take more than 64 registers."""
        if self.s.ck16:
            return self.s.threads < 1024 and int(self.s.key.ck) == 1          # n/2 packed words per thread
        return self.s.threads < 1024 and self.s.n * (2 if self.R == "float" else 4) <= 64

    def compact_kappa(self) -> Tuple[float, float]:
        """kappa = (1 - rho^Ni) / 2 with rho = exp(-2 pi i / 3): Ni = 1 (mod 3) for even log2 Ni,
        2 (mod 3) for odd."""
        k = ilog2(self.s.Ni) % 2 + 1
        ang = -2.0 * math.pi * k / 3.0
        return (1.0 - math.cos(ang)) / 2.0, -math.sin(ang) / 2.0

    def emit_ft_table_park(self, c: Code, sim: bool):
        """Block start, ck = 3: every thread reads its words of the compact table once and parks
        them in its own LDS slots; it reads them back for every tile (no barrier: a thread only
        ever touches its own slots).  Costs no register between tiles and no L2 traffic per tile."""
        sp = self.s
        pre = Code()
        self.map_vars(pre, 0)
        W = sp.ck_words
        pre(f"unsigned cw0[{W}];")
        for q in range(W):
            pre(f"cw0[{q}] = CKW(ck, {sp.Tr * q}u, x);")
        for g in range(W // 4):
            pre(f"{{ tfft_cw4 v; v.x = cw0[{4 * g}]; v.y = cw0[{4 * g + 1}]; v.z = cw0[{4 * g + 2}]; v.w = cw0[{4 * g + 3}]; CWL_ST({sp.cw_off_bytes}, {g * sp.threads}u + tx, v); }}")
        pre("(void)s;")
        c("if (it0 < it1) {")
        c.ind += 1
        self.thread_block(c, sim, pre.text())
        c.ind -= 1
        c("}")

    def emit_ft_table_resident_load(self, c: Code, sim: bool):
        sp = self.s
        pre = Code()
        self.map_vars(pre, 0)
        if sp.ck16:
            for q in range(sp.n // 2 if self.R == "float" else sp.n):
                pre(f"cwr[{q}] = CKW(ck, {sp.Tr * q}u, x);")
        else:
            for e in range(sp.n):
                pre(f"cvr[{e}] = {self.TWLU}(ck, {sp.Tr * e}u, x);")
        pre("(void)s;")
        c("if (it0 < it1) {")
        c.ind += 1
        self.thread_block(c, sim, pre.text())
        c.ind -= 1
        c("}")

    def emit_ft_table_load(self, c: Code):
        """Lane index of the per-tile table reads (kernels that do not keep the table in
        registers).  Opaque, so that the reads stay inside the tile loop."""
        if self.ft_table_resident():
            return
        if self.s.ck_lds:
            c("unsigned txc = tx;")
            c("OPAQUE(txc);")
            return
        c("unsigned xc = x;")
        c("OPAQUE(xc);")

    def emit_ft_input(self, c: Code):
        """in1 += re+im of x*c[m]; in2 += cnt * (...)   (fft_codegen.py:354-367),
        then the optional compute-side error injection (:412-415).
        re+im of x*c = x.re*(c.re+c.im) + x.im*(c.re-c.im): the table holds the two
        real factors, so an element costs two fused multiply-adds."""
        sp = self.s
        c("if (!is_redo) {")
        c.ind += 1
        # two independent multiply-add chains (one per component): two operations per element;
        # a single `acc += a*b + c*d` costs three, since the sum may not be reassociated
        c(f"{self.R} acc = 0, acy = 0;")
        if sp.ck16:
            # Compact table.  With the exact cube root rho the input-side vector has the closed form
            #   c[m] = (1 - rho^Ni) / (1 - rho W^m) = kappa (1 - i t[m]),  t[m] = cot(pi (m/Ni + 1/3)),
            # so one real number per element carries it: re+im of x c = kp*(sum x.re + sum t x.im)
            # + kq*(sum x.im - sum t x.re) with kp, kq = re kappa +- im kappa.  fp32 kernels store t in
            # half precision, two elements of a thread per 32-bit word (word [x + Tr*q] holds elements
            # x + Tr*2q and x + Tr*(2q+1)): 16 KiB for 8192 points, a quarter of the complex table;
            # fp64 kernels store it in single precision, one word per element.  Small enough to be
            # read again for every tile, or cheap enough to keep (n/2 or n registers per thread).
            kr, ki = self.compact_kappa()
            c(f"{self.R} sa = 0, sb = 0, sc = 0, sd = 0;")
            B = 8
            half = self.R == "float"       # fp32: two half-precision values per word; fp64: one float per word
            W = sp.n // 2 if half else sp.n
            def use(word: str, q: int):
                if half:
                    for h, e in ((0, 2 * q), (1, 2 * q + 1)):
                        c(f"{{ const float tt = CKH({word}, {h}); sa += r[{e}].x; sb += r[{e}].y; sc += tt * r[{e}].y; sd += tt * r[{e}].x; }}")
                else:
                    c(f"{{ const double tt = (double)CKF({word}); sa += r[{q}].x; sb += r[{q}].y; sc += tt * r[{q}].y; sd += tt * r[{q}].x; }}")
            if self.ft_table_resident():
                for q in range(W):
                    use(f"cwr[{q}]", q)
            elif sp.ck_lds:
                c(f"unsigned cw[{W}];")
                for g in range(W // 4):
                    c(f"{{ const tfft_cw4 v = CWL_LD({sp.cw_off_bytes}, {g * sp.threads}u + txc); cw[{4 * g}] = v.x; cw[{4 * g + 1}] = v.y; cw[{4 * g + 2}] = v.z; cw[{4 * g + 3}] = v.w; }}")
                for q in range(W):
                    use(f"cw[{q}]", q)
            else:
                c(f"unsigned cw[{B}];")
                for b0 in range(0, W, B):
                    hi = min(W, b0 + B)
                    for q in range(b0, hi):
                        c(f"cw[{q - b0}] = CKW(ck, {sp.Tr * q}u, xc);")
                    c("SCHED_FENCE();")
                    for q in range(b0, hi):
                        use(f"cw[{q - b0}]", q)
                    c("SCHED_FENCE();")
            c(f"acc = {self.lit(kr + ki)} * (sa + sc) + {self.lit(kr - ki)} * (sb - sd);")
            c("(void)acy;")
        elif self.ft_table_resident():
            for e in range(sp.n):
                c(f"acc += r[{e}].x * cvr[{e}].x; acy += r[{e}].y * cvr[{e}].y;")
        else:
            # The table is fetched after the data in batches of 8 (a 1024-thread block leaves
            # 128 registers per lane), every load of a batch issued back to back and waited for
            # once.  Left to itself the compiler alternates load / wait / use per element, a
            # chain of n L2 round trips per tile.
            B = 8
            c(f"{self.T2} cv[{B}];")
            for b0 in range(0, sp.n, B):
                for e in range(b0, min(sp.n, b0 + B)):
                    c(f"cv[{e - b0}] = {self.TWLU}(ck, {sp.Tr * e}u, xc);")
                c("SCHED_FENCE();")
                for e in range(b0, min(sp.n, b0 + B)):
                    c(f"acc += r[{e}].x * cv[{e - b0}].x; acy += r[{e}].y * cv[{e - b0}].y;")
                c("SCHED_FENCE();")
        if not sp.ck16:
            c("acc += acy;")
        c("fin1 += acc; fin2 += cntf * acc;")
        if sp.dc:
            # per-thread sum of the group's inputs (fft_codegen.py:355-357), taken before the injection
            for e in range(sp.n):
                c(f"sx[{e}] = cadd(sx[{e}], r[{e}]);")
        # the injected element is one of the first Ni/n of its sub-FFT (register 0 of thread
        # x = m; the reference injects at m = 0)
        c(f"r[0].x += (inj_hit && s == (unsigned)a.ft.inj_s && x == (unsigned)a.ft.inj_m) ? ({self.R})a.ft.inj_mag : ({self.R})0;")
        c.ind -= 1
        c("}")

    def emit_ft_output(self, c: Code):
        """out1 -= re+im of y*r[k%3]; out2 -= cnt * (...)   (fft_codegen.py:374-384),
        taken before the inter-launch twiddle.  re+im of y*r = y.re*(r.re+r.im) +
        y.im*(r.re-r.im); the three (sum, difference) pairs are rotated by x % 3 once."""
        sp = self.s
        c("if (!is_redo) {")
        c.ind += 1
        c("const unsigned x3 = x % 3u;")
        s3 = 0.8660253882408142
        pq = [(1.0, 1.0), (-0.5 - s3, -0.5 + s3), (-0.5 + s3, -0.5 - s3)]      # r[0], r[1], r[2]
        for cc in range(3):
            # element class cc uses r[(x3 + cc) % 3]
            sel = [pq[(v + cc) % 3] for v in range(3)]
            c(f"const {self.R} rp{cc} = (x3 == 0u) ? {self.lit(sel[0][0])} : ((x3 == 1u) ? {self.lit(sel[1][0])} : {self.lit(sel[2][0])});")
            c(f"const {self.R} rq{cc} = (x3 == 0u) ? {self.lit(sel[0][1])} : ((x3 == 1u) ? {self.lit(sel[1][1])} : {self.lit(sel[2][1])});")
        c(f"{self.R} acc = 0, acy = 0;")
        for e in range(sp.n):
            ce = (sp.Tr * e) % 3
            reg = self.out_reg(e)
            c(f"acc += r[{reg}].x * rp{ce}; acy += r[{reg}].y * rq{ce};")
        c("acc += acy;")
        c("fo1 -= acc; fo2 -= cntf * acc;")
        if sp.dc:
            # per-thread sum of the group's outputs as computed, before the inter-launch twiddle
            # (fft_codegen.py:421-423)
            for e in range(sp.n):
                c(f"sy[{e}] = cadd(sy[{e}], r[{self.out_reg(e)}]);")
        c.ind -= 1
        c("}")
        if sp.dc:
            # extra trip: the registers hold FFT(sum of the group's inputs); what the located tile's
            # stored result lacks is that minus the sum of the group's outputs (fft_codegen.py:401-404,
            # 427-429; the notebook's b_out += FFT(A e) - B_out e with unit weights)
            # (a group of one tile is checked before it is stored: its extra trip simply
            # transforms the saved input again and stores that)
            c("else if (!hold) {")
            c.ind += 1
            for e in range(sp.n):
                c(f"r[{self.out_reg(e)}] = csub(r[{self.out_reg(e)}], sy[{e}]);")
            c.ind -= 1
            c("}")

    # ---------- phases ----------
    def emit_xlane_pass(self, c: Code, q: int) -> List[str]:
        """The last radix-RL DFT across RL adjacent lanes, on every register:
        log2(RL) radix-2 DIF stages, partner = lane ^ half through DPP quad
        permutes (half 1, 2) or ds_swizzle (half 4).  Lane j ends with output
        digit bitrev(j).  Returns the phase texts (the lock-step CPU flavour
        needs a thread-loop boundary before each stage)."""
        sp = self.s
        RL, n = sp.RL, sp.n
        out = []
        length = RL
        while length >= 2:
            half = length // 2
            st = Code()
            self.map_vars(st, q)
            st("(void)x; (void)s;")
            st(f"// cross-lane stage: span {length}, partner = lane ^ {half}")
            st("{")
            st.ind += 1
            st(f"const unsigned jj = xraw & {length - 1}u;")
            st(f"const bool hi = (jj & {half}u) != 0u;")
            st(f"const {self.R} sg = hi ? ({self.R})-1 : ({self.R})1;")
            if length > 2:
                # upper lanes multiply by W_length^(jj - half)
                st(f"{self.R} wr = 1, wi = 0;")
                for kk in range(1, half):
                    ang = -2.0 * math.pi * kk / length
                    st(f"if (jj == {half + kk}u) {{ wr = {self.lit(math.cos(ang))}; wi = {self.lit(math.sin(ang))}; }}")
            st(f"{self.T2} pv;")
            for i in range(n):
                st(f"XLANE({i}, {half}, pv);")
                st(f"r[{i}].x = pv.x + sg * r[{i}].x; r[{i}].y = pv.y + sg * r[{i}].y;")
                if length > 2:
                    st(f"r[{i}] = cmulc(r[{i}], wr, wi);")
            st.ind -= 1
            st("}")
            out.append(st.text())
            length = half
        return out

    def emit_store_xlane(self, c: Code, q: int):
        """Store after the cross-lane pass: register o of lane j holds
        k = low + P*o + (Ni/RL)*bitrev(j)."""
        sp = self.s
        lNi = ilog2(sp.Ni)
        RL, L = sp.RL, ilog2(sp.RL)
        P = sp.P[q]
        lR = ilog2(sp.n)
        self.emit_swap_out(c)
        c(f"const unsigned jl = xraw & {RL - 1}u;")
        brev = {1: "jl", 2: "(((jl & 1u) << 1) | (jl >> 1))", 3: "(((jl & 1u) << 2) | (jl & 2u) | (jl >> 2))"}[L]
        c(f"const unsigned kb = (xraw >> {L}) + ({brev} << {lNi - L});")
        c(f"const unsigned go = (s << {lNi}) + kb;")
        if sp.BS > 1:
            c("if ((row0 + s) < a.nrows) {")
            c.ind += 1
        for o in range(sp.n):
            c(f"{self.GST}(out, ubase, {P * o}, go, r[{bitrev(o, lR)}]);")
        if sp.BS > 1:
            c.ind -= 1
            c("}")

    def phases(self) -> List[Tuple[str, str]]:
        """Phases of one tile as (separator before, text).  Separator "barrier"
        is a block barrier; "lane" is nothing on the GPU (lanes of a wavefront
        run in lock step) and a thread-loop boundary in the CPU flavour.
        A complex exchange is [compute] b [write] b [read, compute ...]; a split
        exchange is [compute] b [write re] b [read re] b [write im] b [read im,
        compute ...]: the new real parts land in the .x registers whose old
        contents have all been written, while the .y registers still hold the
        old imaginary parts, so no extra registers are needed."""
        sp = self.s
        out: List[Tuple[str, str]] = []
        for q in range(sp.npass_lds):
            c = Code()
            self.map_vars(c, q)
            c(f"{self.T2} t;")
            if q == 0 and sp.tl:
                c("tbad = false;")
            if q == 0 and sp.pfk:
                # the first pfk elements were fetched during the previous tile's last pass
                for e in range(sp.pfk):
                    c(f"r[{e}] = rn[{e}];")
                c("{")
                c.ind += 1
                self.emit_load(c, "r", "", elems=range(sp.pfk, sp.n))
                c.ind -= 1
                c("}")
            elif q == 0:
                if sp.pf:
                    # this tile's elements were fetched during the previous tile; start the
                    # fetch of the next one now so it overlaps every pass of this tile
                    for e in range(sp.n):
                        c(f"r[{e}] = rn[{e}];")
                    if sp.ft:
                        self.emit_ft_table_load(c)
                        self.emit_ft_input(c)
                    c("if (has_next) {")
                    c.ind += 1
                    self.emit_tile_decode(c, "tile_n", "_n")
                    self.emit_load(c, "rn", "_n")
                    c.ind -= 1
                    c("}")
                else:
                    if sp.ft:
                        self.emit_ft_table_load(c)
                    # A wave that is about to fetch its tile goes first: the loads of a block that
                    # has just started are issued before the arithmetic of the blocks already
                    # resident gets the slot.  Measured per size; a policy bit of the plan row.
                    prio = bool(int(sp.key.nt) & 4)
                    if prio:
                        c("TFFT_WAVE_PRIO(3);")
                    if sp.dc:
                        c("if (!is_redo) {")
                        c.ind += 1
                    if self.role == "A" and self.prefetched:
                        c("if (use_rn) {")
                        for e in range(sp.n):
                            c(f"    r[{e}] = rn[{e}];")
                        c("} else {")
                        c.ind += 1
                    self.emit_load(c)
                    if self.role == "A" and self.prefetched:
                        c.ind -= 1
                        c("}")
                    if self.role == "B" and os.environ.get("TFFT_PAIR_PROFILE"):
                        c("TFFT_WAIT_VMEM();")
                        c("if (f.prof) { const long long now_ = (long long)wall_clock64(); pt[7] += now_ - pt_last; pt_last = now_; }")
                    if sp.dc:
                        c.ind -= 1
                        c("} else {")
                        c.ind += 1
                        for e in range(sp.n):
                            c(f"r[{e}] = sx[{e}];")
                        c.ind -= 1
                        c("}")
                    if prio:
                        c("TFFT_WAVE_PRIO(0);")
                    if sp.ft:
                        self.emit_ft_input(c)
            else:
                if sp.pfk and q == sp.npass_lds - 1:
                    # start on the next tile while this one runs its last pass: a 1024-thread block
                    # is alone on its CU and would otherwise have nothing in flight while it computes
                    c("if (has_next) {")
                    c.ind += 1
                    if sp.maps[q] != sp.maps[0]:
                        # a tile is loaded with the thread map of its first pass (this scope's s and x)
                        self.map_vars(c, 0)
                    self.emit_tile_decode(c, "tile_n", "_n")
                    self.emit_load(c, "rn", "_n", elems=range(sp.pfk))
                    c.ind -= 1
                    c("}")
                self.emit_lds_read(c, q, ".y" if sp.split else "")
            self.emit_pass_compute(c, q)
            if q == sp.npass_lds - 1:
                if sp.xl:
                    c("(void)t;")
                    stages = self.emit_xlane_pass(c, q)
                    out.append(("barrier", c.text()))
                    for i, st in enumerate(stages):
                        # (the CPU flavour snapshots every thread's registers in a phase of
                        # its own, so that no thread sees a partner that already moved on)
                        out.append(("lane", "SNAP();\n"))
                        if i == len(stages) - 1:
                            fin = Code()
                            fin(st.rstrip("\n"))
                            self.emit_store_xlane(fin, q)
                            out.append(("lane", fin.text()))
                        else:
                            out.append(("lane", st))
                    continue
                if sp.ft:
                    self.emit_ft_output(c)
                if sp.tl:
                    # The tile waits in registers for the block's verdict: every wavefront leaves a word that
                    # says whether one of its threads objected, the block reads them all behind a barrier
                    # (separator "vote", emitted by emit()), and only an accepted tile -- or the recomputed
                    # one -- is stored.
                    c("(void)t;")
                    c(f"TL_VOTE({sp.red_off_bytes + (3 * (sp.threads // WAVE) * 8 if sp.ft else 0)}, tbad);")
                    out.append(("barrier", c.text()))
                    st = Code()
                    self.map_vars(st, q)
                    st("(void)x; (void)s;")
                    st("if (is_redo || !(tany && a.ft.correct)) {")
                    st.ind += 1
                    self.emit_store(st)
                    st.ind -= 1
                    st("}")
                    out.append(("vote", st.text()))
                    continue
                if sp.dc:
                    # the only tile of a group is held back until the group has been checked
                    c("if (!hold || is_redo) {")
                    c.ind += 1
                self.emit_store(c)
                if sp.dc:
                    c.ind -= 1
                    c("}")
                c("(void)t;")
                out.append(("barrier", c.text()))
            else:
                c("(void)t;")
                out.append(("barrier", c.text()))
                if not sp.split:
                    w = Code()
                    self.map_vars(w, q)
                    self.emit_lds_write(w, q)
                    out.append(("barrier", w.text()))
                else:
                    w = Code()
                    self.map_vars(w, q)
                    self.emit_lds_write(w, q, ".x")
                    out.append(("barrier", w.text()))
                    rd = Code()
                    self.map_vars(rd, q + 1)
                    self.emit_lds_read(rd, q + 1, ".x")
                    out.append(("barrier", rd.text()))
                    w = Code()
                    self.map_vars(w, q)
                    self.emit_lds_write(w, q, ".y")
                    out.append(("barrier", w.text()))
        return out

    # ---------- whole kernel ----------
    def emit(self, sim: bool) -> str:
        sp = self.s
        c = Code()
        T2, R = self.T2, self.R
        c(f"// {sp.name}: {sp.kind} kernel, {T2}, Ni={sp.Ni}, BS={sp.BS}, n={sp.n}, passes={'x'.join(map(str, sp.passes))},")
        c(f"// {sp.threads} threads, LDS {sp.lds_bytes} B{' (split re/im exchange)' if sp.split else ''}{', next-tile prefetch' if sp.pf else ''}{', cross-lane last pass' if sp.xl else ''}, thread maps {sp.maps}, pads {sp.pads}{', fault tolerant' + (' (delayed batch correction)' if sp.dc else '') if sp.ft else ''}{', thread-level verification' if sp.tl else ''}")
        if sim:
            c(f'extern "C" void {sp.name}_sim(const {T2}* in, {T2}* out, const {T2}* tw, const tfft_kargs* ap, long long grid, const long long* limits)')
            c("{")
            c.ind += 1
            c("const tfft_kargs a = *ap;")
            c("const long long in_limit = limits[0], out_limit = limits[1], tw_limit = limits[2];")
            c("const long long twhi_limit = limits[3], twlo_limit = limits[4], ck_limit = limits[5];")
            c(f"const long long lds_limit = {sp.lds_elems};")
            c("(void)in_limit; (void)out_limit; (void)tw_limit; (void)twhi_limit; (void)twlo_limit; (void)ck_limit; (void)lds_limit;")
            c(f"struct TS {{ {T2} r[{sp.n}]; {T2} rn[{sp.n}]; {T2} sh[{sp.n}]; {T2} cvr[{sp.n}]; unsigned cwr[{sp.n}]; {T2} sx[{sp.n}]; {T2} sy[{sp.n}]; {R} fin1, fin2, fo1, fo2; bool tbad; }};")
            c("for (long long pbx = 0; pbx < grid; ++pbx) {")
            c.ind += 1
            c("long long bx = pbx; const long long pbx_raw = pbx; (void)pbx_raw;")
            LT = R if sp.split else T2
            c(f"std::vector<{LT}> ldsv({sp.lds_elems}); {LT}* lds = ldsv.data();")
            c(f"std::vector<TS> ts({sp.threads}); for (auto& z : ts) z = TS();")
            c(f"std::vector<tfft_cw4> cwlv({max(1, sp.ck_words // 4 * sp.threads if sp.ck_lds else 1)}); tfft_cw4* cwl = cwlv.data(); const long long cwl_limit = (long long)cwlv.size(); (void)cwl; (void)cwl_limit;")
        else:
            wv = int(sp.key.wv)
            c(f'extern "C" __global__ __launch_bounds__({sp.threads})' + (f" __attribute__((amdgpu_waves_per_eu({wv}, {wv})))" if wv else ""))
            c(f"void {sp.name}(const {T2}* __restrict__ in, {T2}* __restrict__ out, const {T2}* __restrict__ tw, const tfft_kargs a)")
            c("{")
            c.ind += 1
            c("extern __shared__ __align__(16) unsigned char lds_raw[];")
            LT = R if sp.split else T2
            c(f"{LT}* lds = ({LT}*)lds_raw;")
            c("const unsigned tx = threadIdx.x;")
            c("const long long grid = gridDim.x;")
            c("long long bx = blockIdx.x; const long long pbx_raw = blockIdx.x; (void)pbx_raw;")
            c(f"{T2} r[{sp.n}];")
            if sp.pf:
                c(f"{T2} rn[{sp.pfk or sp.n}];")
            if sp.tl:
                c("bool tbad = false;")
            if sp.ft:
                c(f"{R} fin1 = 0, fin2 = 0, fo1 = 0, fo2 = 0;")
                if self.ft_table_resident():
                    c(f"unsigned cwr[{sp.n // 2 if R == 'float' else sp.n}];" if sp.ck16 else f"{T2} cvr[{sp.n}];")
                if sp.dc:
                    c(f"{T2} sx[{sp.n}], sy[{sp.n}];")
                    c(f"for (int e = 0; e < {sp.n}; ++e) {{ sx[e] = czero(sx[e]); sy[e] = czero(sy[e]); }}")
        # XCD-aware renumbering: hardware deals blocks round-robin to the 8 XCDs, so block
        # b runs on XCD b % 8.  Give every XCD chunks of `xcd_chunk` consecutive tiles (its
        # L2 then streams contiguous memory) while the 8 XCDs stay in one neighbourhood.
        # (block and tile counts fit 32 bits: the host rejects larger grids)
        c("if (a.xcd_chunk > 0) {")
        c("    const unsigned ub = (unsigned)bx, xc = (unsigned)a.xcd_chunk, span = 8u * xc, full = ((unsigned)grid / span) * span;")
        c("    if (ub < full) { const unsigned q = ub >> 3, xcd = ub & 7u; bx = (long long)((q / xc) * span + xcd * xc + q % xc); }")
        c("}")
        c(f"const {T2}* twhi = (const {T2}*)a.tw_hi; const {T2}* twlo = (const {T2}*)a.tw_lo; const {T2}* ck = (const {T2}*)a.ft.cksum;")
        c("(void)twhi; (void)twlo; (void)ck;")
        # tile group of this block (fft_codegen.py:218,260-261 with a rounded-up grid)
        parts = sp.ft and not sp.dc       # the group of a block may be shared with other blocks
        if parts:
            # a group walked by several blocks: block b is part b / groups of group b % groups
            c("long long ngroups = grid; unsigned part = 0;")
            c("if (a.ft.parts > 1) {")
            c("    const unsigned ng = (unsigned)grid / (unsigned)a.ft.parts, ub = (unsigned)bx;")
            c("    ngroups = ng; part = tfft_uni(ub / ng); bx = (long long)tfft_uni(ub % ng);")
            c("}")
        else:
            c("const long long ngroups = grid;")
        c("long long gstride = 1, tile0 = bx;")
        c("int count = bx < a.ntiles ? 1 : 0;")
        c("if (a.thread_bs > 1) {")
        c("    const unsigned ub = (unsigned)bx, gap = (unsigned)a.tb_gap, ug = (unsigned)ngroups, tbs = (unsigned)a.thread_bs;")
        c("    const unsigned chunk = ub / gap;")
        c("    const unsigned gs = ((chunk + 1u) * gap <= ug) ? gap : (ug - chunk * gap);")
        c("    const unsigned long long t0 = (unsigned long long)chunk * gap * tbs + ub % gap;")
        c("    gstride = gs; tile0 = (long long)t0; count = 0;")
        c("    if (tile0 < a.ntiles) { const unsigned left = (unsigned)((a.ntiles - tile0 + gs - 1) / gs); count = left < tbs ? (int)left : (int)tbs; }")
        c("}")
        # the tiles [it0, it1) of the group are this block's
        if parts:
            c("gstride = tfft_uni(gstride); tile0 = tfft_uni(tile0); count = tfft_uni(count);")
        c("int it0 = 0, it1 = count;")
        if parts:
            c("if (a.ft.parts > 1) { it0 = (int)part * a.ft.part_len; it1 = it0 + a.ft.part_len < count ? it0 + a.ft.part_len : count; if (it0 > it1) it0 = it1; }")
            # the fix-up launch: no tiles of its own, only queued ones (block b takes entries b, b + grid, ...)
            c("if (a.ft.fix_mode) { it0 = 0; it1 = 0; }")
        c("const long long tile_first = tile0 + it0 * gstride; (void)tile_first;")
        if sp.pf:
            c("if (it0 < it1) {")
            c.ind += 1
            self.emit_tile_decode(c, "tile_first", "_n")
            pre = Code()
            self.map_vars(pre, 0)
            self.emit_load(pre, "rn", "_n", elems=range(sp.pfk) if sp.pfk else None)
            self.thread_block(c, sim, pre.text())
            c.ind -= 1
            c("}")
        if sp.ft:
            # checksum groups run: one per block, counted once per launch by its first block
            if sim:
                c("if (pbx == 0 && !a.ft.fix_mode) a.ft.counters[0] += (unsigned long long)ngroups;")
            else:
                c("if (blockIdx.x == 0 && tx == 0 && !a.ft.fix_mode) atomicAdd(&a.ft.counters[0], (unsigned long long)ngroups);")
            c("long long redo_tile = -1; int extra = 0;")
            if parts:
                c("if (a.ft.fix_mode) { const long long nfix = (long long)a.ft.fix_ctl[0]; if (pbx_raw < nfix) extra = (int)((nfix - pbx_raw + grid - 1) / grid); }")
            if sp.dc:
                # A group of a single tile (thread_bs = 1, or a ragged last group) is verified
                # before its result leaves the registers: nothing is stored until the block has
                # decided, and a flagged tile is transformed again from the input the threads
                # still hold -- no second pass over HBM in either direction.
                c("const bool hold = count == 1 && a.ft.correct != 0;")
            if self.ft_table_resident():
                self.emit_ft_table_resident_load(c, sim)
            elif sp.ck_lds:
                self.emit_ft_table_park(c, sim)
            c("for (int it = it0; it < it1 + extra; ++it) {")
            c.ind += 1
            c("const bool is_redo = it >= it1;")
            if parts:
                c("if (is_redo && a.ft.fix_mode) redo_tile = a.ft.fix_list[pbx_raw + (long long)(it - it1) * grid];")
            c("const long long tile = is_redo ? redo_tile : tile0 + it * gstride;")
            c(f"const {R} cntf = ({R})(it + 1);")
            c("bool inj_hit = false;")
            c("if (a.ft.inj_mode == 1) inj_hit = (it == (int)(bx % a.thread_bs)) && (bx % a.ft.inj_every == 0);")
            c("else if (a.ft.inj_mode == 2) inj_hit = (tile % a.ft.inj_every) == a.ft.inj_tile;")
            c("(void)cntf; (void)inj_hit;")
        elif sp.tl:
            # tiles checked: one per tile, counted once per launch by its first block
            if sim:
                c("if (pbx == 0) a.ft.counters[0] += (unsigned long long)a.ntiles;")
            else:
                c("if (blockIdx.x == 0 && tx == 0) atomicAdd(&a.ft.counters[0], (unsigned long long)a.ntiles);")
            c("for (int it = it0; it < it1; ++it) {")
            c.ind += 1
            c("const long long tile = tile0 + it * gstride;")
            c("bool inj_hit = false;")
            c("if (a.ft.inj_mode == 1) inj_hit = (it == (int)(bx % a.thread_bs)) && (bx % a.ft.inj_every == 0);")
            c("else if (a.ft.inj_mode == 2) inj_hit = (tile % a.ft.inj_every) == a.ft.inj_tile;")
            c("(void)inj_hit;")
            # second trip: the tile is transformed again, unchecked, when a thread objected to the first
            c("for (int trip = 0; trip < 2; ++trip) {")
            c.ind += 1
            c("const bool is_redo = trip != 0;")
        else:
            c("for (int it = it0; it < it1; ++it) {")
            c.ind += 1
            c("const long long tile = tile0 + it * gstride;")
        if sp.pf:
            c("const bool has_next = it + 1 < it1;")
            c("const long long tile_n = tile0 + (long long)(it + 1) * gstride;")
            c("(void)has_next; (void)tile_n;")
        self.emit_tile_decode(c)
        phases = self.phases()
        for i, (sep, ph) in enumerate(phases):
            if i:
                if sim:
                    c(f"// ---- {sep} ----")
                elif sep in ("barrier", "vote"):
                    c("__syncthreads();")
            if sep == "vote":
                self.emit_tl_verdict(c, sim)
            self.thread_block(c, sim, ph)
        if sp.ft:
            self.emit_ft_decide(c, sim)
            if sp.dc:
                st = Code()
                self.map_vars(st, sp.npass_lds - 1)
                st("(void)x; (void)s;")
                st("if (hold && !is_redo && !extra) {")
                st.ind += 1
                self.emit_store(st)
                st.ind -= 1
                st("}")
                self.thread_block(c, sim, st.text())
            if sp.pf:
                # the tile to recompute is known only now: fetch it for the extra trip
                c("if (extra && it == it1 - 1) {")
                c.ind += 1
                self.emit_tile_decode(c, "redo_tile", "_n")
                pre = Code()
                self.map_vars(pre, 0)
                self.emit_load(pre, "rn", "_n")
                self.thread_block(c, sim, pre.text())
                c.ind -= 1
                c("}")
        if sp.tl:
            c("if (is_redo || !(tany && a.ft.correct)) break;")
            c.ind -= 1
            c("}")  # trip loop
        c.ind -= 1
        c("}")  # tile loop
        if parts:
            self.emit_ft_decide(c, sim, shared=True)
            # every block of the fix-up launch has read the queue length before it gets here
            if sim:
                c("if (a.ft.fix_mode && ++a.ft.fix_ctl[1] == (unsigned)grid) { a.ft.fix_ctl[0] = 0; a.ft.fix_ctl[1] = 0; }")
            else:
                c("if (a.ft.fix_mode) {")
                c("    __syncthreads();")
                c("    if (tx == 0 && atomicAdd(&a.ft.fix_ctl[1], 1u) == (unsigned)grid - 1u) { atomicExch(&a.ft.fix_ctl[0], 0u); atomicExch(&a.ft.fix_ctl[1], 0u); }")
                c("}")
        if sim:
            c.ind -= 1
            c("}")  # block loop
        c.ind -= 1
        c("}")
        return c.text()

    def thread_block(self, c: Code, sim: bool, body: str):
        """Per-thread code: a plain block on the GPU, a loop over the block's
        threads in the CPU lock-step flavour."""
        sp = self.s
        if sim:
            c(f"for (unsigned tx = 0; tx < {sp.threads}u; ++tx) {{")
            c.ind += 1
            c("auto& r = ts[tx].r; auto& rn = ts[tx].rn; auto& cvr = ts[tx].cvr; auto& cwr = ts[tx].cwr; auto& sx = ts[tx].sx; auto& sy = ts[tx].sy; auto& fin1 = ts[tx].fin1; auto& fin2 = ts[tx].fin2; auto& fo1 = ts[tx].fo1; auto& fo2 = ts[tx].fo2; auto& tbad = ts[tx].tbad;")
            c("(void)r; (void)rn; (void)cvr; (void)cwr; (void)sx; (void)sy; (void)fin1; (void)fin2; (void)fo1; (void)fo2; (void)tbad;")
        else:
            c(f"if (tx < {sp.threads}u) {{" if self.block_threads > sp.threads else "{")
            c.ind += 1
        c(body.rstrip("\n"))
        c.ind -= 1
        c("}")

    def emit_tile_body(self, c: Code, sim: bool, before_last=None, after_first=None):
        """One tile of a plain kernel: address decode, then the phases with their barriers.  `before_last`
        and `after_first` emit block-level code ahead of the tile's last phase (the one that stores) and
        behind its first (the one that loads)."""
        self.emit_tile_decode(c)
        phases = self.phases()
        for i, (sep, ph) in enumerate(phases):
            if i:
                if sim:
                    c(f"// ---- {sep} ----")
                elif sep == "barrier":
                    c("__syncthreads();")
            if before_last and i == len(phases) - 1:
                before_last()
            self.thread_block(c, sim, ph)
            if after_first and i == 0:
                after_first()

    def emit_tl_verdict(self, c: Code, sim: bool):
        """Thread-level verification, behind the barrier that follows a tile's last pass: did any thread of the
        block object?  A detection is counted and listed like one of the block-level scheme (one atomic on
        one of 64 counter lines); the tile is its own group, so it needs no locating."""
        sp = self.s
        nw = sp.threads // WAVE
        off = sp.red_off_bytes + (3 * nw * 8 if sp.ft else 0)
        if sim:
            c("bool tany = false; for (auto& z : ts) tany = tany || z.tbad;")
            c("if (tany && !is_redo) {")
        else:
            c("bool tany = false;")
            c(f"{{ const unsigned* tv = (const unsigned*)(lds_raw + {off}); unsigned tor = 0u; for (int w = 0; w < {nw}; ++w) tor |= tv[w]; tany = tfft_uni(tor) != 0u; }}")
            if sp.npass_lds < 2:
                # no other barrier separates this read from the next trip's votes
                c("__syncthreads();")
            c("if (tany && !is_redo && tx == 0) {")
        c.ind += 1
        c("const unsigned sub = (unsigned)(pbx_raw & 63);")
        c("unsigned long long* sc = a.ft.counters + TFFT_FT_SUB0 + TFFT_FT_SUB_STRIDE * sub;")
        c("const unsigned long long region = (unsigned long long)(a.ft.flagged_cap >> 6);")
        c("const unsigned long long slot = sc[0]++;" if sim else "const unsigned long long slot = atomicAdd(sc, 1ull);")
        c("if (slot < region) { long long* fl = a.ft.flagged + 2 * (sub * region + slot); fl[0] = a.ft.launch; fl[1] = tile; }")
        c.ind -= 1
        c("}")

    def emit_ft_handoff(self, c: Code, sim: bool):
        """A group shared by several blocks (a.ft.parts > 1), after the block's last tile: leave
        every thread's four running checksums in the group's slots, take a ticket; the block that
        takes the last ticket of the group adds the parts up in part order (so the sums do not
        depend on which block comes last) and goes on to decide for the whole group, every other
        block is done.  Nobody waits for anybody."""
        sp = self.s
        R = self.R
        T = sp.threads
        c("if (a.ft.parts > 1) {")
        c.ind += 1
        c(f"{R}* ps = ({R}*)a.ft.part_sums;")
        c("const unsigned nparts = (unsigned)((count + a.ft.part_len - 1) / a.ft.part_len);      // parts of this group that hold tiles")
        c(f"const unsigned long long slot0 = (unsigned long long)bx * (unsigned)a.ft.parts * {4 * T}ull;")
        if sim:
            c(f"for (unsigned tx = 0; tx < {T}u; ++tx) {{ {R}* q = ps + slot0 + (unsigned long long)part * {4 * T}ull + tx; q[0] = ts[tx].fin1; q[{T}] = ts[tx].fin2; q[{2 * T}] = ts[tx].fo1; q[{3 * T}] = ts[tx].fo2; }}")
            c("const unsigned ticket = a.ft.tickets[bx]++;")
            c("if (ticket != nparts - 1) break;")
            c("a.ft.tickets[bx] = 0;")
            c(f"for (unsigned tx = 0; tx < {T}u; ++tx) {{")
            c("    ts[tx].fin1 = ts[tx].fin2 = ts[tx].fo1 = ts[tx].fo2 = 0;")
            c(f"    for (unsigned pp = 0; pp < nparts; ++pp) {{ const {R}* q = ps + slot0 + (unsigned long long)pp * {4 * T}ull + tx; ts[tx].fin1 += q[0]; ts[tx].fin2 += q[{T}]; ts[tx].fo1 += q[{2 * T}]; ts[tx].fo2 += q[{3 * T}]; }}")
            c("}")
        else:
            c(f"{{ {R}* q = ps + slot0 + (unsigned long long)part * {4 * T}ull + tx; tfft_ps_store(q, fin1); tfft_ps_store(q + {T}, fin2); tfft_ps_store(q + {2 * T}, fo1); tfft_ps_store(q + {3 * T}, fo2); }}")
            # Ordering of the hand-off.  The sums are written with agent-scope atomic stores, which go
            # through the XCD's L2 to memory; a wave's vector-memory counter reaches zero only when every
            # store it issued has been acknowledged there.  __syncthreads() alone is a workgroup-scope
            # fence and is not required to wait for outstanding global stores, so each wave waits for its
            # own (TFFT_WAIT_VMEM) before the barrier; thread 0 takes the ticket after the barrier, i.e.
            # after every store of the block is in memory.  The deciding block reads the slots with
            # agent-scope atomic loads (never served from its own L2) issued after its ticket returned.
            c("TFFT_WAIT_VMEM();")
            c("__syncthreads();")
            c(f"unsigned* lastp = (unsigned*)(lds_raw + {sp.red_off_bytes});")
            c("if (tx == 0) {")
            c("    const unsigned ticket = atomicAdd(&a.ft.tickets[bx], 1u);")
            c("    lastp[0] = ticket == nparts - 1 ? 1u : 0u;")
            c("    if (ticket == nparts - 1) tfft_ps_store(&a.ft.tickets[bx], 0u);      // every part has come by: ready for the next launch (an atomic store like every other access to the word)")
            c("}")
            c("__syncthreads();")
            c("const bool last = lastp[0] != 0u;")
            c("__syncthreads();                       // the slot is reused by the reduction below")
            c("if (!last) break;")
            c("fin1 = 0; fin2 = 0; fo1 = 0; fo2 = 0;      // (the other parts' sums are read after their tickets were seen)")
            c(f"for (unsigned pp = 0; pp < nparts; ++pp) {{ const {R}* q = ps + slot0 + (unsigned long long)pp * {4 * T}ull + tx; fin1 += tfft_ps_load(q); fin2 += tfft_ps_load(q + {T}); fo1 += tfft_ps_load(q + {2 * T}); fo2 += tfft_ps_load(q + {3 * T}); }}")
        c.ind -= 1
        c("}")

    def emit_ft_decide(self, c: Code, sim: bool, shared: bool = False):
        """Block-wide reduction and the detect / locate decision
        (fft_codegen.py:432-503), then scheduling of the recompute.  Emitted inside the tile loop
        after the group's last tile (a located tile is recomputed by one more trip through the
        loop) and, `shared`, once more behind the loop for a group that several blocks walked:
        there the block first hands its sums on, only the block with the group's last ticket
        decides, and a located tile is queued for the fix-up launch.  (With the hand-off inside
        the loop the loop body needed about nine more vector registers.)"""
        sp = self.s
        R = self.R
        nw = sp.threads // WAVE
        if shared:
            c("if (a.ft.parts > 1 && it0 < it1) do {")
            c.ind += 1
            self.emit_ft_handoff(c, sim)
        elif sp.dc:
            c("if (it == it1 - 1) {")
            c.ind += 1
        else:
            c("if (it == it1 - 1 && a.ft.parts <= 1) {")
            c.ind += 1
        c(f"{R} delta, mag, delta2;")
        if sim:
            c("delta = 0; mag = 0; delta2 = 0;")
            c("for (auto& z : ts) { delta += z.fin1 + z.fo1; mag += fabs(z.fo1) + fabs(z.fin1); delta2 += z.fin2 + z.fo2; }")
            c("const unsigned tx = 0;")
        else:
            c(f"{R}* red = ({R}*)(lds_raw + {sp.red_off_bytes});")
            c(f"{R} v0 = wave_sum(fin1 + fo1), v1 = wave_sum(fabs(fo1) + fabs(fin1)), v2 = wave_sum(fin2 + fo2);")
            c("if ((tx & 63u) == 0u) { red[(tx >> 6) * 3 + 0] = v0; red[(tx >> 6) * 3 + 1] = v1; red[(tx >> 6) * 3 + 2] = v2; }")
            c("__syncthreads();")
            c("delta = 0; mag = 0; delta2 = 0;")
            c(f"for (int w = 0; w < {nw}; ++w) {{ delta += red[w * 3 + 0]; mag += red[w * 3 + 1]; delta2 += red[w * 3 + 2]; }}")
        c(f"const bool det = fabs(delta) / (({R})a.ft.err_smoothing + fabs(mag)) > ({R})a.ft.err_threshold;")
        c("int k = -1;")
        c("if (det) k = (int)round(fabs(delta2) / fabs(delta));")
        c("const bool valid = det && k >= 1 && k <= count;")
        c("const long long bad = valid ? tile0 + (long long)(k - 1) * gstride : -1;")
        c("if (tx == 0 && det) {")
        c.ind += 1
        # One atomic per detection.  Detections are counted in 64 counters on separate cache
        # lines, chosen by the block index, and each owns a 64th of the flagged list: a launch in
        # which every group flags a tile (the reference's injection cadence with small groups)
        # would otherwise queue all its blocks on one address.
        c("const unsigned sub = (unsigned)(pbx_raw & 63);")
        c("unsigned long long* sc = a.ft.counters + TFFT_FT_SUB0 + TFFT_FT_SUB_STRIDE * sub;")
        c("const unsigned long long region = (unsigned long long)(a.ft.flagged_cap >> 6);")
        if sim:
            c("const unsigned long long slot = sc[0]++;")
        else:
            c("const unsigned long long slot = atomicAdd(sc, 1ull);")
        c("if (slot < region) { long long* fl = a.ft.flagged + 2 * (sub * region + slot); fl[0] = a.ft.launch; fl[1] = bad; }")
        if sim:
            c("if (!valid) sc[1] += 1;")
        else:
            c("if (!valid) atomicAdd(sc + 1, 1ull);")
        c.ind -= 1
        c("}")
        if shared:
            # the tile was stored by another block, perhaps on another XCD: the fix-up launch recomputes it
            if sim:
                c("if (valid && a.ft.correct) a.ft.fix_list[a.ft.fix_ctl[0]++] = bad;")
            else:
                c("if (valid && a.ft.correct && tx == 0) a.ft.fix_list[atomicAdd(&a.ft.fix_ctl[0], 1u)] = bad;")
            c.ind -= 1
            c("} while (0);")
        else:
            c("if (valid && a.ft.correct) { redo_tile = bad; extra = 1; }")
            c.ind -= 1
            c("}")


FILE_HEADER = """// GENERATED by turbofft_amd/codegen/fft_codegen.py -- do not edit.
#include "../tfft_device.h"
"""


@dataclass
class FusedSpec:
    """Both launches of a two-launch plan as one kernel: a team of blocks on one XCD runs the column
    launch of a piece (a few whole transforms) into a slot that the XCD's L2 holds, meets, and runs
    the row launch out of the slot, so the intermediate of the plan never travels to memory."""
    a: KernelKey       # the column launch (kind "col")
    b: KernelKey       # the row launch with the transposed store (kind "rowT")

    def __post_init__(self):
        for k in (self.a, self.b):
            if int(k.ft) or k.pf or k.xl or k.inv or k.ck or k.wv:
                raise ValueError(f"{k}: a fused pair is made of plain forward kernels without prefetch or a register budget")
        if self.a.kind != "col" or self.b.kind != "rowT" or self.a.dtype != self.b.dtype:
            raise ValueError("a fused pair is a column launch followed by a row launch of the same type")
        self.sa = KernelSpec(self.a)
        self.sb = KernelSpec(self.b)
        self.T2, self.R = self.sa.T2, self.sa.R
        self.threads = max(self.sa.threads, self.sb.threads)
        self.lds_bytes = max(self.sa.lds_bytes, self.sb.lds_bytes)
        self.n = max(self.sa.n, self.sb.n)

    @property
    def name(self) -> str:
        t = "f32" if self.a.dtype == "float2" else "f64"
        a, b = self.a, self.b
        return (f"tfft_{t}_pair_N{a.logNi}x{b.logNi}_b{a.BS}x{b.BS}_n{a.n}x{b.n}"
                + (f"_s{int(a.split)}{int(b.split)}" if a.split or b.split else "") + (f"_t{int(a.nt)}{int(b.nt)}" if a.nt or b.nt else ""))


def emit_fused(fs: FusedSpec, sim: bool) -> str:
    c = Code()
    T2 = fs.T2
    ea = KernelEmitter(fs.sa, role="A", block_threads=fs.threads)
    eb = KernelEmitter(fs.sb, role="B", block_threads=fs.threads)
    ea.prefetched = True
    prof = bool(os.environ.get("TFFT_PAIR_PROFILE")) and not sim     # diagnostic build: time per part of a round, per block

    def tick(k: int):
        if prof:
            c(f"if (f.prof) {{ const long long now_ = (long long)wall_clock64(); pt[{k}] += now_ - pt_last; pt_last = now_; }}")
    c(f"// {fs.name}: column launch (Ni={fs.sa.Ni}, BS={fs.sa.BS}, n={fs.sa.n}, {fs.sa.threads} threads) and row launch")
    c(f"// (Ni={fs.sb.Ni}, BS={fs.sb.BS}, n={fs.sb.n}, {fs.sb.threads} threads) of a two-launch plan in one kernel, {fs.threads} threads, LDS {fs.lds_bytes} B")

    def scope(e: KernelEmitter, kargs: str, src: str, dst: Optional[str]):
        sp = e.s
        c(f"const tfft_kargs& a = {kargs};")
        c(f"const {T2}* in = {src};" + (f" {T2}* out = {dst};" if dst else ""))
        c(f"const {T2}* twhi = (const {T2}*)a.tw_hi; const {T2}* twlo = (const {T2}*)a.tw_lo; (void)twhi; (void)twlo;")
        LT = fs.R if sp.split else T2
        if sim:
            c(f"std::vector<{LT}> ldsv({sp.lds_elems}); {LT}* lds = ldsv.data(); const long long lds_limit = {sp.lds_elems}; (void)lds; (void)lds_limit;")
            c("const long long twhi_limit = limits[3], twlo_limit = limits[4]; (void)twhi_limit; (void)twlo_limit;")
            if e.role == "A":
                c("const long long in_limit = limits[0], out_limit = f.piece_elems; (void)in_limit; (void)out_limit;")
            else:
                c("const long long in_limit = f.piece_elems, out_limit = limits[1]; (void)in_limit; (void)out_limit;")
        else:
            c(f"{LT}* lds = ({LT}*)lds_raw; (void)lds;")

    def prefetch(piece: str, member: str):
        """A member's first column tile of `piece` into rn[]: issued while the member still works on the piece
        before, so that the latency of memory is spent behind that work."""
        c("{")
        c.ind += 1
        scope(ea, "a0", "in_g", None)
        c(f"const long long piece_base = ({piece}) * f.piece_elems; (void)piece_base;")
        c(f"const long long tile_n = ({piece}) * f.tiles_a + {member};")
        c(f"if ({member} < f.tiles_a && tile_n < a.ntiles) {{")
        c.ind += 1
        ea.emit_tile_decode(c, "tile_n", "_n")
        pre = Code()
        ea.map_vars(pre, 0)
        ea.emit_load(pre, "rn", "_n")
        ea.thread_block(c, sim, pre.text())
        c.ind -= 1
        c("}")
        c.ind -= 1
        c("}")

    def half(e: KernelEmitter, kargs: str, tiles: str, src: str, dst: str, member: str, before_last=None, after_first=None):
        c("{")
        c.ind += 1
        scope(e, kargs, src, dst)
        c(f"for (long long j = {member}; j < {tiles}; j += f.team) {{")
        c.ind += 1
        c(f"const long long tile = piece * {tiles} + j;")
        c("if (tile >= a.ntiles) break;")
        c(f"const bool use_rn = j == {member}; (void)use_rn;")
        e.emit_tile_body(c, sim, before_last, after_first)
        c.ind -= 1
        c("}")
        c.ind -= 1
        c("}")

    if sim:
        # one team and one slot, its members one after the other: the index algebra and the slot's bounds
        c(f'extern "C" void {fs.name}_sim(const {T2}* in_g, {T2}* out_g, const {T2}* tw, const tfft_kargs* a0p, const tfft_kargs* a1p,')
        c(f"        const tfft_fuse_args* fp, {T2}* slot, const long long* limits)")
        c("{")
        c.ind += 1
        c("const tfft_kargs a0 = *a0p, a1 = *a1p; const tfft_fuse_args f = *fp;")
        c("const long long tw_limit = limits[2]; (void)tw_limit;")
        c(f"struct TS {{ {T2} r[{fs.n}]; {T2} rn[{fs.n}]; {T2} sh[{fs.n}]; {T2} cvr[{fs.n}]; unsigned cwr[{fs.n}]; {T2} sx[{fs.n}]; {T2} sy[{fs.n}]; {fs.R} fin1, fin2, fo1, fo2; bool tbad; }};")
        c(f"std::vector<TS> ts({fs.threads}); for (auto& z : ts) z = TS();")
        c("for (long long piece = 0; piece < f.npieces; ++piece) {")
        c.ind += 1
        c("const long long piece_base = piece * f.piece_elems;")
        c("for (long long member = 0; member < f.team; ++member) {")
        c.ind += 1
        prefetch("piece", "member")
        half(ea, "a0", "f.tiles_a", "in_g", "slot", "member")
        c.ind -= 1
        c("}")
        c("for (long long member = 0; member < f.team; ++member)")
        half(eb, "a1", "f.tiles_b", "slot", "out_g", "member")
        c.ind -= 1
        c("}")
        c.ind -= 1
        c("}")
        return c.text()
    c(f'extern "C" __global__ __launch_bounds__({fs.threads})')
    c(f"void {fs.name}(const {T2}* __restrict__ in_g, {T2}* __restrict__ out_g, const {T2}* __restrict__ tw, const tfft_kargs a0, const tfft_kargs a1, const tfft_fuse_args f)")
    c("{")
    c.ind += 1
    c("extern __shared__ __align__(16) unsigned char lds_raw[];")
    c("__shared__ unsigned team_words[4];")
    c("const unsigned tx = threadIdx.x;")
    c(f"{T2} r[{fs.n}];")
    c(f"{T2} rn[{fs.sa.n}];")
    c("tfft_team tm;")
    c("if (tfft_team_join(f, tm, team_words)) {")
    c.ind += 1
    c(f"{T2}* const slot = ({T2}*)f.slots + (long long)tm.slot * f.piece_elems;")
    c("const long long member = (long long)tm.member;")
    c("long long piece = tfft_team_first(f, tm, team_words);")
    c("if (piece >= 0)")
    prefetch("piece", "member")
    if prof:
        c("long long pt[8] = {0, 0, 0, 0, 0, 0, 0, 0}; long long pt_last = (long long)wall_clock64();")
    c("for (unsigned round = 0; piece >= 0; ++round) {")
    c.ind += 1
    c("const long long piece_base = piece * f.piece_elems;")

    def slot_free():
        # the tile's last phase stores into the slot: not before every member has read what the round before left there
        tick(0)
        c("if (use_rn && round && !tfft_team_free(f, tm, round, team_words)) goto tfft_out;")
        tick(3)

    half(ea, "a0", "f.tiles_a", "in_g", "slot", "member", before_last=slot_free)
    # every member's part of the slot is in the L2 before any member reads a row of it
    c("long long next = -1;")
    tick(0)
    c("if (!tfft_team_meet(f, tm, round, team_words, next)) goto tfft_out;")
    tick(1)
    c("bool fetched = false;")

    def fetch_next():
        # behind the loads of this member's first row tile: its first column tile of the next piece
        tick(5)
        c("if (!fetched && next >= 0) {")
        c.ind += 1
        prefetch("next", "member")
        c("fetched = true;")
        c.ind -= 1
        c("}")
        tick(6)

    half(eb, "a1", "f.tiles_b", "slot", "out_g", "member", after_first=fetch_next)
    fetch_next()
    c("tfft_team_release(tm);")
    tick(2)
    if prof:
        c("pt[4] += 1;")
    c("piece = next;")
    c.ind -= 1
    c("}")
    if prof:
        c("if (f.prof && tx == 0) for (int k = 0; k < 8; ++k) f.prof[8 * (size_t)blockIdx.x + k] = (unsigned long long)pt[k];")
        c.ind -= 1
        c("}")
        c("tfft_out:")
    else:
        c.ind -= 1
        c("}")
        c("tfft_out:")
    c("tfft_team_leave(f, team_words);")
    c.ind -= 1
    c("}")
    return c.text()


def generate_fused_source(fs: FusedSpec, sim: bool) -> str:
    head = FILE_HEADER
    if sim:
        head = FILE_HEADER.replace('#include "../tfft_device.h"', '#define TFFT_SIM 1\n#include "../tfft_device.h"')
    return head + "\n" + emit_fused(fs, sim)


def generate_source(specs: Sequence[KernelSpec], sim: bool) -> str:
    out = [FILE_HEADER]
    if sim:
        out[0] = FILE_HEADER.replace('#include "../tfft_device.h"', '#define TFFT_SIM 1\n#include "../tfft_device.h"')
    for sp in specs:
        out.append(KernelEmitter(sp).emit(sim))
    return "\n".join(out)


def registry_source(specs: Sequence[KernelSpec], pairs: Sequence["FusedSpec"] = ()) -> str:
    """C table the host driver uses to find a kernel for a launch
    (the role of TurboFFT_Kernel_Entry, include/TurboFFT.h:22-25,118-526)."""
    c = Code()
    c("// GENERATED by turbofft_amd/codegen/fft_codegen.py -- do not edit.")
    c('#include <hip/hip_runtime.h>')
    c('#include "../tfft_registry.h"')
    for sp in specs:
        c(f'extern "C" __global__ void {sp.name}(const {sp.T2}*, {sp.T2}*, const {sp.T2}*, const tfft_kargs);')
    c("static const tfft_kernel_entry tfft_kernel_table_[] = {")
    kinds = {"row1": 0, "col": 1, "rowT": 2}
    for sp in specs:
        k = sp.key
        c(f'    {{"{sp.name}", (const void*){sp.name}, {0 if k.dtype == "float2" else 1}, {kinds[k.kind]}, {k.logNi}, {k.BS}, {k.n}, {int(k.ft)}, {int(k.split)}, {int(k.pf)}, {int(k.xl)}, {int(k.wv)}, {int(k.nt)}, {int(k.inv)}, {int(k.ck)}, {sp.threads}, {sp.lds_bytes}}},')
    c("};")
    c('extern "C" const tfft_kernel_entry* tfft_kernel_table(int* count) {')
    c("    *count = (int)(sizeof(tfft_kernel_table_) / sizeof(tfft_kernel_table_[0]));")
    c("    return tfft_kernel_table_;")
    c("}")
    for fs in pairs:
        c(f'extern "C" __global__ void {fs.name}(const {fs.T2}*, {fs.T2}*, const {fs.T2}*, const tfft_kargs, const tfft_kargs, const tfft_fuse_args);')
    c("static const tfft_pair_entry tfft_pair_table_[] = {")
    for fs in pairs:
        a, b = fs.a, fs.b
        c(f'    {{"{fs.name}", (const void*){fs.name}, {0 if a.dtype == "float2" else 1}, {a.logNi}, {a.BS}, {a.n}, {int(a.split)}, {int(a.nt)}, '
          f'{b.logNi}, {b.BS}, {b.n}, {int(b.split)}, {int(b.nt)}, {fs.threads}, {fs.lds_bytes}}},')
    c('    {nullptr, nullptr, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0},')
    c("};")
    c('extern "C" const tfft_pair_entry* tfft_pair_table(int* count) {')
    c("    *count = (int)(sizeof(tfft_pair_table_) / sizeof(tfft_pair_table_[0])) - 1;")
    c("    return tfft_pair_table_;")
    c("}")
    return c.text()


def pair_of_row(row: PlanRow, dtype: str) -> "FusedSpec":
    """The fused pair of a two-launch row: tile shapes and exchange forms are the row's, the column half
    keeps the load policy bit and the row half the store policy bit (the slot side of each is fixed)."""
    if row.launches != 2:
        raise ValueError(f"row {row.logN}: a fused pair needs a two-launch row")
    return FusedSpec(KernelKey(dtype, "col", row.logNi[0], row.BS[0], row.n[0], 0, int(row.split[0]) if row.split else 0, 0, 0, 0, (int(row.nt[0]) & 1) if row.nt else 0),
                     KernelKey(dtype, "rowT", row.logNi[1], row.BS[1], row.n[1], 0, int(row.split[1]) if row.split else 0, 0, 0, 0, (int(row.nt[1]) & 2) if row.nt else 0))


def collect_keys(rows: Sequence[PlanRow], dtype: str, ft_variants: Sequence[int], inverse: bool = False) -> List[KernelKey]:
    keys: List[KernelKey] = []
    seen = set()
    for row in rows:
        if row.launches == 0:
            continue
        for ft in ft_variants:
            ks = kernels_for_row(row, dtype, ft)
            if ft == 1 and any(row.ck):
                # a launch that reads the compact checksum table also needs its full-table flavour
                # (tight detection rules and the reference's own table run that one)
                ks = ks + kernels_for_row(row, dtype, ft, compact=False)
            for k in ks:
                if k not in seen:
                    seen.add(k)
                    keys.append(k)
        if inverse:
            for k in kernels_for_row(row, dtype, 0, inverse=True):
                if k not in seen:
                    seen.add(k)
                    keys.append(k)
    return keys


def main(argv=None):
    ap = argparse.ArgumentParser(description="turboFFT gfx950 kernel generator.")
    # the reference generator's flags (fft_codegen.py:709-723)
    ap.add_argument("--if_ft", type=int, default=0, help="emit the fault-tolerant variants (0/1)")
    ap.add_argument("--if_err_injection", type=int, default=0,
                    help="accepted for compatibility: injection and correction are run-time switches of the FT kernels")
    ap.add_argument("--err_smoothing", type=int, default=1000, help="default only; passed at run time")
    ap.add_argument("--err_inj", type=int, default=100, help="default only; passed at run time")
    ap.add_argument("--err_threshold", type=float, default=1e-3, help="default only; passed at run time")
    ap.add_argument("--datatype", type=str, default="double2")
    ap.add_argument("--gpu", type=str, default="gfx950")
    # this generator's own
    ap.add_argument("--param", type=str, default=None, help="plan CSV (default: param/<gpu>/param_<datatype>.csv)")
    ap.add_argument("--outdir", type=str, default=None)
    ap.add_argument("--sim", type=int, default=0, help="emit the CPU lock-step flavour")
    ap.add_argument("--list", action="store_true", help="print the kernel names and exit")
    args = ap.parse_args(argv)
    here = os.path.dirname(os.path.abspath(__file__))
    param = args.param or os.path.join(here, "..", "param", args.gpu, f"param_{args.datatype}.csv")
    rows = load_plan_csv(param)
    keys = collect_keys(rows, args.datatype, [1] if args.if_ft else [0])
    specs = [KernelSpec(k) for k in keys]
    if args.list:
        for sp in specs:
            print(sp.name, sp.threads, sp.lds_bytes, sp.passes, sp.pads)
        return 0
    outdir = args.outdir or os.path.join(here, "..", "csrc", "generated")
    os.makedirs(outdir, exist_ok=True)
    for sp in specs:
        path = os.path.join(outdir, sp.name + (".sim.cpp" if args.sim else ".hip"))
        with open(path, "w") as f:
            f.write(generate_source([sp], bool(args.sim)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
