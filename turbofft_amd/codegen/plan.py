"""Plan rows and the kernels they need.

A plan CSV keeps the reference's 11-column row
`logN, launches, logN1, logN2, logN3, BS1, BS2, BS3, n1, n2, n3`
(readme.md:48-60; consumed at fft_codegen.py:745-752 and main.cu:8-9,16,22-24),
row index == logN.  Three optional trailing columns `x1, x2, x3` select, per
launch, the split exchange (re and im go through a half-size LDS buffer in two
rounds), three more `p1, p2, p3` the next-tile prefetch and three more
`c1, c2, c3` the cross-lane last pass; a row without them means all zeros.  A
21st column is the number of tiles a block of a plain (not fault-tolerant) plan
walks when the caller leaves thread_bs at 1 (0 or absent: one); columns 22-24
`w1, w2, w3` ask the compiler to fit that many wavefronts per SIMD (0: its own
choice) for the plain kernel of the launch; columns 25-27 `t1, t2, t3` mark the
launch's tile loads (1), stores (2) or both (3) as non-temporal (streamed past the
caches; tables and twiddles stay cached); columns 28-30 `g1, g2, g3` give the number of
consecutive tiles each of the 8 XCDs works on in that launch (a run-time launch parameter,
0 = 64).  Launch i transforms a digit of size 2^logNi with BSi
sub-FFTs per tile and ni elements per thread; launch 0 owns the most-strided
digit and the last launch the contiguous one.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence, Tuple


@dataclass(frozen=True)
class PlanRow:
    logN: int
    launches: int
    logNi: Tuple[int, ...]
    BS: Tuple[int, ...]
    n: Tuple[int, ...]
    split: Tuple[int, ...] = ()      # optional columns 12-14: 1 = exchange re and im separately
    pf: Tuple[int, ...] = ()         # optional columns 15-17: 1 = prefetch the next tile
    xl: Tuple[int, ...] = ()         # optional columns 18-20: 1 = last small-radix pass across lanes
    tiles: int = 0                   # optional column 21: tiles per block of the plain plan (0 = 1)
    wv: Tuple[int, ...] = ()         # optional columns 22-24: wavefronts per SIMD to compile for (0 = free)
    nt: Tuple[int, ...] = ()         # optional columns 25-27, tile access policy: +1 non-temporal tile loads, +2 non-temporal stores, +4 raised wave priority while the loads are issued
    xc: Tuple[int, ...] = ()         # optional columns 28-30: consecutive tiles per XCD (run time only; 0 = 64)
    ck: Tuple[int, ...] = ()         # optional columns 31-33: the fault-tolerant kernel of the launch reads the compact
                                     # (half-precision cotangent) form of the checksum table (fp32 only): 1 = words kept in
                                     # registers by blocks of fewer than 1024 threads, 2 = read again for every tile,
                                     # 3 = parked in LDS behind the exchange buffer (each thread its own words)
    gp: Tuple[int, ...] = ()         # optional columns 34-36 (fault-tolerant tables, run time only): tiles a block walks of a
                                     # checksum group that is shared by several blocks (0 = the library's default)

    @staticmethod
    def from_list(row: Sequence[int]) -> "PlanRow":
        row = [int(v) for v in row]
        if len(row) < 11:
            raise ValueError(f"plan row needs 11 columns, got {len(row)}: {row}")
        L = row[1]
        if not 0 <= L <= 3:
            raise ValueError(f"launches must be 0..3: {row}")
        ext = (row[11:14] + [0, 0, 0])[:3]
        ext2 = (row[14:17] + [0, 0, 0])[:3]
        ext3 = (row[17:20] + [0, 0, 0])[:3]
        p = PlanRow(row[0], L, tuple(row[2:2 + L]), tuple(row[5:5 + L]), tuple(row[8:8 + L]), tuple(ext[:L]),
                    tuple(ext2[:L]), tuple(ext3[:L]), row[20] if len(row) > 20 else 0,
                    tuple((row[21:24] + [0, 0, 0])[:L]), tuple((row[24:27] + [0, 0, 0])[:L]), tuple((row[27:30] + [0, 0, 0])[:L]),
                    tuple((row[30:33] + [0, 0, 0])[:L]), tuple((row[33:36] + [0, 0, 0])[:L]))
        if any(t not in range(8) for t in p.nt):
            raise ValueError(f"tile access policy columns must be 0..7 in row {row}")
        if L and sum(p.logNi) != p.logN:
            raise ValueError(f"logN1+logN2+logN3 != logN in row {row}")
        return p

    @property
    def N(self) -> int:
        return 1 << self.logN


@dataclass(frozen=True)
class KernelKey:
    dtype: str       # "float2" | "double2"
    kind: str        # "row1" | "col" | "rowT"
    logNi: int
    BS: int
    n: int
    ft: int          # 0 plain; 1 fused checksums, a located tile is recomputed from its input; 2 the same
                     # checksums with delayed batch correction (per-thread sums of the group's inputs and
                     # outputs, the located tile is patched with FFT(sum x) - sum y); 3 thread-level
                     # verification: every thread checks the register-level DFTs it computes in each pass
                     # against the checksum vector of their radix, no block-wide sums, a flagged tile is
                     # recomputed before it is stored
    split: int = 0   # 1: every LDS exchange moves re and im in two rounds through a half-size buffer
    pf: int = 0      # 1: the next tile is fetched into a second register set while this one is computed;
                     # k > 1: only the first k elements of a thread, from the start of the tile's last pass on
    xl: int = 0      # 1: the last pass (radix 2, 4 or 8) runs across lanes (DPP / ds_swizzle), no LDS exchange
    wv: int = 0      # > 0: compiled to fit this many wavefronts per SIMD (register budget 512 / wv)
    nt: int = 0      # bit 0: tile loads are non-temporal, bit 1: tile stores are, bit 2: raised wave priority while the tile loads are issued (plain kernels)
    inv: int = 0     # 1: the flavour an inverse plan uses in this position -- re and im exchanged as
                     # they are loaded (row1, col as first launch) and/or before they are stored
                     # (row1, rowT): inverse = swap . forward . swap
    ck: int = 0      # > 0: fault-tolerant fp32 kernel that reads the compact checksum table (one half-precision
                     # cotangent per element, two per 32-bit word); 1: the words stay in registers for the tiles
                     # of a block where the block has fewer than 1024 threads, 2: they are read again for every tile,
                     # 3: every thread parks its words in LDS when the block starts and reads them back per tile

    @property
    def name(self) -> str:
        t = "f32" if self.dtype == "float2" else "f64"
        return (f"tfft_{t}_{self.kind}_N{self.logNi}_b{self.BS}_n{self.n}" + ("_s" if self.split else "") + ("_p" if self.pf == 1 else (f"_p{self.pf}" if self.pf else "")) + ("_x" if self.xl else "")
                + (f"_w{self.wv}" if self.wv else "") + (f"_t{self.nt}" if self.nt else "") + ("_i" if self.inv else "") + ({0: "", 1: "_h", 2: "_h2", 3: "_h3"}[int(self.ck)]) + ({0: "", 1: "_ft", 2: "_fd", 3: "_tt"}[int(self.ft)]))


def load_plan_csv(path: str) -> List[PlanRow]:
    rows = []
    with open(path) as f:
        for line in f:
            line = line.strip()
            if not line or line.startswith("#"):
                continue
            rows.append(PlanRow.from_list([int(t) for t in line.split(",")[:36] if t.strip()]))
    return rows


def launch_kinds(launches: int) -> List[str]:
    return {1: ["row1"], 2: ["col", "rowT"], 3: ["col", "col", "rowT"]}[launches]


def kernels_for_row(row: PlanRow, dtype: str, ft: int, inverse: bool = False, compact: bool = True) -> List[KernelKey]:
    """Kernels of the row's launches; with `inverse` the first and the last launch use their
    component-swapping flavour (plain plans only), launches in between are the forward ones.
    `compact`: honour the row's compact-checksum-table columns (recompute-correcting fp32
    fault-tolerant kernels only); False gives the full-table flavour of the same launches."""
    if inverse and ft:
        raise ValueError("inverse plans have no fault-tolerant flavour")
    last = row.launches - 1
    return [KernelKey(dtype, kind, row.logNi[i], row.BS[i], row.n[i], int(ft), int(row.split[i]) if row.split else 0,
                      # (partial prefetch, pf > 1, exists for the plain forward kernel only)
                      ((int(row.pf[i]) if (int(row.pf[i]) <= 1 or not (ft or (inverse and i in (0, last)))) else 0) if row.pf else 0) if int(ft) != 3 else 0,
                      # fault-tolerant plans keep the LDS path: the checksum model fixes which
                      # outputs a thread owns
                      (int(row.xl[i]) if row.xl else 0) if not ft else 0,
                      # the register budget hint was tuned on the plain kernel only (fault-tolerant
                      # kernels keep their table in registers and spill under any tighter budget)
                      # (the compact-table flavour is the exception: its budget is tuned with it)
                      # (thread-level verification runs the plain rows without their hint: timed with budgets of 2, 3 and
                      # none for every size, none was the best or within a point of it at all but two)
                      (int(row.wv[i]) if row.wv else 0) if (not ft or (compact and int(ft) == 1 and row.ck and int(row.ck[i]))) else 0,
                      # the priority bit was timed on the plain kernel only
                      (int(row.nt[i]) & (3 if ft else 7)) if row.nt else 0,
                      1 if inverse and i in (0, last) else 0,
                      int(row.ck[i]) if (compact and int(ft) == 1 and row.ck and int(row.ck[i])) else 0)
            for i, kind in enumerate(launch_kinds(row.launches))]


def radix_passes(Ni: int, n: int) -> List[int]:
    """Pass radices inside a block: n, n, ..., leftover (leftover last), the
    same split the reference uses (fft_codegen.py:36-43, 127-138)."""
    if n > Ni:
        raise ValueError(f"n={n} exceeds the sub-FFT length {Ni}")
    out = []
    m = Ni
    while m > 1:
        r = n if m >= n else m
        out.append(r)
        m //= r
    return out
