"""CPU lock-step runs of the fused pairs (both launches of a two-launch plan in one kernel) against the
fp64 DFT: the generated text of the two halves, the slot-relative addresses and the slot's bounds."""
import os

import numpy as np
import pytest

from oracle import turbofft_oracle as O
from tests import simlib
from turbofft_amd.codegen.fft_codegen import FusedSpec, pair_of_row
from turbofft_amd.codegen.plan import KernelKey, load_plan_csv

# dtype, logN1, BS1, n1, split1, logN2, BS2, n2, split2, team, transforms per piece, transforms
PAIRS = [("float2", 7, 32, 32, 0, 9, 16, 32, 0, 8, 1, 3),        # halves of 128 and 256 threads
         ("float2", 6, 16, 8, 0, 6, 16, 8, 1, 4, 2, 5),          # ragged last piece, one split half
         ("double2", 5, 16, 4, 0, 6, 16, 16, 0, 3, 1, 2),        # a team size that does not divide the tiles
         ("double2", 7, 16, 8, 1, 8, 16, 16, 0, 8, 1, 2)]


@pytest.mark.parametrize("dtype,l1,b1,n1,s1,l2,b2,n2,s2,team,per_piece,bs", PAIRS)
def test_fused_pair_matches_the_dft(dtype, l1, b1, n1, s1, l2, b2, n2, s2, team, per_piece, bs):
    fs = FusedSpec(KernelKey(dtype, "col", l1, b1, n1, 0, s1, 0, 0, 0, 1), KernelKey(dtype, "rowT", l2, b2, n2, 0, s2, 0, 0, 0, 2))
    rng = np.random.default_rng(l1 * 100 + l2)
    x = rng.uniform(-1, 1, (bs, 1 << (l1 + l2))) + 1j * rng.uniform(-1, 1, (bs, 1 << (l1 + l2)))
    y = simlib.run_pair_sim(fs, x, bs, team, per_piece)
    assert O.rel_l2(y, O.fft_ref(x.astype(simlib.ctype_of(dtype)))) < O.tolerance(dtype, l1 + l2)


def builtin_pairs():
    here = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "turbofft_amd", "param", "gfx950")
    out = []
    for dtype in ("float2", "double2"):
        path = os.path.join(here, f"param_{dtype}_pair.csv")
        with open(path) as f:
            lines = [ln for ln in f.read().splitlines() if ln.strip() and not ln.startswith("#")]
        for row, ln in zip(load_plan_csv(path), lines):
            extra = [int(t) for t in ln.split(",")][36:39]
            out.append((dtype, row, extra))
    return out


@pytest.mark.parametrize("dtype,row,extra", builtin_pairs(), ids=[f"{d}-{r.logN}" for d, r, _ in builtin_pairs()])
def test_builtin_pair_rows(dtype, row, extra):
    # the rows the library ships: team size, transforms per piece and teams per XCD are there, every member has a tile
    # in both halves, the slots of an XCD stay within its 4 MiB of L2, and the generated text transforms right
    team, per_piece, teams = extra
    fs = pair_of_row(row, dtype)
    assert team >= 1 and per_piece >= 1 and 1 <= teams <= 64
    tiles_a = per_piece * ((1 << row.logNi[1]) // row.BS[0])
    tiles_b = per_piece * ((1 << row.logNi[0]) // row.BS[1])
    assert tiles_a >= team and tiles_b >= team
    assert teams * per_piece * (1 << row.logN) * fs.sa.esize <= 4 << 20
    assert fs.lds_bytes <= 160 * 1024 and fs.threads <= 1024
    bs = 2 * per_piece + 1
    rng = np.random.default_rng(row.logN)
    x = rng.uniform(-1, 1, (bs, 1 << row.logN)) + 1j * rng.uniform(-1, 1, (bs, 1 << row.logN))
    y = simlib.run_pair_sim(fs, x, bs, team, per_piece)
    assert O.rel_l2(y, O.fft_ref(x.astype(simlib.ctype_of(dtype)))) < O.tolerance(dtype, row.logN)
