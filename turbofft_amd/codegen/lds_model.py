"""LDS bank-conflict model used to pick the padding of every exchange.

gfx950 LDS is modelled as 32 banks of 4 bytes.  An access of `esize` bytes per
lane is served in groups of (128 / esize) lanes per cycle (16 lanes for a
64-bit access, 8 for a 128-bit one); a group costs as many cycles as the worst
bank is hit by distinct addresses.  With these numbers the model reproduces
the measured SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE ratios of the kernels
that were profiled (0.40 and 0.25 where it predicts 0.40 and 0.25, 0 where it
predicts 0); a 64-bank model predicted no conflicts for all of them.  Reads are
unit-stride across lanes by construction (the layout of an exchange follows
the thread map of the pass that reads it), so only the writes are scored.

Padding is phys(a) = a + ((a >> ps) << pl) in elements; (-1, 0) means none.
"""
from __future__ import annotations

from typing import List, Tuple

BANKS = 32
BANK_BYTES = 4


def access_cost(byte_addrs: List[int], esize: int) -> int:
    lanes_per_group = max(1, (BANKS * BANK_BYTES) // esize)
    cost = 0
    for g in range(0, len(byte_addrs), lanes_per_group):
        per_bank = {}
        for a in byte_addrs[g:g + lanes_per_group]:
            for w in range(esize // BANK_BYTES):
                b = ((a // BANK_BYTES) + w) % BANKS
                per_bank.setdefault(b, set()).add(a // BANK_BYTES + w)
        cost += max(len(v) for v in per_bank.values())
    return cost


def exchange_write_cost(spec, x: int, pad: Tuple[int, int]) -> Tuple[int, int]:
    """(cycles, ideal cycles) for wavefront 0 writing the outputs of pass x."""
    R = spec.passes[x]
    U = spec.n // R
    total = 0
    ideal = 0
    waves = [0] if spec.threads <= 64 else [0, spec.threads // 64 - 1]
    for w in waves:
        for u in range(U):
            for o in range(R):
                addrs = [spec.phys_const(spec.logical_write_addr(x, w * 64 + lane, u, o), pad) * spec.lds_esize
                         for lane in range(64)]
                total += access_cost(addrs, spec.lds_esize)
                ideal += max(1, 64 * spec.lds_esize // (BANKS * BANK_BYTES))
    return total, ideal


def exchange_read_cost(spec, x: int, pad: Tuple[int, int]) -> Tuple[int, int]:
    total = 0
    ideal = 0
    for e in range(spec.n):
        addrs = [spec.phys_const(spec.logical_read_addr(x + 1, lane, e), pad) * spec.lds_esize for lane in range(64)]
        total += access_cost(addrs, spec.lds_esize)
        ideal += max(1, 64 * spec.lds_esize // (BANKS * BANK_BYTES))
    return total, ideal


def choose_padding(spec, x: int) -> Tuple[int, int]:
    """Smallest-cost (ps, pl) for exchange x; ties go to the least extra LDS."""
    E = spec.E
    best = None
    cands = [(-1, 0)]
    for ps in range(1, max(2, E.bit_length() - 1)):
        for pl in range(0, 5):
            if (1 << pl) >= (1 << ps):
                continue
            cands.append((ps, pl))
    for pad in cands:
        w, _ = exchange_write_cost(spec, x, pad)
        r, _ = exchange_read_cost(spec, x, pad)
        extra = spec.phys_const(E - 1, pad) + 1 - E
        if extra * 8 > E:          # at most 12.5 % extra LDS
            continue
        score = (w + r, extra)
        if best is None or score < best[0]:
            best = (score, pad)
    return best[1]
