"""GPU fault-tolerance parity: counters, located tiles and corrected output of
the FT kernels against the oracle's model of the reference checksum scheme
(same thresholds, same group formula, same injection cadence)."""
import numpy as np
import pytest

import turbofft_amd
from oracle import turbofft_oracle as O

pytestmark = pytest.mark.gpu


def _torch():
    import torch
    assert torch.cuda.is_available()
    return torch


def cdtype(dt):
    return np.complex64 if dt == "float2" else np.complex128


def make(bs, N, dt, seed=0):
    rng = np.random.default_rng(seed)
    return (rng.uniform(-1, 1, (bs, N)) + 1j * rng.uniform(-1, 1, (bs, N))).astype(cdtype(dt))


def run(plan, x):
    torch = _torch()
    print(f"[ft case] logN={plan.logN} dt={plan.datatype} bs={x.shape[0]} launches={plan.launches} Ni={plan.logNi} "
          f"BS={plan.BS} n={plan.n} tbs={plan.thread_bs}", flush=True)
    plan.reset_ft_counters()
    y = plan.fft(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    return y.cpu().numpy(), plan.ft_counters()


CASES = [("float2", 10, 64), ("double2", 10, 16), ("float2", 13, 32), ("double2", 15, 8), ("float2", 16, 4),
         ("float2", 21, 1), ("double2", 20, 2)]


@pytest.mark.parametrize("dt,logN,bs", CASES)
@pytest.mark.parametrize("tbs", [1, 4])
def test_clean_ft_run(dt, logN, bs, tbs):
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=tbs)
    x = make(bs, 1 << logN, dt, logN)
    y, c = run(plan, x)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    assert c["checked"] == sum(plan.grid(i, bs) for i in range(plan.launches))
    assert c["detected"] == 0 and c["corrected"] == 0 and c["flagged"] == []


@pytest.mark.parametrize("dt,logN,bs", CASES)
@pytest.mark.parametrize("tbs", [2, 8])
def test_reference_cadence_matches_oracle_model(dt, logN, bs, tbs):
    # if_err=1: every block of the last launch injects into element 0 of the tile
    # cnt == block % thread_bs + 1, detects, locates and recomputes it.  The expected
    # decisions come from the oracle's model of the reference scheme; the magnitude is
    # 100 (the reference default) for the 1024-point plans; for the larger ones the model
    # says the relative rule |delta|/(1000+|mag|) > 1e-3 does not fire at 100 on U[-1,1)
    # data (see the next test), so they inject an error sized from the data's checksum magnitude.
    plan = turbofft_amd.TurboFFT(logN, dt, if_err=1, thread_bs=tbs)
    gaps = [7, 5, 3][:plan.launches]
    for i, g in enumerate(gaps):
        plan.set_tb_gap(i, g)
    x = make(bs, 1 << logN, dt, logN + 1)
    row = O.PlanRow.from_list(plan.plan_row())
    if logN <= 10:
        mag = 100.0
    else:
        # the rule is relative to the checksum magnitude of the data, which grows with the
        # tile and with every launch: size the error 30x above the rule's floor for this data
        clean, _ = O.ft_plan_model(x, row, dt, tbs, gaps, None)
        mag = float(np.ceil(30e-3 * (1000.0 + max(d.mag for d in clean[-1])) / 0.366))
    plan.set_injection(1, mag=mag)
    y, c = run(plan, x)
    geoms = O.launch_geometry(row, bs)
    last = geoms[-1]
    groups = O.tile_groups(last.ntiles, tbs, gaps[plan.launches - 1])
    injs = O.reference_injections(groups, tbs, mag)
    dec, _ = O.ft_plan_model(x, row, dt, tbs, gaps, injs)
    # keep away from the decision boundary: reduction order differs between GPU and model
    for dl in dec:
        for d in dl:
            ratio = abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3
            assert ratio < 0.67 or ratio > 1.5, "test case sits on the detection threshold"
    model = sorted((li, d.tile) for li, dl in enumerate(dec) for d in dl if d.detected)
    assert model == sorted((plan.launches - 1, i.tile) for i in injs)      # every injection is caught
    assert sorted(c["flagged"]) == model
    assert c["detected"] == len(injs) == c["corrected"] and c["uncorrectable"] == 0
    # corrected result is bit-identical to a run without injection
    plan.set_injection(0)
    y0, c0 = run(plan, x)
    assert c0["detected"] == 0
    assert np.array_equal(y, y0)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)


@pytest.mark.parametrize("dt,logN,bs", [("float2", 10, 64), ("double2", 10, 16), ("float2", 13, 32), ("double2", 13, 8)])
def test_reference_checksum_table_clean_run(dt, logN, bs):
    # the table the reference's kernels actually read (abft.h:21-61: angles rounded to float
    # before the division): decisions on clean data must equal the oracle model fed the same
    # table.  At 8192 points that table is off by up to 3e-3 rad; the model says whether the
    # residual this leaves on clean data stays below the rule, the GPU has to agree.
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=4)
    plan.set_checksum_mode("reference")
    plan.set_tb_gap(0, 5)
    x = make(bs, 1 << logN, dt, 40 + logN)
    y, c = run(plan, x)
    row = O.PlanRow.from_list(plan.plan_row())
    dec, _ = O.ft_plan_model(x, row, dt, 4, [5], None, table_mode="reference")
    exact, _ = O.ft_plan_model(x, row, dt, 4, [5], None, table_mode="exact")
    worst = max(abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3 for d in dec[0])
    worst_exact = max(abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3 for d in exact[0])
    print(f"clean-data ratio to the threshold: reference table {worst:.3e}, exact table {worst_exact:.3e}", flush=True)
    assert all(r < 0.67 or r > 1.5 for r in (abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3 for d in dec[0]))
    model = sorted((0, d.tile) for d in dec[0] if d.detected)
    assert sorted(c["flagged"]) == model and c["detected"] == len(model)
    assert c["checked"] == plan.grid(0, bs)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)       # a false alarm only recomputes
    plan.close()


@pytest.mark.parametrize("dt,bs", [("float2", 64), ("double2", 16)])
@pytest.mark.parametrize("tbs", [2, 4])
def test_reference_checksum_table_reference_cadence(dt, bs, tbs):
    # if_err=1 at 2^10 with the reference's own table: every block injects 100 into element 0
    # of one of its tiles, detects, locates and recomputes it; decisions against the model run
    # with table_mode="reference"
    logN = 10
    plan = turbofft_amd.TurboFFT(logN, dt, if_err=1, thread_bs=tbs)
    plan.set_checksum_mode("reference")
    plan.set_tb_gap(0, 7)
    x = make(bs, 1 << logN, dt, 77)
    y, c = run(plan, x)
    row = O.PlanRow.from_list(plan.plan_row())
    groups = O.tile_groups(O.launch_geometry(row, bs)[0].ntiles, tbs, 7)
    injs = O.reference_injections(groups, tbs, 100.0)
    dec, _ = O.ft_plan_model(x, row, dt, tbs, [7], injs, table_mode="reference")
    for d in dec[0]:
        ratio = abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3
        assert ratio < 0.67 or ratio > 1.5, "test case sits on the detection threshold"
    model = sorted((0, d.tile) for d in dec[0] if d.detected)
    assert model == sorted((0, i.tile) for i in injs)
    assert sorted(c["flagged"]) == model and c["detected"] == len(injs) == c["corrected"]
    plan.set_injection(0)
    y0, c0 = run(plan, x)
    assert c0["detected"] == 0 and np.array_equal(y, y0)
    # back to the exact table: same decisions on this case, same corrected output
    plan.set_checksum_mode("exact")
    plan.set_injection(1, mag=100.0)
    y1, c1 = run(plan, x)
    assert sorted(c1["flagged"]) == model and np.array_equal(y1, y0)
    plan.close()


@pytest.mark.parametrize("dt,logN,bs", CASES)
@pytest.mark.parametrize("tbs", [2, 8])
def test_delayed_batch_correction_matches_oracle_model(dt, logN, bs, tbs):
    # correct=2: the located tile is patched with FFT(sum x) - sum y of its group instead of
    # being recomputed from its input (fft_codegen.py:355-357,421-423 live sums, :401-404,
    # 427-429 and test.ipynb cell 0 for the patch).  Same detections as the recompute flavour;
    # the patched result meets the accuracy bar (to rounding, not bit for bit) and every
    # patched tile agrees with the oracle's delayed_batch_correction of the same group.
    plan = turbofft_amd.TurboFFT(logN, dt, if_err=1, thread_bs=tbs)
    plan.set_ft_params(1000.0, 1e-3, correct=2)
    gaps = [7, 5, 3][:plan.launches]
    for i, g in enumerate(gaps):
        plan.set_tb_gap(i, g)
    x = make(bs, 1 << logN, dt, logN + 1)
    row = O.PlanRow.from_list(plan.plan_row())
    if logN <= 10:
        mag = 100.0
    else:
        clean, _ = O.ft_plan_model(x, row, dt, tbs, gaps, None)
        mag = float(np.ceil(30e-3 * (1000.0 + max(d.mag for d in clean[-1])) / 0.366))
    plan.set_injection(1, mag=mag)
    y, c = run(plan, x)
    geoms = O.launch_geometry(row, bs)
    last = geoms[-1]
    groups = O.tile_groups(last.ntiles, tbs, gaps[plan.launches - 1])
    injs = O.reference_injections(groups, tbs, mag)
    dec, _ = O.ft_plan_model(x, row, dt, tbs, gaps, injs)
    for dl in dec:
        for d in dl:
            ratio = abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3
            assert ratio < 0.67 or ratio > 1.5, "test case sits on the detection threshold"
    model = sorted((li, d.tile) for li, dl in enumerate(dec) for d in dl if d.detected)
    assert model == sorted((plan.launches - 1, i.tile) for i in injs)
    assert sorted(c["flagged"]) == model
    assert c["detected"] == len(injs) == c["corrected"] and c["uncorrectable"] == 0
    ref = O.fft_ref(x)
    assert O.rel_l2(y, ref) <= O.tolerance(dt, logN)
    worst = max(O.rel_l2(y[b], ref[b]) for b in range(bs))
    assert worst <= O.tolerance(dt, logN) * 2
    # the patch against the oracle's, tile by tile, for the single-launch plans (the tiles of a
    # last launch are rows of the previous launch's output, compared through the bar above)
    if plan.launches == 1:
        BS, n = plan.BS[0], plan.n[0]
        xt = last.gather(x)
        yt = O.fft_ref(xt).astype(cdtype(dt))
        got = last.gather(y)
        for inj in injs[:16]:
            g = next(gr for gr in groups if inj.tile in gr)
            yg = yt[g].copy()
            yg[g.index(inj.tile), inj.s, :] += inj.mag
            want = O.delayed_batch_correction(xt[g], yg, g.index(inj.tile), n, dt)
            assert O.rel_l2(got[inj.tile], want) <= O.tolerance(dt, logN)
    # without injection the flavour is transparent
    plan.set_injection(0)
    y0, c0 = run(plan, x)
    assert c0["detected"] == 0 and O.rel_l2(y0, ref) <= O.tolerance(dt, logN)
    plan.close()


@pytest.mark.parametrize("dt,logN,bs", [("float2", 10, 64), ("double2", 10, 16), ("float2", 8, 512), ("double2", 16, 4), ("float2", 21, 1)])
def test_delayed_correction_of_single_tile_groups_is_bit_identical(dt, logN, bs):
    # thread_bs = 1 with the reference cadence: every tile of the last launch carries an error.
    # The delayed flavour holds a one-tile group in registers until it is checked and transforms
    # the saved input again when it is flagged: every tile is flagged and corrected, nothing is
    # read twice, and the result equals the undisturbed run bit for bit.
    plan = turbofft_amd.TurboFFT(logN, dt, if_err=1, thread_bs=1)
    plan.set_ft_params(1000.0 if logN <= 10 else 0.0, 1e-3 if logN <= 10 else (1e-4 if dt == "float2" else 1e-9), correct=2)
    plan.set_injection(1, mag=100.0 if logN <= 10 else 1e4)
    x = make(bs, 1 << logN, dt, logN + 3)
    y, c = run(plan, x)
    last = plan.launches - 1
    ntiles = plan.grid(last, bs)
    assert c["detected"] == ntiles == c["corrected"] and c["uncorrectable"] == 0
    if ntiles <= 4096:
        assert sorted(c["flagged"]) == [(last, t) for t in range(ntiles)] and not c["flagged_truncated"]
    else:
        assert c["flagged_truncated"] and len(c["flagged"]) == 4096
    plan.set_injection(0)
    y0, c0 = run(plan, x)
    assert c0["detected"] == 0 and np.array_equal(y, y0)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    plan.close()


def test_delayed_batch_correction_host_chosen_tiles_and_earlier_launch():
    plan = turbofft_amd.TurboFFT(15, "double2", if_ft=1, thread_bs=2)
    plan.set_ft_params(1000.0, 1e-3, correct=2)
    plan.set_injection(2, launch=0, every=1 << 30, tile_phase=9, s=3, m=1, mag=1000.0)
    x = make(4, 1 << 15, "double2", 5)
    y, c = run(plan, x)
    assert c["flagged"] == [(0, 9)] and c["corrected"] == 1
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance("double2", 15)
    plan.close()
    # ragged single-launch batch: the last tile holds fewer transforms than BS
    plan = turbofft_amd.TurboFFT(7, "float2", if_ft=1, thread_bs=3)
    plan.set_ft_params(1000.0, 1e-3, correct=2)
    bs = plan.BS[0] * 10 + 3
    plan.set_injection(2, every=1 << 30, tile_phase=10, s=1, m=0, mag=1000.0)
    x = make(bs, 128, "float2", 6)
    y, c = run(plan, x)
    assert c["flagged"] == [(0, 10)] and c["corrected"] == 1
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance("float2", 7)
    plan.close()


COMPACT = [("float2", 7, 4096), ("float2", 9, 1024), ("float2", 13, 64), ("float2", 14, 32), ("float2", 15, 16), ("float2", 16, 8), ("float2", 17, 4), ("float2", 18, 2), ("float2", 19, 2), ("float2", 20, 2), ("float2", 22, 1), ("float2", 23, 1), ("double2", 7, 4096), ("double2", 15, 16), ("double2", 20, 2), ("double2", 23, 1)]


@pytest.mark.parametrize("dt,logN,bs", COMPACT)
def test_compact_checksum_table_rows(dt, logN, bs):
    # rows of the fault-tolerant table that read the compact (reduced-precision cotangent) form of
    # the checksum vector: clean data raises nothing, an error sized above the rule is caught,
    # located and recomputed bit-identically, decisions equal the oracle model fed the compact
    # vector, and a rule too tight for the table's precision (or the reference's own table)
    # runs the full-table flavour of the same launches
    tbs = 4
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=tbs)
    names = plan.kernel_names()
    assert any(n.endswith(("_h_ft", "_h2_ft", "_h3_ft")) for n in names), names
    gaps = [7, 5, 3][:plan.launches]
    for i, g in enumerate(gaps):
        plan.set_tb_gap(i, g)
    x = make(bs, 1 << logN, dt, logN + 11)
    y, c = run(plan, x)
    assert c["detected"] == 0 and O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    row = O.PlanRow.from_list(plan.plan_row())
    last = plan.launches - 1
    compact_last = "_h" in names[last]
    clean, _ = O.ft_plan_model(x, row, dt, tbs, gaps, None, table_mode="compact" if compact_last else "exact")
    assert max(abs(d.delta) / (1000.0 + abs(d.mag)) for d in clean[last]) < (3e-4 if dt == "float2" else 1e-6)
    sized = float(np.ceil(30e-3 * (1000.0 + max(d.mag for d in clean[last])) / 0.366))
    plan.set_ft_params(1000.0, 1e-3, correct=True)
    groups = O.tile_groups(O.launch_geometry(row, bs)[last].ntiles, tbs, gaps[last])
    # an error sized from the data; where the rule saturates next to its threshold for this tile
    # shape (long sub-FFTs: the ratio tends to a constant as the error grows), a smaller one that
    # the model leaves clearly undetected -- the GPU has to agree either way
    # The compact table is a design of this build; the reference multiplies by the complex c_N
    # (fft_codegen.py:354-367).  The decisions of a compact-table kernel must therefore equal what
    # the rule gives with the exact vector and with the table the reference's kernels read (abft.h:
    # 21-61, built by the reference for sub-FFTs of up to 8192 points, main.cu:85-93) on the same
    # case: the three models are run side by side and their flagged lists have to be the same.
    modes = ["compact" if compact_last else "exact", "exact"]
    if max(plan.logNi) <= 13:
        modes.append("reference")
    for mag in (sized, sized * 64, sized / 256):
        injs = O.reference_injections(groups, tbs, mag)
        decs = {m: O.ft_plan_model(x, row, dt, tbs, gaps, injs, table_mode=m)[0] for m in modes}
        dec = decs[modes[0]]
        if all(r < 0.67 or r > 1.5 for dm in decs.values() for r in (abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3 for d in dm[last])):
            break
    else:
        pytest.fail("no error size keeps this case away from the detection threshold under all three tables")
    flagged = {m: sorted((li, d.tile) for li, dl in enumerate(dm) for d in dl if d.detected) for m, dm in decs.items()}
    print(f"flagged per table: { {m: len(v) for m, v in flagged.items()} }", flush=True)
    assert all(v == flagged[modes[0]] for v in flagged.values()), flagged
    plan.set_injection(1, mag=mag)
    y1, c1 = run(plan, x)
    model = sorted((last, d.tile) for d in dec[last] if d.detected)
    # (for sub-FFTs of 2048 points and more the rule saturates below its threshold for
    # single-element errors of any size: the model says whether this tile is in that regime)
    print(f"compact rows: {len(model)} of {len(injs)} injections above the rule in the model", flush=True)
    assert sorted(c1["flagged"]) == model and c1["corrected"] == len(model)
    if len(model) == len(injs):
        assert np.array_equal(y1, y)
    # a tight rule, and the reference's own table, switch to the full-table kernels
    plan.set_injection(0)
    plan.set_ft_params(0.0, 1e-4 if dt == "float2" else 1e-9, correct=True)
    tight = plan.kernel_names()
    assert not any(n.endswith(("_h_ft", "_h2_ft", "_h3_ft")) for n in tight), tight
    y2, c2 = run(plan, x)
    assert c2["detected"] == 0 and np.array_equal(y2, y)
    plan.set_ft_params(1000.0, 1e-3, correct=True)
    assert plan.kernel_names() == names
    plan.set_checksum_mode("reference")
    assert not any("_h" in n for n in plan.kernel_names())
    plan.close()


def test_reference_default_magnitude_is_below_the_rule_at_8192_points():
    # the model of the reference rule predicts NO detection for err_inj=100 on a
    # U[-1,1) fp32 8192-point tile (|delta| = 36.6, mag ~ 1.5e5): the GPU must agree
    plan = turbofft_amd.TurboFFT(13, "float2", if_err=1, thread_bs=2)
    plan.set_tb_gap(0, 7)
    x = make(32, 1 << 13, "float2", 14)
    y, c = run(plan, x)
    row = O.PlanRow.from_list(plan.plan_row())
    groups = O.tile_groups(32, 2, 7)
    injs = O.reference_injections(groups, 2, 100.0)
    dec, _ = O.ft_plan_model(x, row, "float2", 2, [7], injs)
    assert not any(d.detected for d in dec[0])
    assert c["detected"] == 0 and c["checked"] == len(groups)
    err = np.abs(y - O.fft_ref(x))
    for inj in injs:                      # the undetected error is still in the output
        assert np.allclose(err[inj.tile], 100.0, rtol=1e-3)


def test_detect_only_leaves_error_in_place():
    plan = turbofft_amd.TurboFFT(10, "double2", if_ft=1, thread_bs=4)
    plan.set_ft_params(1000.0, 1e-3, correct=False)
    plan.set_injection(2, every=1 << 30, tile_phase=5, s=0, m=0, mag=100.0)
    x = make(32, 1024, "double2", 3)
    y, c = run(plan, x)
    assert c["detected"] == 1 and c["corrected"] == 0 and c["flagged"] == [(0, 5)]
    err = np.abs(y - O.fft_ref(x))
    hit = 5 * plan.BS[0]                      # sub-FFT 0 of tile 5 (a tile holds BS transforms)
    assert np.allclose(err[hit], 100.0, rtol=1e-9) and np.delete(err, hit, axis=0).max() < 1e-9


def test_threshold_rule():
    # |delta| / (err_smoothing + |mag|) > err_threshold with delta = -mag_inj (Ni = 1 mod 3)
    x = make(16, 1024, "double2", 4)
    for mag, expect in ((0.5, 0), (100.0, 1)):      # data checksum magnitude ~1e4: floor ~11
        plan = turbofft_amd.TurboFFT(10, "double2", if_ft=1, thread_bs=1)
        plan.set_injection(2, every=1 << 30, tile_phase=3, mag=mag)
        _, c = run(plan, x)
        assert c["detected"] == expect
    plan = turbofft_amd.TurboFFT(10, "double2", if_ft=1, thread_bs=1)
    plan.set_ft_params(0.0, 1e-6, correct=True)          # tight rule catches the small error too
    plan.set_injection(2, every=1 << 30, tile_phase=3, mag=0.5)
    y, c = run(plan, x)
    assert c["detected"] == 1 and c["corrected"] == 1
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance("double2", 10)


def test_injection_in_an_earlier_launch_is_caught_there():
    plan = turbofft_amd.TurboFFT(15, "double2", if_ft=1, thread_bs=2)
    plan.set_ft_params(1000.0, 1e-3, correct=True)
    plan.set_injection(2, launch=0, every=1 << 30, tile_phase=9, s=3, m=1, mag=1000.0)
    x = make(4, 1 << 15, "double2", 5)
    y, c = run(plan, x)
    assert c["flagged"] == [(0, 9)] and c["corrected"] == 1
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance("double2", 15)


def _model_groups_last_launch(xsel, row, dt, groups, tiles_per_transform, injs, tbs):
    """Oracle decisions for selected tile groups of the last launch.  xsel maps a batch
    index to that transform's input; only the transforms the groups touch are needed."""
    cache = {}
    geom1 = O.launch_geometry(row, 1)[-1]
    xin, yout, remap = [], [], {}
    for g in groups:
        for t in g:
            b, lt = divmod(t, tiles_per_transform)
            if b not in cache:
                _, stages = O.plan_fft(xsel[b][None, :], row, dt, return_stages=True)
                cache[b] = (geom1.gather(stages[-1][0]), geom1.gather(stages[-1][1]))
            remap[t] = len(xin)
            xin.append(cache[b][0][lt])
            yout.append(cache[b][1][lt].copy())
    for inj in injs:
        if inj.tile in remap:
            k = np.arange(geom1.Ni)
            yout[remap[inj.tile]][inj.s] += inj.mag * np.exp(-2j * np.pi * ((inj.m * k) % geom1.Ni) / geom1.Ni)
    lg = [[remap[t] for t in g] for g in groups]
    dec = O.ft_launch_model(np.stack(xin), np.stack(yout), geom1.n, lg, dt,
                            O.dft_checksum_vector(geom1.Ni, dt))
    return dec


def test_config5_fp64_2p20_batch256():
    # benchmark configuration 5: fp64, N=2^20, batch 256, threshold 1e-3, err_smoothing 1000, one
    # error in 1 of every 1000 tile groups of the last launch.  Run (i) with the stated
    # magnitude 100 and (ii) with an error sized above the rule's floor for this data;
    # the decisions of every group that holds an injected tile must equal the oracle model's.
    torch = _torch()
    logN, bs, tbs = 20, 256, 8
    N = 1 << logN
    plan = turbofft_amd.TurboFFT(logN, "double2", if_ft=1, thread_bs=tbs)
    row = O.PlanRow.from_list(plan.plan_row())
    plan.set_ft_params(1000.0, 1e-3, correct=True)
    last = plan.launches - 1
    gap = 64
    plan.set_tb_gap(last, gap)
    tile_elems = (1 << plan.logNi[last]) * plan.BS[last]
    ntiles = N * bs // tile_elems
    tpt = N // tile_elems
    every = 1000 * tbs
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.view_as_complex(torch.rand((bs, N, 2), generator=g, device="cuda", dtype=torch.float64) * 2 - 1)
    groups_all = O.tile_groups(ntiles, tbs, gap)
    inj_tiles = list(range(123, ntiles, every))
    hit_groups = [gr for gr in groups_all if any(t in gr for t in inj_tiles)]
    need = sorted({t // tpt for gr in hit_groups for t in gr})
    xsel = {b: x[b].cpu().numpy() for b in need}
    ref_idx = need[:3]
    # An error e on input element m moves delta by e * (re c[m] + im c[m]) but also every output
    # of the sub-FFT by |e|, i.e. mag by about |e| * Ni / sqrt(n): for long sub-FFTs the ratio
    # saturates below the threshold and the reference rule cannot fire at any magnitude.  The
    # model says which regime this plan's last launch is in; the GPU must agree either way.
    huge = [O.Injection(t, 1, 5, 1e15) for t in inj_tiles]
    detectable = all(d.detected for d in _model_groups_last_launch(xsel, row, "double2", hit_groups, tpt, huge, tbs))
    print("config5 plan", plan.logNi, plan.BS, plan.n, "single-element errors detectable in the last launch:", detectable, flush=True)
    for mag in (100.0, None):
        if mag is None:
            clean = _model_groups_last_launch(xsel, row, "double2", hit_groups, tpt, [], tbs)
            cm = O.dft_checksum_vector(1 << plan.logNi[last], "double2")[5]
            weight = abs(cm.real + cm.imag)
            assert weight > 1e-6
            mag = float(np.ceil(30e-3 * (1000.0 + max(d.mag for d in clean)) / min(weight, 1.0)))
        injs = [O.Injection(t, 1, 5, mag) for t in inj_tiles]
        dec = _model_groups_last_launch(xsel, row, "double2", hit_groups, tpt, injs, tbs)
        for d in dec:
            ratio = abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3
            assert ratio < 0.67 or ratio > 1.5, "test case sits on the detection threshold"
        plan.set_injection(2, every=every, tile_phase=123, s=1, m=5, mag=mag)
        plan.reset_ft_counters()
        y = plan.fft(x)
        torch.cuda.synchronize()
        c = plan.ft_counters()
        model = []
        for d, gr in zip(dec, hit_groups):
            if d.detected:
                model.append((last, gr[d.k - 1] if 1 <= d.k <= len(gr) else -1))
        print("config5 mag", mag, {k: v for k, v in c.items() if k != "flagged"}, "model detections", len(model), flush=True)
        assert c["checked"] == sum(plan.grid(i, bs) for i in range(plan.launches))
        assert sorted(c["flagged"]) == sorted(model)
        assert c["detected"] == len(model) == c["corrected"] and c["uncorrectable"] == 0
        if len(model) == len(inj_tiles):         # everything corrected: transforms must be clean
            for b in ref_idx:
                assert O.rel_l2(y[b].cpu().numpy(), O.fft_ref(xsel[b])) <= O.tolerance("double2", logN)
    # the sized error is caught in every group, unless the rule cannot see it at all
    assert len(model) == (len(inj_tiles) if detectable else 0)


def test_injection_element_is_validated():
    plan = turbofft_amd.TurboFFT(10, "double2", if_ft=1)
    lim = (1 << plan.logNi[-1]) // plan.n[-1]            # the injected element is one of the first Ni/n
    plan.set_injection(2, every=1 << 30, tile_phase=0, s=0, m=lim - 1)
    with pytest.raises(turbofft_amd.TurboFFTError):
        plan.set_injection(2, every=1 << 30, tile_phase=0, s=0, m=lim)
    with pytest.raises(turbofft_amd.TurboFFTError):
        plan.set_injection(2, every=1 << 30, tile_phase=0, s=plan.BS[-1], m=0)


def test_seeded_random_injections_match_the_model():
    """Sixty seeded draws of (type, size, batch, group size, interleave, launch, element,
    magnitude, cadence, correction on/off) with at most one error per checksum group: the
    flagged (launch, tile) list and the counters equal the oracle model's decisions.  Draws
    whose ratio sits within a factor 1.5 of the threshold are redrawn (reduction order
    differs between the GPU and the model)."""
    torch = _torch()
    rng = np.random.default_rng(31)
    done = 0
    while done < 60:
        dt = ["float2", "double2"][int(rng.integers(2))]
        logN = int(rng.integers(4, 17))
        tbs = int(rng.choice([1, 2, 3, 4, 8]))
        plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=tbs)
        row = O.PlanRow.from_list(plan.plan_row())
        L = plan.launches
        li = int(rng.integers(L))
        bs = int(rng.integers(1, 7)) * plan.BS[0] * tbs if L == 1 else int(rng.integers(1, 1 + max(1, (1 << 20) >> logN)))
        gaps = [int(rng.integers(1, 9)) for _ in range(L)]
        for i, g in enumerate(gaps):
            plan.set_tb_gap(i, g)
        x = make(bs, 1 << logN, dt, 500 + done)
        ntiles = O.launch_geometry(row, bs)[li].ntiles
        every = (tbs - 1) * gaps[li] + 1 + int(rng.integers(0, 5))         # at most one error per group
        phase = int(rng.integers(every))
        s = int(rng.integers(plan.BS[li]))
        m = int(rng.integers((1 << plan.logNi[li]) // plan.n[li]))
        mag = float(10 ** rng.uniform(0, 5))
        correct = bool(rng.integers(2))
        injs = [O.Injection(t, s, m, mag) for t in range(phase, ntiles, every)]
        dec, _ = O.ft_plan_model(x, row, dt, tbs, gaps, injs, inj_launch=li)
        if any(0.67 <= abs(d.delta) / (1000.0 + abs(d.mag)) / 1e-3 <= 1.5 for dl in dec for d in dl):
            plan.close()
            continue
        plan.set_ft_params(1000.0, 1e-3, correct=correct)
        plan.set_injection(2, launch=li, every=every, tile_phase=phase, s=s, m=m, mag=mag)
        print(f"[random injection {done}] launch={li} every={every} phase={phase} s={s} m={m} mag={mag:.1f} correct={correct} gaps={gaps}", flush=True)
        y, c = run(plan, x)
        model = sorted((l, d.tile) for l, dl in enumerate(dec) for d in dl if d.detected)
        assert sorted(c["flagged"]) == model
        assert c["detected"] == len(model) and c["uncorrectable"] == 0
        assert c["corrected"] == (len(model) if correct else 0)
        assert c["checked"] == sum(plan.grid(i, bs) for i in range(L))
        if correct and len(model) == len(injs):          # every error caught and recomputed
            assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
        plan.close()
        done += 1


@pytest.mark.parametrize("dt,logN,bs", [("float2", 10, 64), ("double2", 13, 8), ("float2", 16, 4), ("double2", 7, 300),
                                        ("float2", 1, 5)])
def test_offline_checksum_passes(dt, logN, bs):
    # the baseline of cufft_ft.h:19-95 (separate checksum passes around the transform): both passes
    # against the same sums taken in fp64 by torch, agreement on a clean transform, and the shift a
    # corrupted output element causes in its transform only
    import torch
    N = 1 << logN
    rdt = torch.float32 if dt == "float2" else torch.float64
    x = torch.view_as_complex(torch.rand((bs, N, 2), generator=torch.Generator(device="cuda").manual_seed(7 + logN),
                                         device="cuda", dtype=rdt) * 2 - 1)
    plan = turbofft_amd.TurboFFT(logN, dt)
    y = plan.fft(x).clone()
    plan.close()
    a, b = turbofft_amd.offline_checksums(x, y)
    c = torch.from_numpy(turbofft_amd.checksum_vector(N, dt, "exact")).cuda().to(torch.complex128)
    s3 = 0.8660253882408142
    r = torch.tensor([1.0, -0.5 - 1j * s3, -0.5 + 1j * s3], dtype=torch.complex128, device="cuda")[torch.arange(N, device="cuda") % 3]
    def re_plus_im(z):
        return z.real + z.imag
    a_ref = re_plus_im((x.to(torch.complex128) * c).sum(1))
    b_ref = re_plus_im((y.to(torch.complex128) * r).sum(1))
    eps = 1e-5 if dt == "float2" else 1e-13
    scale = (x.abs().to(torch.float64) * c.abs()).sum(1) + (y.abs().to(torch.float64)).sum(1)
    assert ((a.double() - a_ref).abs() <= eps * scale).all()
    assert ((b.double() - b_ref).abs() <= eps * scale).all()
    assert ((a.double() - b.double()).abs() <= 4 * eps * logN * scale).all()          # two-sided identity on clean data
    row, k, e = bs // 2, (5 * N) // 7, 3.0
    y[row, k] += e
    a2, b2 = turbofft_amd.offline_checksums(x, y)
    shift = (b2 - b).double()
    want = torch.zeros(bs, dtype=torch.float64, device="cuda")
    want[row] = re_plus_im(e * r[k]).item()
    assert ((shift - want).abs() <= eps * scale + 1e-6).all()
    # (transforms longer than 8192 points are summed from several partial sums in arrival order)
    assert ((a2 - a).double().abs() <= eps * scale).all()


def test_offline_ft_timing_runs_clean():
    import torch
    for dt, logN, bs in (("float2", 12, 256), ("double2", 17, 8)):
        N = 1 << logN
        x = torch.view_as_complex(torch.rand((bs, N, 2), device="cuda", dtype=torch.float32 if dt == "float2" else torch.float64) * 2 - 1)
        out = torch.empty(2 * bs * N, dtype=x.dtype, device="cuda")
        ms, flagged = turbofft_amd.offline_ft_time(logN, dt, x.data_ptr(), out.data_ptr(), bs, 1, 3,
                                                   torch.cuda.current_stream().cuda_stream)
        assert ms > 0 and flagged == 0
        ref = torch.fft.fft(x.to(torch.complex128), dim=1)
        got = out[: bs * N].view(bs, N).to(torch.complex128)
        assert (torch.linalg.vector_norm(got - ref) / torch.linalg.vector_norm(ref)).item() < (1e-5 if dt == "float2" else 1e-13) * logN


@pytest.mark.parametrize("dt,logN,bs", [("float2", 13, 200), ("double2", 10, 333), ("float2", 16, 24), ("double2", 20, 3), ("float2", 24, 1)])
@pytest.mark.parametrize("tbs", [12, 32])
def test_groups_shared_by_several_blocks(dt, logN, bs, tbs):
    """Long groups are walked by several blocks (partial checksums in slots of the plan, the block
    with a group's last ticket decides, a second launch recomputes the located tiles): flagged
    tiles, counters and the corrected output equal those of one block per group -- with injected
    errors, on clean data, with ragged last groups and parts, and again on a second execution
    (ticket words and the queue are back at zero)."""
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=1, thread_bs=tbs)
    assert all(plan.ft_part_len(i) > 0 for i in range(plan.launches))     # the default: parts of 8 tiles, or the plan row's own length
    gaps = [7, 5, 3][:plan.launches]
    for i, g in enumerate(gaps):
        plan.set_tb_gap(i, g)
    x = make(bs, 1 << logN, dt, 90 + logN)
    row = O.PlanRow.from_list(plan.plan_row())
    clean, _ = O.ft_plan_model(x, row, dt, tbs, gaps, None)
    li = plan.launches - 1
    # large enough to pass the threshold whatever the group's magnitude (it grows with the tile's columns)
    mag = max(100.0, float(np.ceil(30e-3 * (1000.0 + max(d.mag for d in clean[-1])) / 0.366)))
    ntiles = O.launch_geometry(row, bs)[li].ntiles
    every = (tbs - 1) * gaps[li] + 3
    plan.set_ft_params(1000.0, 1e-3, correct=1)
    res = {}
    for mode in ("shared", "shared again", "whole"):
        for i in range(plan.launches):
            plan.set_ft_part_len(i, 0 if mode == "whole" else 3)                 # 3: ragged last parts as well
        plan.set_injection(2, launch=li, every=every, tile_phase=1, s=0, m=0, mag=mag)
        y, c = run(plan, x)
        plan.set_injection(0)
        y0, c0 = run(plan, x)
        assert c0["detected"] == 0 and c0["checked"] == sum(plan.grid(i, bs) for i in range(plan.launches))
        res[mode] = (y, c, y0)
    y, c, y0 = res["whole"]
    injs = [O.Injection(t, 0, 0, mag) for t in range(1, ntiles, every)]
    dec, _ = O.ft_plan_model(x, row, dt, tbs, gaps, injs, inj_launch=li)
    model = sorted((l, d.tile) for l, dl in enumerate(dec) for d in dl if d.detected)
    assert sorted(c["flagged"]) == model and len(model) > 0
    for mode in ("shared", "shared again"):
        ys, cs, ys0 = res[mode]
        assert sorted(cs["flagged"]) == sorted(c["flagged"])
        assert (cs["checked"], cs["detected"], cs["corrected"], cs["uncorrectable"]) == (c["checked"], c["detected"], c["corrected"], c["uncorrectable"])
        assert np.array_equal(ys, y) and np.array_equal(ys0, y0) and np.array_equal(ys, ys0)
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance(dt, logN)
    plan.close()


# ---- thread-level verification (if_ft = 2) ----

TL_CASES = [("float2", 10, 64), ("double2", 10, 16), ("float2", 13, 32), ("double2", 15, 8), ("float2", 16, 4),
            ("float2", 21, 1), ("double2", 20, 2), ("float2", 24, 1), ("float2", 5, 1000), ("double2", 3, 777),
            ("float2", 15, 6), ("double2", 14, 5), ("float2", 23, 1)]


@pytest.mark.parametrize("dt,logN,bs", TL_CASES)
@pytest.mark.parametrize("tbs", [1, 4])
def test_thread_level_verification_matches_oracle_model(dt, logN, bs, tbs):
    # if_ft = 2: every thread checks the register-level DFTs of each pass on its own; no sums cross
    # threads, a tile a thread objects to is recomputed before it is stored.  Clean data raises
    # nothing; the reference's own injection (100 on element 0 of one tile per block of the last
    # launch, after the input sums) is caught in exactly the tiles the oracle's model of the scheme
    # flags, and the stored result is bit-identical to an undisturbed run.  A thread's two sums grow
    # with the data of its launch, not with the tile or the group, so 100 stays visible far beyond the
    # 2^10 points where the block-level sums hide it; only where the model puts it near the rule (the
    # last launch of the three-launch plans and of plans whose first digit has 2^11 points: its inputs
    # have grown to a few hundred) the test takes a larger magnitude.
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=2, if_err=1, thread_bs=tbs)
    assert all(n.endswith("_tt") for n in plan.kernel_names()), plan.kernel_names()
    gaps = [7, 5, 3][:plan.launches]
    for i, g in enumerate(gaps):
        plan.set_tb_gap(i, g)
    x = make(bs, 1 << logN, dt, logN + 21)
    row = O.PlanRow.from_list(plan.plan_row())
    geoms = O.launch_geometry(row, bs)
    plan.set_injection(0)
    y0, c0 = run(plan, x)
    assert c0["detected"] == 0 and c0["flagged"] == [] and c0["checked"] == sum(g.ntiles for g in geoms)
    assert O.rel_l2(y0, O.fft_ref(x)) <= O.tolerance(dt, logN)
    last = plan.launches - 1
    groups = O.tile_groups(geoms[last].ntiles, tbs, gaps[last])
    for mag in (100.0, 1.0e4, 1.0e6):
        injs = O.reference_injections(groups, tbs, mag)
        res, _ = O.thread_level_plan_model(x, row, dt, injs)
        model = sorted((li, int(t)) for li, (fl, _, _) in enumerate(res) for t in np.nonzero(fl)[0])
        # nothing near the rule: every injection well above it, every other thread well below
        if model == sorted((last, i.tile) for i in injs) and all(quiet < 0.1e-3 and all(v.ratio > 5e-3 for v in verdicts) for _, verdicts, quiet in res):
            break
    else:
        pytest.fail("no magnitude keeps this case away from the rule")
    print(f"thread-level case: magnitude {mag:g}, {len(injs)} injections", flush=True)
    assert mag == 100.0 or plan.launches == 3 or row.logNi[0] >= 11
    plan.set_injection(1, mag=mag)
    y, c = run(plan, x)
    want = model if len(model) <= 4096 else None
    assert c["detected"] == len(injs) == c["corrected"] and c["uncorrectable"] == 0
    if want is not None and not c["flagged_truncated"]:
        assert sorted(c["flagged"]) == want
    assert np.array_equal(y, y0)
    # detect only: the tiles are stored as computed
    plan.set_ft_params(1000.0, 1e-3, correct=0)
    y1, c1 = run(plan, x)
    assert c1["detected"] == len(injs) and c1["corrected"] == 0 and not np.array_equal(y1, y0)
    plan.close()


def test_thread_level_verification_in_an_earlier_launch_and_refusals():
    plan = turbofft_amd.TurboFFT(16, "float2", if_ft=2, thread_bs=2)
    plan.set_ft_params(1000.0, 1e-3, correct=1)
    plan.set_injection(2, launch=0, every=1 << 30, tile_phase=9, s=3, m=1, mag=100.0)
    x = make(6, 1 << 16, "float2", 5)
    y, c = run(plan, x)
    assert c["flagged"] == [(0, 9)] and c["corrected"] == 1
    assert O.rel_l2(y, O.fft_ref(x)) <= O.tolerance("float2", 16)
    with pytest.raises(turbofft_amd.TurboFFTError):
        plan.set_ft_params(1000.0, 1e-3, correct=2)          # no delayed correction: the tile never left the registers
    with pytest.raises(turbofft_amd.TurboFFTError):
        plan.set_checksum_mode("reference")                   # no table to choose
    plan.close()


@pytest.mark.parametrize("dt", ["float2", "double2"])
@pytest.mark.parametrize("logN", list(range(1, 25)))
def test_checked_plans_of_every_size_run_clean(dt, logN):
    # every row of the fault-tolerant and of the thread-level tables, the sizes no other case names included:
    # a ragged batch of clean data gives the DFT, raises nothing, and every tile of every launch was checked
    # (groups of four tiles walked by one block, groups of thirty-two shared by several, thread-level)
    bs = (1 << max(0, 20 - logN)) + 3
    x = make(bs, 1 << logN, dt, 700 + logN)
    want = O.fft_ref(x)
    for if_ft, tbs in ((1, 4), (1, 32), (2, 1)):
        plan = turbofft_amd.TurboFFT(logN, dt, if_ft=if_ft, thread_bs=tbs)
        y, c = run(plan, x)
        assert c["detected"] == 0 and c["flagged"] == [], (if_ft, tbs, c)
        assert O.rel_l2(y, want) <= O.tolerance(dt, logN), (if_ft, tbs)
        geoms = O.launch_geometry(O.PlanRow.from_list(plan.plan_row()), bs)
        if if_ft == 2:
            assert c["checked"] == sum(g.ntiles for g in geoms)
        else:
            assert c["checked"] == sum(plan.grid(i, bs) for i in range(plan.launches))
        plan.close()


def _thread_level_rows():
    import os
    out = []
    for dt in ("float2", "double2"):
        path = os.path.join(os.path.dirname(turbofft_amd.__file__), "param", "gfx950", f"param_{dt}_tt.csv")
        with open(path) as f:
            out += [(dt, [int(v) for v in line.split(",")]) for line in f if line.strip() and not line.startswith("#")]
    return out


@pytest.mark.parametrize("dt,csv_row", _thread_level_rows(), ids=lambda v: v if isinstance(v, str) else f"2^{v[0]}")
def test_thread_level_rows_of_their_own(dt, csv_row):
    # every size whose thread-level plan runs a row of its own (param_<T>_tt.csv): the plan has that shape,
    # clean data (a ragged batch) raises nothing and gives the DFT, one large error in one tile of the last
    # launch is caught in exactly that tile, and the tile recomputed before it is stored leaves the result
    # bit-identical to the undisturbed run
    logN, L = csv_row[0], csv_row[1]
    plan = turbofft_amd.TurboFFT(logN, dt, if_ft=2)
    assert plan.launches == L and list(plan.logNi) == csv_row[2:2 + L] and list(plan.BS) == csv_row[5:5 + L] and list(plan.n) == csv_row[8:8 + L]
    assert all(n.endswith("_tt") for n in plan.kernel_names()), plan.kernel_names()
    bs = (1 << max(0, 21 - logN)) + 3
    x = make(bs, 1 << logN, dt, 300 + logN)
    plan.set_ft_params(1000.0, 1e-3, correct=1)
    plan.set_injection(0)
    y0, c0 = run(plan, x)
    row = O.PlanRow.from_list(plan.plan_row())
    geoms = O.launch_geometry(row, bs)
    assert c0["detected"] == 0 and c0["checked"] == sum(g.ntiles for g in geoms)
    assert O.rel_l2(y0, O.fft_ref(x)) <= O.tolerance(dt, logN)
    last = L - 1
    tile = min(5, geoms[last].ntiles - 1)
    plan.set_injection(2, launch=last, every=1 << 30, tile_phase=tile, s=plan.BS[last] - 1, m=0, mag=1.0e6)
    y, c = run(plan, x)
    assert c["flagged"] == [(last, tile)] and c["detected"] == 1 == c["corrected"] and c["uncorrectable"] == 0
    assert np.array_equal(y, y0)
    plan.close()
