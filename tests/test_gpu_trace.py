"""Recorded-trace path on the device: branch scores, dense reference pass and
the end-to-end window replay against the oracle fed by torch.load."""
import math

import pytest
import torch

from oracle import replay as OR
from oracle import select as SEL
from oracle import trace as OT
from tests.util import rel_close, same_bits
from trace_fixture import make_trace

pytestmark = pytest.mark.gpu


def _oracle_inputs(d, t0, W):
    cat, names, numel, s_files, g_files = OT.discover(d)
    st = OT.load_file(s_files[t0])
    entries = OT.entries_for(cat, names, numel, st["meta"])
    n = sum(numel.values())
    w0, m0, v0, g0 = (OT.flat_slice(st["payload"][k], entries, n) for k in ("w", "m", "v", "g"))
    gs, metas = [], []
    for s in range(t0, t0 + W):
        f = OT.load_file(g_files[s])
        gs.append(OT.flat_slice(f["payload"], entries, n))
        metas.append(f["meta"])
    return entries, n, w0, m0, v0, g0, gs, metas, st["meta"]


@pytest.mark.parametrize("opt", ["adamw", "adams"])
@pytest.mark.parametrize("score", ["abs_g", "abs_m", "update", "coi"])
def test_branch_scores_fp64(dev, tmp_path, score, opt):
    from sga_amd import trace_io as T
    from sga_amd.replay_run import _branch_grad, branch_scores
    d = str(tmp_path)
    make_trace(d, steps=1)
    entries, n, w0, m0, v0, g0, _, _, meta = _oracle_inputs(d, 10, 1)
    catalog, names, _o, N, s_files, _g = T.discover_trace(d)
    sp = T.ShardParams(names, catalog, meta, 0, N)
    dw, dm, dv, _ = T.load_branch_state(s_files[10], sp, dev)
    dg = _branch_grad(s_files[10], sp, dev)
    assert torch.equal(dg.cpu(), g0)
    got = branch_scores(score, opt, sp, dw, dm, dv, dg, meta["step"] + 1).cpu()
    ref = OT.branch_scores(score, opt, entries, w0, m0, v0, g0, meta["step"] + 1)
    # one fp64 chain of correctly rounded operations on each side, rounded to fp32 once
    assert same_bits(got, ref)


@pytest.mark.parametrize("g_dtype,opt", [(None, "adamw"), (torch.bfloat16, "adamw"),
                                         (torch.bfloat16, "adams")])
def test_dense_pass_matches_oracle(dev, tmp_path, g_dtype, opt):
    from sga_amd import trace_io as T
    from sga_amd.replay_dense import dense_replay_dev
    d = str(tmp_path)
    W, t0 = 6, 10
    make_trace(d, steps=W, g_dtype=g_dtype)
    entries, n, w0, m0, v0, _g0, gs, metas, meta = _oracle_inputs(d, t0, W)
    lab, lab_total, den, recon, snaps = OT.dense_replay(entries, w0, m0, v0, gs, metas, t0,
                                                        (2, 6), optimizer=opt)
    catalog, names, _o, N, s_files, g_files = T.discover_trace(d)
    sp = T.ShardParams(names, catalog, meta, 0, N)
    dw, dm, dv, _ = T.load_branch_state(s_files[t0], sp, dev)
    reader = T.WindowReader(g_files, T.window_steps_for(g_files, t0, W), sp, dev)
    total, dden, drecon, dsnaps, dense = dense_replay_dev(sp.entries, dw, dm, dv, reader, t0,
                                                          (2, 6), optimizer=opt)
    # same rounding recipe as the in-place host chain: moments bitwise
    ow, om, ov = w0.clone(), m0.clone(), v0.clone()
    olab = torch.zeros(n)
    for si in range(W):
        for e in entries:
            a, b = e["a"], e["a"] + e["n"]
            OR.opt_step_inplace(gs[si][a:b].clone(), om[a:b], ov[a:b], ow[a:b], olab[a:b],
                                OT.lr_for(metas[si], e["group"]), e["wd"], e["b1"], e["b2"],
                                *OR.bc_pair(opt, t0 + si + 1, e["b1"], e["b2"]), e["eps"],
                                optimizer=opt)
    assert torch.equal(dense.m.cpu(), om) and torch.equal(dense.v.cpu(), ov)
    assert same_bits(dense.w, ow)
    assert torch.equal(olab, lab)
    assert same_bits(dense.label, lab)
    assert abs(total - lab_total) <= 1e-5 * lab_total
    assert set(dden) == {2, 6}
    for h in (2, 6):
        assert abs(dden[h] - den[h]) <= 1e-5 * den[h]
        assert same_bits(dsnaps[h], snaps[h])
    for a, b, mt in zip(drecon, recon, metas):
        assert a["coef_dense"] == b["coef_dense"]
        assert abs(a["recon_grad_norm"] - b["recon_grad_norm"]) <= 1e-9 * b["recon_grad_norm"]
        if g_dtype is None:     # post-clip g / coef reconstructs the recorded pre-clip norm
            assert abs(a["recon_rel_err"]) < 1e-5
            assert a["grad_norm"] == mt["grad_norm"]


@pytest.mark.parametrize("clip,g_dtype,semantics", [(0.0, torch.bfloat16, "topk"),
                                                    (0.3, None, "topk"),
                                                    (0.0, torch.bfloat16, "balanced-histogram")])
def test_replay_window_end_to_end(dev, tmp_path, clip, g_dtype, semantics):
    """One selection semantics at BOTH select sites (the branch-point select
    and every boundary re-selection, replay_fused.py:1340-1344), against the
    oracle's loop under the same semantics."""
    from sga_amd.replay_run import Config, replay_window
    d = str(tmp_path)
    W, t0 = 9, 10
    make_trace(d, steps=W, g_dtype=g_dtype, clip=clip, absent=(2, 3))
    specs = [("abs_g", 1.0, 1), ("abs_g", 10.0, 4), ("abs_m", 1.0, 3),
             ("abs_g", 1.0, 4, "adams", True), ("abs_g", 5.0, 4, "adamw", False, 0.25)]
    res = replay_window(d, t0, W, [Config(*s) for s in specs], (1, 4, 9, 99), dev,
                        selection_semantics=semantics)
    assert res["window_steps"] == list(range(t0, t0 + W)) and res["horizons"] == [1, 4, 9]
    entries, n, w0, m0, v0, g0, gs, metas, meta = _oracle_inputs(d, t0, W)
    ocfg = [OR.Config(*s) for s in specs]
    dense = {o: OT.dense_replay(entries, w0, m0, v0, gs, metas, t0, (1, 4, 9), optimizer=o)
             for o in ("adamw", "adams")}
    for ci, c in enumerate(ocfg):
        sc = OT.branch_scores(c.score, c.optimizer, entries, w0, m0, v0, g0, meta["step"] + 1)
        if semantics == "topk":
            sel0, _ = SEL.select_topk_flat(sc, SEL.replay_k(n, c.ratio))
        else:
            sel0, _ = SEL.shard_select_balanced(sc, SEL.replay_k(n, c.ratio), entries)
        ometas = [{"clip_grad": m["clip_grad"], "grad_norm": m["grad_norm"],
                   "lr": m["lr"]} for m in metas]
        o = OR.group_replay(entries, w0, m0, v0, [sel0], [c], gs, ometas, t0,
                            horizons=(1, 4, 9), snapshots=dense[c.optimizer][4],
                            selection_semantics=semantics)[0]
        r = res["configs"][ci]
        s = r["group"].state[r["slot"]]
        den = dense[c.optimizer][2]
        for h in (1, 4, 9):
            assert abs(res["dense"][c.optimizer]["den_at"][h] - den[h]) <= 1e-5 * den[h]
            # the reference's own band for ||w_s - w_d|| (test_replay_cycle.py:318-319)
            assert abs(r["dist_at"][h] - o["dist"][h]) <= 1e-3 * max(1.0, o["dist"][h]), (ci, h)
            # tighter, with a floor relative to the dense movement: at T = 1 the oracle's own clip
            # coefficient undoes the recorded one exactly (distance 0.0), the device's differs in
            # its last bits (order of the norm's sum) and leaves a few ulps of w
            assert abs(r["dist_at"][h] - o["dist"][h]) <= 2e-3 * o["dist"][h] + 1e-6 * den[h], (ci, h)
            assert r["distortion"][h] == r["dist_at"][h] / res["dense"][c.optimizer]["den_at"][h]
        if c.T == 1:
            assert r["dist_at"][9] <= 1e-3 * den[9]          # T = 1 is the dense trajectory
        atol = 1e-6 * W * 5e-5 * 3
        if clip == 0.0:
            assert torch.equal(s["sel"].cpu().bool(), o["sel"]), ci
            assert torch.equal(s["m"].cpu(), o["m"]) and torch.equal(s["v"].cpu(), o["v"]), ci
            assert torch.equal(s["res"].cpu(), o["res"]), ci
            assert same_bits(s["w"], o["w"]), ci
        else:
            # the clip coefficient comes from a double sum whose order differs between the two
            # sides (1e-6 band): a last-bit change of the coefficient moves a few selections
            agree = float((s["sel"].cpu().bool() == o["sel"]).float().mean())
            assert agree > 0.9999, (ci, agree)
            bad, worst = rel_close(s["w"], o["w"], 1e-5, atol=10 * atol)
            assert bad == 0, (ci, worst)
