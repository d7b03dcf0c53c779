"""Pins the arithmetic oracles (scores, AdamW commit, replay commit, cycle
machine, pack) against independent float64 closed forms, brute force and the
identities the reference's own tests assert."""
import math

import pytest
import torch

from oracle import adamw as A
from oracle import fused_step as F
from oracle import kernels as OK
from oracle import replay as R
from oracle import scores as S
from oracle import select as SEL


def _f64_scores(w, m, v, g, b1, b2, eps, wd, bc1, bc2, adams=False):
    w, m, v, g = (t.double() for t in (w, m, v, g))
    m_new = b1 * m + (1 - b1) * g
    if adams:
        v_new = b2 * m * m + (1 - b2) * g * g
        v0 = b2 * m * m
        bc1 = bc2 = 1.0
    else:
        v_new = b2 * v + (1 - b2) * g * g
        v0 = b2 * v
    ug = (m_new / bc1) / ((v_new / bc2).sqrt() + eps)
    u0 = (b1 * m / bc1) / ((v0 / bc2).sqrt() + eps)
    return {"abs_g": g.abs(), "abs_m": m.abs(), "update": wd * w + ug,
            "coi": (ug - u0).abs()}


def _state(n, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g), torch.randn(n, generator=g) * 0.1,
            torch.rand(n, generator=g) * 0.1 + 1e-4, torch.randn(n, generator=g))


@pytest.mark.parametrize("opt", ["adamw", "adams"])
def test_scores_vs_f64(opt):
    b1, b2, eps, wd, step = 0.9, 0.95, 1e-8, 1e-2, 7
    bc1, bc2 = 1 - b1 ** step, 1 - b2 ** step
    w, m, v, g = _state(513, 3)
    ref = _f64_scores(w, m, v, g, b1, b2, eps, wd, bc1, bc2, adams=opt == "adams")
    for name in S.FORMULAS:
        out = S.get_formula(name)(w, m, v, g, b1, b2, eps, wd, bc1, bc2,
                                  optimizer=opt)
        torch.testing.assert_close(out.double(), ref[name], rtol=1e-5,
                                   atol=2e-6 if name == "coi" else 1e-7)
        if opt == "adams":   # replay-side substitution gives the same thing
            out2 = S.score_formula(name, w, m, v, g, b1, b2, eps, wd, bc1, bc2,
                                   "adams", update_includes_wd=True)
            assert torch.equal(out, out2)
    with pytest.raises(ValueError) as ei:
        S.get_formula("nope")
    assert "nope" in str(ei.value) and "abs_g" in str(ei.value)
    u = S.update(w, m, v, g, b1, b2, eps, wd, bc1, bc2, update_includes_wd=False)
    torch.testing.assert_close(u.double(), ref["update"] - wd * w.double(),
                               rtol=1e-5, atol=1e-7) if opt == "adamw" else None


def _f64_adamw(p, g, m, v, lr, b1, b2, eps, wd, step):
    p, g, m, v = (t.double() for t in (p, g, m, v))
    m2 = b1 * m + (1 - b1) * g
    v2 = b2 * v + (1 - b2) * g * g
    upd = wd * p + (m2 / (1 - b1 ** step)) / ((v2 / (1 - b2 ** step)).sqrt() + eps)
    return p - lr * upd, m2, v2, upd


def test_grad_correct_vs_f64_and_fused_knobs():
    n = 3000
    lr, b1, b2, eps, wd, step = 1e-3, 0.9, 0.95, 1e-8, 0.1, 5
    p, m, v, g = _state(n, 11)
    mask = (torch.rand(n, generator=torch.Generator().manual_seed(1)) < 0.3).to(torch.uint8)
    # sparse step vs f64 with g' = where(mask, g, 0)
    pp, gg, mm, vv = p.clone(), g.clone(), m.clone(), v.clone()
    A.adamw_grad_correct(pp, gg, mm, vv, lr, b1, b2, eps, wd, step, mask=mask)
    rp, rm, rv, _ = _f64_adamw(p, torch.where(mask > 0, g, torch.zeros(())), m, v,
                               lr, b1, b2, eps, wd, step)
    torch.testing.assert_close(pp.double(), rp, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(mm.double(), rm, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(vv.double(), rv, rtol=1e-4, atol=1e-6)
    assert torch.equal(gg, g)          # untouched without clear/fold
    # fused coeff/clear/fold == standalone 3-pass sequence, bitwise
    # (tests/test_kernels_gpu.py:227-268)
    p1, g1, m1, v1 = p.clone(), g.clone(), m.clone(), v.clone()
    A.adamw_grad_correct(p1, g1, m1, v1, lr, b1, b2, eps, wd, step, mask=mask,
                         coeff=0.37, clear=True, fold=True, interval=4.0)
    p2, g2, m2, v2 = p.clone(), g.clone(), m.clone(), v.clone()
    g2 = torch.where(mask > 0, g2 * 0.37, g2)
    A.adamw_grad_correct(p2, g2, m2, v2, lr, b1, b2, eps, wd, step, mask=mask)
    g2[mask > 0] = 0.0
    g2 /= 4.0
    for a, b in ((p1, p2), (g1, g2), (m1, m2), (v1, v2)):
        assert torch.equal(a, b)
    # full step: score lands in grad, commit is mask-blind
    for name in S.FORMULAS:
        p3, g3, m3, v3 = p.clone(), g.clone(), m.clone(), v.clone()
        A.adamw_grad_correct(p3, g3, m3, v3, lr, b1, b2, eps, wd, step,
                             emit_score=name)
        rp, rm, rv, _ = _f64_adamw(p, g, m, v, lr, b1, b2, eps, wd, step)
        torch.testing.assert_close(p3.double(), rp, rtol=1e-5, atol=1e-7)
        ref = _f64_scores(p, m, v, g, b1, b2, eps, wd, 1 - b1 ** step, 1 - b2 ** step)
        # coi subtracts two O(1) directions: tolerance at operand scale
        torch.testing.assert_close(g3.double(), ref[name], rtol=1e-5,
                                   atol=2e-6 if name == "coi" else 1e-7)
    # dual-lr: p == w - where(mask, lr, lr*s) * score(update); m/v mask-blind
    p4, g4, m4, v4 = p.clone(), g.clone(), m.clone(), v.clone()
    A.adamw_grad_correct(p4, g4, m4, v4, lr, b1, b2, eps, wd, step, mask=mask,
                         emit_score="update", inactive_lr_scale=0.25)
    p5, g5, m5, v5 = p.clone(), g.clone(), m.clone(), v.clone()
    A.adamw_grad_correct(p5, g5, m5, v5, lr, b1, b2, eps, wd, step, emit_score="update")
    assert torch.equal(m4, m5) and torch.equal(v4, v5) and torch.equal(g4, g5)
    assert torch.equal(p4, p - torch.where(mask > 0, lr, lr * 0.25) * g4)
    p6 = p.clone()
    A.adamw_grad_correct(p6, g.clone(), m.clone(), v.clone(), lr, b1, b2, eps, wd,
                         step, mask=mask, emit_score="update", inactive_lr_scale=0.0)
    assert torch.equal(p6[mask == 0], p[mask == 0])


def test_knob_refusals():
    z = torch.zeros(4)
    mk = torch.ones(4, dtype=torch.uint8)
    for kw, sub in (
            (dict(coeff=0.5), "requires a sparse step"),
            (dict(mask=mk, emit_score="update"), "masked-commit full step"),
            (dict(mask=mk, inactive_lr_scale=0.5), "requires a full step"),
            (dict(mask=mk, emit_score="update", inactive_lr_scale=float("nan")),
             "inactive_lr_scale"),
            (dict(emit_score="bogus"), "no _grad_correct_kernel branch")):
        with pytest.raises(ValueError) as ei:
            A.adamw_grad_correct(z.clone(), z.clone(), z.clone(), z.clone(), 1e-3,
                                 0.9, 0.95, 1e-8, 0.0, 1, **kw)
        assert sub in str(ei.value)


def test_compact_commit_equals_masked_commit_and_dir_table():
    n_bucket, rec_start, n = 9000, 1500, 4000
    lr, b1, b2, eps, wd, step = 1e-3, 0.9, 0.95, 1e-8, 0.1, 3
    gen = torch.Generator().manual_seed(2)
    buf = torch.randn(n_bucket, generator=gen)
    mask = (torch.rand(n_bucket, generator=gen) < 0.2).to(torch.uint8)
    idx = OK.compact_mask_u8(mask)
    p, m, v, _ = _state(n, 5)
    # masked path on the record's slice
    b1_, p1, m1, v1 = buf.clone(), p.clone(), m.clone(), v.clone()
    A.adamw_grad_correct(p1, b1_[rec_start:rec_start + n], m1, v1, lr, b1, b2, eps,
                         wd, step, mask=mask[rec_start:rec_start + n], clear=True)
    # compact path: pack first, then merge-join commit
    b2_, p2, m2, v2 = buf.clone(), p.clone(), m.clone(), v.clone()
    vals = torch.empty(idx.numel())
    OK.pack_selected(b2_, idx, vals, 1.0)
    assert torch.equal(vals, buf[mask.bool()]) and bool((b2_[mask.bool()] == 0).all())
    assert torch.equal(b2_[~mask.bool()], buf[~mask.bool()])
    A.adamw_grad_correct_compact(p2, b2_[rec_start:rec_start + n], m2, v2, idx, vals,
                                 rec_start, lr, b1, b2, eps, wd, step)
    assert torch.equal(p1, p2) and torch.equal(m1, m2) and torch.equal(v1, v2)
    assert torch.equal(b1_[rec_start:rec_start + n], b2_[rec_start:rec_start + n])
    # dir table == brute-force lower_bound
    tab = A.build_dir_table(idx, n_bucket)
    il = idx.tolist()
    for j in range(tab.numel()):
        assert tab[j].item() == sum(1 for x in il if x < j * 1024)
    assert A.build_dir_table(torch.empty(0, dtype=torch.int32), 5000).tolist() == [0] * 6


def test_pack_scatter_bruteforce_and_bf16():
    gen = torch.Generator().manual_seed(9)
    grad = torch.randn(1000, generator=gen)
    idx = torch.tensor([3, 17, 500, 999], dtype=torch.int32)
    for factor in (1.0, 0.125):
        g = grad.clone()
        vals = torch.empty(4)
        OK.pack_selected(g, idx, vals, factor)
        for j, i in enumerate(idx.tolist()):
            assert vals[j].item() == (grad[i] * factor if factor != 1.0 else grad[i]).item()
            assert g[i].item() == 0.0
        vb = torch.empty(4, dtype=torch.bfloat16)
        g = grad.clone()
        OK.pack_selected(g, idx, vb, factor)
        assert torch.equal(vb, (grad[idx.long()] * factor).to(torch.bfloat16))
        dst = torch.zeros(1000)
        OK.scatter_selected(dst, idx, vals)
        assert torch.equal(dst[idx.long()], vals) and int((dst != 0).sum()) <= 4
    tot = torch.zeros(())
    OK.compact_norm_sq_contribution(vals, tot)
    assert abs(tot.item() - sum(x * x for x in vals.tolist())) < 1e-5
    mask = torch.zeros(1000, dtype=torch.uint8)
    mask[idx.long()] = 1
    tot2 = torch.zeros(())
    OK.masked_norm_sq_contribution(grad, mask, tot2)
    assert abs(tot2.item() - sum(grad[i].item() ** 2 for i in idx.tolist())) < 1e-5
    pl = OK.mask_layout_pack(grad, mask, 1.0, slices=2)
    assert [x.numel() for x in pl] == [2, 2] and torch.equal(torch.cat(pl), grad[mask.bool()])


def _f64_replay(q, m, v, w, lr, wd, b1, b2, bc1, bc2, eps, adams, inactive=None, lr_i=None):
    q, m, v, w = (t.double() for t in (q, m, v, w))
    v2 = (b2 * m * m if adams else b2 * v) + (1 - b2) * q * q
    m2 = b1 * m + (1 - b1) * q
    upd = (m2 / bc1) / ((v2 / bc2).sqrt() + eps)
    if inactive is None:
        w2 = w * (1 - lr * wd) - lr * upd
    else:
        w2 = w - torch.where(inactive, lr_i, lr) * (wd * w + upd)
    return m2, v2, w2, upd


@pytest.mark.parametrize("opt", ["adamw", "adams"])
@pytest.mark.parametrize("lr,wd,count", [(1e-3, .01, 7), (3e-4, .01, 1), (1e-3, 0.0, 100)])
def test_replay_commit_vs_f64(opt, lr, wd, count):
    b1, b2, eps = 0.9, 0.999, 1e-8
    w, m, v, q = _state(2000, count)
    bc1, bc2 = R.bc_pair(opt, count, b1, b2)
    inactive = torch.rand(2000, generator=torch.Generator().manual_seed(3)) < 0.5
    for ina, lri in ((None, None), (inactive, lr * 0.3)):
        mm, vv, ww, lab = m.clone(), v.clone(), w.clone(), torch.zeros(2000)
        R.opt_step_inplace(q, mm, vv, ww, lab, lr, wd, b1, b2, bc1, bc2, eps,
                           optimizer=opt, inactive=ina, lr_inactive=lri)
        rm, rv, rw, ru = _f64_replay(q, m, v, w, lr, wd, b1, b2, bc1, bc2, eps,
                                     opt == "adams", ina, lri)
        torch.testing.assert_close(mm.double(), rm, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(vv.double(), rv, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(ww.double(), rw, rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(lab.double(), (lr * ru) ** 2, rtol=1e-4, atol=1e-9)
    with pytest.raises(ValueError):
        R.opt_step_inplace(q, m, v, w, None, lr, wd, b1, b2, bc1, bc2, eps,
                           inactive=inactive)


def test_coef_dense():
    assert R.coef_dense_for(0.0, 5.0) == 1.0
    assert R.coef_dense_for(1.0, float("nan")) == 1.0
    assert R.coef_dense_for(1.0, 0.5) == 1.0
    assert R.coef_dense_for(0.3, 2.0) == 0.3 / (2.0 + 1e-6)


def _spec_balanced(score, k, sizes):
    """Balanced-histogram select from its wording (_histogram.py:115-123,
    203-216; replay_fused.py:405-489 with p_off = 0): the sample is every
    eighth element of each tensor counted from the tensor's own start, r the
    rounded rank of the k-th largest inside the sample, the crossing bin the
    r-th smallest sampled top-16 pattern, and every coordinate whose top 16
    bits reach that bin is selected."""
    top = score.float().abs().view(torch.int32) >> 16
    sample, off = [], 0
    for sz in sizes:
        sample += top[off:off + sz][::8].tolist()
        off += sz
    sample.sort()
    n = score.numel()
    r = max(1, round(len(sample) * (n - k + 1) / n))
    return top >= sample[r - 1]


def _spec_cycle(w0, m0, v0, grads, norms, lr, clip, t0, k, T, b1, b2, eps, wd,
                fold=False, optimizer="adamw", dual_lr=1.0, semantics="topk", sizes=None):
    """From-spec loop (shape of tests/test_replay_cycle.py:141-223), abs_g
    score, written out of place from the formulas: AdamW, or AdamS (the second
    moment rebuilt from the PRE-commit m, no bias corrections: replay.py:708-729);
    at a boundary with dual_lr != 1 the whole displacement wd*w + upd is applied
    at lr on the coordinates of the OUTGOING mask and at lr*dual_lr elsewhere
    (replay_fused.py:1817-1824, 1866-1877; replay.py:674-684)."""
    def select(score):
        if semantics == "topk":
            return SEL.select_topk_flat(score, k)[0]
        return _spec_balanced(score, k, sizes)

    def commit(w, m, v, q, count, lr_vec):
        if optimizer == "adams":
            v = b2 * (m * m) + (1 - b2) * q * q
            m = b1 * m + (1 - b1) * q
            upd = m / (torch.sqrt(v) + eps)
        else:
            m = b1 * m + (1 - b1) * q
            v = b2 * v + (1 - b2) * q * q
            upd = (m / (1 - b1 ** count)) / (torch.sqrt(v / (1 - b2 ** count)) + eps)
        return w - lr_vec * (wd * w + upd), m, v
    ws, ms, vs = w0.clone(), m0.clone(), v0.clone()
    res = torch.zeros_like(w0)
    sel = select(grads[0].abs())
    for si, gl in enumerate(grads):
        count = t0 + si + 1
        cd = min(1.0, clip / (norms[si] + 1e-6)) if clip > 0 else 1.0
        g = gl / cd
        lr_vec = lr
        if si % T == 0:
            if fold and si > 0:
                res = res / T
            qp = g + res
            coef = min(1.0, clip / (float(qp.norm()) + 1e-6)) if clip > 0 else 1.0
            q = qp * coef
            outgoing = sel
            if si > 0 and si + 1 < len(grads):
                sel = select(q.abs())
            if dual_lr != 1.0:
                lr_vec = torch.where(outgoing, torch.tensor(lr), torch.tensor(lr * dual_lr))
            res = torch.zeros_like(res)
        else:
            coef = min(1.0, clip / (float((g * sel).norm()) + 1e-6)) if clip > 0 else 1.0
            q = g * sel * coef
            res = res + g * (~sel)
        ws, ms, vs = commit(ws, ms, vs, q, count, lr_vec)
    return ws, sel, res


@pytest.mark.parametrize("T,fold,optimizer,dual_lr,semantics", [
    (1, False, "adamw", 1.0, "topk"), (4, False, "adamw", 1.0, "topk"),
    (4, True, "adamw", 1.0, "topk"), (3, False, "adamw", 1.0, "topk"),
    (4, False, "adams", 1.0, "topk"), (3, True, "adams", 2.0, "topk"),
    (4, False, "adamw", 0.25, "topk"), (2, False, "adamw", 0.0, "topk"),
    (4, False, "adamw", 1.0, "balanced-histogram"),
    (3, True, "adams", 0.25, "balanced-histogram")])
def test_group_replay_vs_spec(T, fold, optimizer, dual_lr, semantics):
    """The oracle's group loop against the from-spec loop on every arm of the
    replay axis product: cycle length, fold, AdamS, the boundary dual-lr split
    against the outgoing mask, and both selection semantics."""
    n, W, t0 = 5000, 9, 10
    b1, b2, eps, wd, lr, clip = 0.9, 0.95, 1e-8, 0.1, 5e-5, 0.3
    gen = torch.Generator().manual_seed(2026)
    w0 = torch.randn(n, generator=gen) * 0.02
    m0 = torch.randn(n, generator=gen) * 1e-3
    v0 = torch.rand(n, generator=gen) * 1e-6
    grads = [torch.randn(n, generator=gen) * 1e-2 for _ in range(W)]
    norms = [float(g.norm()) for g in grads]
    k = SEL.replay_k(n, 10.0)
    sizes = [3001, 1999]                    # the second tensor starts off the stride-8 grid
    entries = [{"a": 0, "n": sizes[0], "b1": b1, "b2": b2, "eps": eps, "wd": wd},
               {"a": sizes[0], "n": sizes[1], "b1": b1, "b2": b2, "eps": eps, "wd": wd}]
    cfg = R.Config("abs_g", 10.0, T, optimizer=optimizer, fold=fold, dual_lr=dual_lr)
    if semantics == "topk":
        sel0 = SEL.select_topk_flat(grads[0].abs(), k)[0]
    else:
        sel0 = _spec_balanced(grads[0].abs(), k, sizes)
        assert torch.equal(sel0, SEL.shard_select_balanced(grads[0].abs(), k, entries)[0])
        assert abs(int(sel0.sum()) - k) < 0.02 * n and int(sel0.sum()) != k
    metas = [{"clip_grad": clip, "grad_norm": norms[i], "lr": lr} for i in range(W)]
    out = R.group_replay(entries, w0, m0, v0, [sel0], [cfg], grads, metas, t0,
                         selection_semantics=semantics)[0]
    ws, sel, res = _spec_cycle(w0, m0, v0, grads, norms, lr, clip, t0, k, T, b1, b2,
                               eps, wd, fold, optimizer, dual_lr, semantics, sizes)
    assert torch.equal(out["sel"], sel)
    torch.testing.assert_close(out["w"], ws, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(out["res"], res, rtol=1e-5, atol=1e-9)
    if T == 1:   # every step a boundary: residual never survives a step
        assert float(out["res"].abs().max()) == 0.0
    if dual_lr == 0.0:
        # scale 0 freezes the coordinates outside the outgoing mask at every boundary
        # (tests/test_plugins_unit.py:992-1069): with T = 2 the one step that moves them is
        # the masked step, where q = 0 there and only m's decay and weight decay act
        assert not torch.equal(out["w"], w0)


def test_fused_step_end_state_invariant():
    """buf[idx]==0 and buf[~mask]==(g+r)[~mask] bitwise
    (tests/test_plugins_unit.py:785-837)."""
    n = 1 << 14
    gen = torch.Generator().manual_seed(0)
    segs = [dict(start=0, n=10000, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.1),
            dict(start=10000, n=n - 10000, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.0)]
    p = torch.randn(n, generator=gen) * 0.02
    m, v, r = torch.zeros(n), torch.zeros(n), torch.zeros(n)
    for step in range(1, 4):
        g = (torch.randn(n, generator=gen) * 1e-3).to(torch.bfloat16)
        before = r + g.float()
        p0, m0, v0 = p.clone(), m.clone(), v.clone()
        idx, vals, mask, th = F.fused_sparse_step(g, r, p, m, v, segs, step,
                                                  ratio_percent=1.0,
                                                  values_dtype=torch.bfloat16)
        assert idx.numel() == SEL.k_for(n, 1.0) == int(mask.sum())
        assert bool((r[mask] == 0).all()) and torch.equal(r[~mask], before[~mask])
        assert torch.equal(vals, before[mask].to(torch.bfloat16))
        gq = torch.where(mask, before.to(torch.bfloat16).float(), torch.zeros(()))
        rp, rm, rv, _ = _f64_adamw(p0[:10000], gq[:10000], m0[:10000], v0[:10000],
                                   1e-4, 0.9, 0.95, 1e-8, 0.1, step)
        torch.testing.assert_close(p[:10000].double(), rp, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(m[:10000].double(), rm, rtol=1e-5, atol=1e-9)


def test_adams_grad_correct_vs_f64():
    n = 2000
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.95, 1e-8, 0.1
    p, m, v, g = _state(n, 21)
    mask = (torch.rand(n, generator=torch.Generator().manual_seed(1)) < 0.3).to(torch.uint8)
    pp, gg, mm, vv = p.clone(), g.clone(), m.clone(), v.clone()
    A.adams_grad_correct(pp, gg, mm, vv, lr, b1, b2, eps, wd, mask=mask, clear=True)
    ge = torch.where(mask > 0, g, torch.zeros(())).double()
    m2 = b1 * m.double() + (1 - b1) * ge
    v2 = b2 * m.double() ** 2 + (1 - b2) * ge * ge
    p2 = p.double() - lr * (wd * p.double() + m2 / (v2.sqrt() + eps))
    torch.testing.assert_close(mm.double(), m2, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(vv.double(), v2, rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(pp.double(), p2, rtol=1e-5, atol=1e-7)
    assert bool((gg[mask > 0] == 0).all()) and torch.equal(gg[mask == 0], g[mask == 0])
    for name in S.FORMULAS:
        p3, g3 = p.clone(), g.clone()
        A.adams_grad_correct(p3, g3, m.clone(), v.clone(), lr, b1, b2, eps, wd, emit_score=name)
        ref = _f64_scores(p, m, v, g, b1, b2, eps, wd, 1.0, 1.0, adams=True)
        torch.testing.assert_close(g3.double(), ref[name], rtol=1e-5,
                                   atol=2e-6 if name == "coi" else 1e-7)


def test_trace_dense_replay_against_fp64_recursion(tmp_path):
    """oracle.trace.dense_replay (the dense reference pass over a recorded
    window) against the textbook AdamW recursion in float64: weights, label
    sum((lr*upd)^2), horizon norms ||w - w0|| and the pre-clip reconstruction
    norm sqrt(sum((g/coef)^2))."""
    import math
    from oracle import trace as OT
    from trace_fixture import make_trace
    d = str(tmp_path)
    W, t0 = 6, 10
    make_trace(d, steps=W, clip=0.3)
    cat, names, numel, s_files, g_files = OT.discover(d)
    st = OT.load_file(s_files[t0])
    entries = OT.entries_for(cat, names, numel, st["meta"])
    n = sum(numel.values())
    w0, m0, v0 = (OT.flat_slice(st["payload"][k], entries, n) for k in ("w", "m", "v"))
    gs, metas = [], []
    for s in range(t0, t0 + W):
        f = OT.load_file(g_files[s])
        gs.append(OT.flat_slice(f["payload"], entries, n))
        metas.append(f["meta"])
    lab, lab_total, den, recon, snaps = OT.dense_replay(entries, w0, m0, v0, gs, metas, t0, (3, 6))
    w, m, v = w0.double(), m0.double(), v0.double()
    lab64 = torch.zeros(n, dtype=torch.float64)
    for si in range(W):
        g = gs[si].double()
        for e in entries:
            a, b = e["a"], e["a"] + e["n"]
            lr = metas[si]["lr"][e["group"]]
            t = t0 + si + 1
            m[a:b] = e["b1"] * m[a:b] + (1 - e["b1"]) * g[a:b]
            v[a:b] = e["b2"] * v[a:b] + (1 - e["b2"]) * g[a:b] ** 2
            upd = (m[a:b] / (1 - e["b1"] ** t)) / ((v[a:b] / (1 - e["b2"] ** t)).sqrt() + e["eps"])
            w[a:b] = w[a:b] * (1 - lr * e["wd"]) - lr * upd
            lab64[a:b] += (lr * upd) ** 2
        coef = min(1.0, metas[si]["clip_grad"] / (metas[si]["grad_norm"] + 1e-6))
        assert recon[si]["coef_dense"] == coef
        ref_norm = math.sqrt(float(((g / coef) ** 2).sum()))
        assert abs(recon[si]["recon_grad_norm"] - ref_norm) <= 1e-9 * ref_norm
        # the fixture records post-clip gradients: g / coef is the pre-clip gradient
        assert abs(ref_norm - metas[si]["grad_norm"]) <= 1e-5 * ref_norm
        if si + 1 in (3, 6):
            ref_den = math.sqrt(float(((w - w0.double()) ** 2).sum()))
            assert abs(den[si + 1] - ref_den) <= 1e-4 * ref_den
            assert float((snaps[si + 1].double() - w).abs().max()) <= 1e-6
    assert float((lab.double() - lab64).abs().max()) <= 1e-5 * float(lab64.max())
    assert abs(lab_total - float(lab64.sum())) <= 1e-5 * float(lab64.sum())


def test_trace_branch_scores_against_fp64_closed_form():
    """oracle.trace.branch_scores: |registry score| in double, rounded once to
    fp32 -- against the formulas written out independently in float64."""
    from oracle import trace as OT
    gen = torch.Generator().manual_seed(3)
    n = 50_000
    w = torch.randn(n, generator=gen) * 0.02
    m = torch.randn(n, generator=gen) * 1e-3
    v = torch.rand(n, generator=gen) * 1e-5 + 1e-12
    g = torch.randn(n, generator=gen) * 1e-2
    e = {"a": 0, "n": n, "b1": 0.9, "b2": 0.95, "eps": 1e-8, "wd": 0.1}
    t = 11
    W, M, V, G = (x.double() for x in (w, m, v, g))
    bc1, bc2 = 1 - 0.9 ** t, 1 - 0.95 ** t
    def u(gg, vv, c1, c2):
        return ((0.9 * M + 0.1 * gg) / c1) / (((0.95 * vv + 0.05 * gg * gg) / c2).sqrt() + 1e-8)
    want = {("abs_g", "adamw"): G.abs(), ("abs_m", "adams"): M.abs(),
            ("update", "adamw"): (0.1 * W + u(G, V, bc1, bc2)).abs(),
            ("update", "adams"): (0.1 * W + u(G, M * M, 1.0, 1.0)).abs(),
            ("coi", "adamw"): (u(G, V, bc1, bc2) - u(torch.zeros_like(G), V, bc1, bc2)).abs(),
            ("coi", "adams"): (u(G, M * M, 1.0, 1.0) - u(torch.zeros_like(G), M * M, 1.0, 1.0)).abs()}
    for (score, opt), ref in want.items():
        got = OT.branch_scores(score, opt, [e], w, m, v, g, t).double()
        # fp32 rounding of the result (2^-24) plus operand-scale cancellation for coi
        scale = ref.abs() + (3.0 if score == "coi" else 0.0) * 1e-7
        assert float(((got - ref).abs() / (scale + 1e-30)).max()) <= 2e-7, (score, opt)


def test_clip_routes_against_closed_form():
    """oracle.clip.masked_clip_grad_norm: norm = sqrt of the fp64 sum over the
    contributing coordinates; coefficient clip/(norm+1e-6); each route scales
    exactly the coordinates engine.py:1172-1216 scales."""
    from types import SimpleNamespace
    from oracle.clip import masked_clip_grad_norm

    class Rec:
        def __init__(self, grad, bucket, a, b):
            self.grad, self.bucket_state, self.a, self.b = grad, bucket, a, b

        def mask_u8(self):
            m = self.bucket_state.active_mask_u8
            return None if m is None else m[self.a:self.b]

    def build(masked_tail=True):
        gen = torch.Generator().manual_seed(2)
        flat = torch.randn(3000, generator=gen)
        mask = (torch.rand(3000, generator=gen) < 0.1).to(torch.uint8)
        b = SimpleNamespace(active_mask_u8=mask)
        b2 = SimpleNamespace(active_mask_u8=mask if masked_tail else None)
        recs = [Rec(flat[0:1000], b, 0, 1000), Rec(flat[1000:3000], b2, 1000, 3000)]
        return recs, flat, mask

    recs, flat, mask = build()
    before = flat.clone()
    full = float(flat.double().pow(2).sum().sqrt())
    sel = float(flat.double()[mask > 0].pow(2).sum().sqrt())
    n, c = masked_clip_grad_norm(recs, 0.0, True)
    assert abs(n - full) < 1e-5 * full and c == 1.0 and torch.equal(flat, before)
    n, c = masked_clip_grad_norm(recs, 0.5 * full, True)          # full step: scaled in place
    assert c == 1.0 and torch.allclose(flat, before * (0.5 * full / (n + 1e-6)), rtol=1e-6)
    recs, flat, mask = build()
    before = flat.clone()
    n, c = masked_clip_grad_norm(recs, 0.5 * sel, False)          # sparse: coefficient handed on
    assert abs(n - sel) < 1e-5 * sel and abs(c - 0.5 * sel / (n + 1e-6)) < 1e-12
    assert torch.equal(flat, before)
    n, c = masked_clip_grad_norm(recs, 0.5 * sel, False, trace_dumps=True)   # dump step
    assert c == 1.0 and torch.equal(flat[mask == 0], before[mask == 0])
    assert torch.allclose(flat[mask > 0], before[mask > 0] * (0.5 * sel / (n + 1e-6)), rtol=1e-6)
    recs, flat, mask = build(masked_tail=False)                   # mask-less record counts whole
    before = flat.clone()
    mix = float((before.double()[:1000][mask[:1000] > 0].pow(2).sum()
                 + before.double()[1000:].pow(2).sum()).sqrt())
    n, c = masked_clip_grad_norm(recs, 0.5 * mix, False)
    assert abs(n - mix) < 1e-5 * mix and c < 1.0
    assert torch.equal(flat[:1000], before[:1000])
    assert torch.allclose(flat[1000:], before[1000:] * c, rtol=1e-6)


def test_ieee_sqrt_is_correctly_rounded():
    """oracle.ieee.sqrt against the definition of round-to-nearest: the exact
    value lies between the midpoints to the neighbouring floats.  s and ulp/2
    have at most 25 significant bits, so the midpoints and their squares are
    exact in float64 and the check involves no rounding at all."""
    from oracle import ieee
    gen = torch.Generator().manual_seed(5)
    x = torch.cat([torch.rand(200_000, generator=gen) * 1e-6 + 1e-14,
                   torch.rand(100_000, generator=gen) * 4.0,
                   torch.rand(50_000, generator=gen) * 1e30,
                   torch.tensor([1.0, 2.0, 4.0, 0.25, 1e-30, 3.0])])
    x = x[x >= 2.0 ** -100]              # normal results, far from the subnormal range
    s = ieee.sqrt(x)
    assert s.dtype == torch.float32
    nxt = (s.view(torch.int32) + 1).view(torch.float32)
    half_ulp = (nxt.double() - s.double()) / 2
    # going down across a power of two the spacing halves
    prv = (s.view(torch.int32) - 1).view(torch.float32)
    half_ulp_dn = (s.double() - prv.double()) / 2
    lo, hi = s.double() - half_ulp_dn, s.double() + half_ulp
    assert bool(((lo * lo <= x.double()) & (x.double() <= hi * hi)).all())
    assert ieee.sqrt(torch.tensor([0.0, float("inf")])).tolist() == [0.0, float("inf")]
    # and the reason it exists: the tensor library's own routine is not that
    # (informational, never asserted): torch.sqrt may differ from it.


def test_torch_sqrt_deviation_is_bounded(monkeypatch):
    """The oracle's one deliberate departure from a literal torch-CPU run of
    the reference: square roots come from oracle.ieee (correctly rounded), the
    reference calls torch.sqrt (scores.py:216-226, replay.py:695-705), which on
    the CPU is a vector-library routine that may be one ulp off.  This test
    runs every chain that holds a square root both ways on config-1-sized
    inputs (2^22 Student-t gradients, p ~ N(0, 0.02)) and bounds the gap:
    p / w / scores agree within the 1e-6 the parity bar allows (relative to the
    operands of the final subtraction), m and v do not depend on the root at
    all, and the top-k sets by `update` / `coi` differ by a handful of
    threshold neighbours at most."""
    from oracle import ieee
    from tests.util import rel_close, student_t, sub_scale
    n = 1 << 22
    gen = torch.Generator().manual_seed(0)
    p0 = torch.randn(n, generator=gen) * 0.02
    m0 = torch.randn(n, generator=gen) * 1e-4
    v0 = torch.rand(n, generator=gen) * 1e-8
    g = student_t(n, 1)
    b1, b2, eps, wd, lr, step = 0.9, 0.95, 1e-8, 0.1, 1e-4, 3
    bc1, bc2 = 1 - b1 ** step, 1 - b2 ** step
    k = SEL.k_for(n, 1.0)

    def run_all():
        out = {}
        for name in ("update", "coi"):
            out[name] = S.score_formula(name, p0, m0, v0, g, b1, b2, eps, wd, bc1, bc2, "adamw",
                                        update_includes_wd=True)
            out[name + "_sel"] = SEL.select_topk_flat(out[name].abs(), k)[0]
        p, gg, m, v = p0.clone(), g.clone(), m0.clone(), v0.clone()
        A.grad_correct(p, gg, m, v, lr, b1, b2, eps, wd, bc1, bc2, None, "update")
        out.update(gc_p=p, gc_m=m, gc_v=v, gc_score=gg)
        w, m, v = p0.clone(), m0.clone(), v0.clone()
        R.opt_step_inplace(g, m, v, w, None, lr, wd, b1, b2, bc1, bc2, eps)
        out.update(rp_w=w, rp_m=m, rp_v=v)
        return out

    exact = run_all()
    monkeypatch.setattr(ieee, "sqrt", torch.sqrt)
    literal = run_all()
    monkeypatch.undo()
    lanes = int((exact["update"] != literal["update"]).sum())
    for key in ("gc_m", "gc_v", "rp_m", "rp_v"):                 # no square root upstream
        assert torch.equal(exact[key], literal[key]), key
    for key in ("gc_p", "rp_w"):
        bad, worst = rel_close(exact[key], literal[key], rtol=1e-6,
                               scale=sub_scale(p0, exact[key]))
        assert bad == 0, (key, bad, worst)
    for key in ("update", "coi", "gc_score"):
        # one ulp of the root moves U by at most ~2 ulp (one for the root, one for the quotient's
        # rounding): 2^-22 relative to |U|, the larger operand of wd*w + U and of U(g) - U(0)
        bad, worst = rel_close(exact[key], literal[key], rtol=1e-6,
                               scale=exact["update"] - wd * p0)
        assert bad == 0, (key, bad, worst)
    moved = {}
    for name in ("update", "coi"):
        moved[name] = int((exact[name + "_sel"] ^ literal[name + "_sel"]).sum())
        assert moved[name] <= max(16, k // 1000), (name, moved[name], k)
    print(f"torch.sqrt vs correctly rounded sqrt at n=2^22: {lanes} score lanes differ in the "
          f"last bits; top-{k} sets differ by {moved} coordinates (symmetric difference)")


def test_benchmark_score_closed_forms():
    """The two build-side benchmark scores have no reference implementation
    (parity unpinned); their oracle is pinned only by the closed form in
    float64: |q| / sqrt(v + eps) within a few fp32 roundings, and the blind
    score is |g| itself."""
    g = torch.Generator().manual_seed(3)
    q = torch.randn(50_000, generator=g) * 1e-3
    v = torch.rand(50_000, generator=g) * 1e-8
    m = torch.randn(50_000, generator=g) * 1e-4
    for eps in (1e-8, 1e-12):
        got = S.abs_gr_over_sqrt_v(q, v, eps)
        ref = q.double().abs() / (v.double() + eps).sqrt()
        assert got.dtype == torch.float32
        assert torch.allclose(got.double(), ref, rtol=4e-7, atol=0.0)
        ad = S.step_score("abs_gr_over_sqrt_v", None, m, v, q, q, .9, .95, eps, .1, 1., 1., "adams")
        refa = q.double().abs() / ((m * m).double() + eps).sqrt()
        assert torch.allclose(ad.double(), refa, rtol=4e-7, atol=0.0)
    assert torch.equal(S.step_score("abs_g_blind", None, m, v, q + 1.0, q, .9, .95, 1e-8, .1, 1.,
                                    1., "adamw"), q.abs())
