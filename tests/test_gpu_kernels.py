"""GPU parity: pack / scatter / compaction / norms / AdamW commit (masked,
full-step, compact) through the C ABI vs the CPU oracle on the same seeded
inputs.  Everything is bit-exact: integer, index and pure-store results, and
m, v, p and the emitted scores too -- the kernels run the oracle's chain of
separately rounded IEEE-754 fp32 operations, correctly rounded division and
square root included."""
import pytest
import torch

from oracle import adamw as OA
from oracle import kernels as OK
from tests.util import adv, same_bits

pytestmark = pytest.mark.gpu


def _state(n, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g) * 0.02, torch.randn(n, generator=g) * 1e-3,
            torch.rand(n, generator=g) * 1e-6 + 1e-12, torch.randn(n, generator=g) * 1e-3)


@pytest.mark.parametrize("factor", [1.0, 0.125])
@pytest.mark.parametrize("vdtype", [torch.float32, torch.bfloat16])
def test_pack_scatter_bitwise(dev, factor, vdtype):
    from sga_amd import kernels as K
    n = 300_000
    gen = torch.Generator().manual_seed(1)
    grad = torch.randn(n, generator=gen)
    mask = (torch.rand(n, generator=gen) < 0.25)
    idx = torch.nonzero(mask).reshape(-1).to(torch.int32)
    for ix in (idx, idx[:0], idx[:1], idx[:3]):
        g_ref, v_ref = grad.clone(), torch.empty(ix.numel(), dtype=vdtype)
        OK.pack_selected(g_ref, ix, v_ref, factor)
        g_dev, v_dev = grad.to(dev), torch.empty(ix.numel(), dtype=vdtype, device=dev)
        K.pack_selected(g_dev, ix.to(dev), v_dev, factor)
        assert torch.equal(g_dev.cpu(), g_ref)
        assert torch.equal(v_dev.cpu().view(torch.int16 if vdtype == torch.bfloat16 else torch.int32),
                           v_ref.view(torch.int16 if vdtype == torch.bfloat16 else torch.int32))
    dst_ref, dst_dev = torch.zeros(n), torch.zeros(n, device=dev)
    src = torch.randn(idx.numel(), generator=gen)
    OK.scatter_selected(dst_ref, idx, src)
    K.scatter_selected(dst_dev, idx.to(dev), src.to(dev))
    assert torch.equal(dst_dev.cpu(), dst_ref)


def test_pack_adversarial_lanes_bf16(dev):
    from sga_amd import kernels as K
    x = adv(70_000, 3)
    idx = torch.arange(0, 70_000, 3, dtype=torch.int32)
    v_ref = torch.empty(idx.numel(), dtype=torch.bfloat16)
    g_ref = x.clone()
    OK.pack_selected(g_ref, idx, v_ref, 0.5)
    g_dev, v_dev = x.to(dev), torch.empty(idx.numel(), dtype=torch.bfloat16, device=dev)
    K.pack_selected(g_dev, idx.to(dev), v_dev, 0.5)
    assert torch.equal(v_dev.cpu().view(torch.int16), v_ref.view(torch.int16))
    assert torch.equal(g_dev.cpu().view(torch.int32), g_ref.view(torch.int32))


@pytest.mark.parametrize("n,dens", [(0, 0.5), (1, 1.0), (1023, 0.5), (1024, 1.0), (1025, 0.0),
                                    (300_001, 0.4), (5_000_003, 0.01)])
def test_compact_mask_equals_nonzero(dev, n, dens):
    from sga_amd.support import IndexPool, compact_mask_u8
    gen = torch.Generator().manual_seed(n)
    m = (torch.rand(n, generator=gen) < dens).to(torch.uint8)
    ref = OK.compact_mask_u8(m)
    got = compact_mask_u8(m.to(dev))
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), ref)
    pool = IndexPool()
    got2 = compact_mask_u8(m.to(dev), pool)
    assert torch.equal(got2.cpu(), ref)
    if n:
        assert got2.data_ptr() == pool.buf.data_ptr()
    # unaligned view (scalar path)
    if n > 10:
        got3 = compact_mask_u8(m.to(dev)[1:])
        assert torch.equal(got3.cpu(), OK.compact_mask_u8(m[1:]))


def test_norms(dev):
    from sga_amd import kernels as K
    gen = torch.Generator().manual_seed(5)
    for n in (1, 777, 300_000, 2_000_001):
        v = torch.randn(n, generator=gen)
        mask = (torch.rand(n, generator=gen) < 0.3).to(torch.uint8)
        t_ref, t_dev = torch.tensor(1.5), torch.tensor(1.5, device=dev)
        OK.compact_norm_sq_contribution(v, t_ref)
        K.compact_norm_sq_contribution(v.to(dev), t_dev)
        assert abs(t_dev.item() - t_ref.item()) <= 1e-5 * abs(t_ref.item())
        t2 = torch.tensor(1.5, device=dev)
        K.compact_norm_sq_contribution(v.to(dev), t2)
        assert t2.item() == t_dev.item()                      # rerun bitwise
        m_ref, m_dev = torch.zeros(()), torch.zeros((), device=dev)
        OK.masked_norm_sq_contribution(v, mask, m_ref)
        K.masked_norm_sq_contribution(v.to(dev), mask.to(dev), m_dev)
        assert abs(m_dev.item() - m_ref.item()) <= 1e-4 * abs(m_ref.item()) + 1e-12


def test_block_gather_scatter(dev):
    from sga_amd import kernels as K
    gen = torch.Generator().manual_seed(6)
    n, x = 10_007, 8
    grad = torch.randn(n, generator=gen)
    mask = (torch.rand(n, generator=gen) < 0.5).to(torch.uint8)
    bidx = torch.arange(0, n, 40, dtype=torch.int32)
    bidx[-1] = n - 3                                    # tail block reads short
    for factor in (1.0, 0.25):
        v_ref = torch.full((bidx.numel() * x,), 7.0)
        OK.gather_selected_blocks(grad, mask, bidx, v_ref, x, factor)
        v_dev = torch.full((bidx.numel() * x,), 7.0, device=dev)
        K.gather_selected_blocks(grad.to(dev), mask.to(dev), bidx.to(dev), v_dev, x, factor)
        assert torch.equal(v_dev.cpu(), v_ref)
    d_ref, d_dev = torch.zeros(n), torch.zeros(n, device=dev)
    OK.scatter_selected_blocks(d_ref, mask, bidx, v_ref, x)
    K.scatter_selected_blocks(d_dev, mask.to(dev), bidx.to(dev), v_ref.to(dev), x)
    assert torch.equal(d_dev.cpu(), d_ref)
    with pytest.raises(AssertionError, match="k_blocks\\*x"):
        K.gather_selected_blocks(grad.to(dev), mask.to(dev), bidx.to(dev), v_dev[:5], x, 1.0)


def _run_gc(dev, n, seed, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8, wd=0.1, step=5, off=0, **kw):
    from sga_amd import adamw as A
    p, m, v, g = _state(n + off, seed)
    mask = kw.pop("mask", None)
    ref = [t[off:].clone() for t in (p, g, m, v)]
    OA.adamw_grad_correct(*ref, lr, b1, b2, eps, wd, step, mask=mask, **kw)
    devt = [t.to(dev)[off:] for t in (p, g, m, v)]
    A.adamw_grad_correct(*devt, lr, b1, b2, eps, wd, step,
                         mask=None if mask is None else mask.to(dev), **kw)
    return ref, [t.cpu() for t in devt] + [p[off:]]


@pytest.mark.parametrize("off", [0, 1])
def test_grad_correct_sparse_and_knobs(dev, off):
    n = 200_003
    mask = (torch.rand(n, generator=torch.Generator().manual_seed(2)) < 0.3).to(torch.uint8)
    for kw in (dict(), dict(mask=mask), dict(mask=mask, coeff=0.37, clear=True),
               dict(mask=mask, clear=True, fold=True, interval=4.0),
               dict(mask=mask, coeff=0.37, clear=True, fold=True, interval=3.0),
               dict(mask=torch.zeros(n, dtype=torch.uint8), clear=True)):
        (rp, rg, rm, rv), (dp, dg, dm, dv, p0) = _run_gc(dev, n, 7, off=off, **dict(kw))
        assert torch.equal(dm, rm) and torch.equal(dv, rv), kw
        assert torch.equal(dg, rg), kw
        assert same_bits(dp, rp), kw


@pytest.mark.parametrize("score", ["update", "abs_g", "abs_m", "coi"])
def test_grad_correct_full_step_scores(dev, score):
    n = 150_001
    (rp, rg, rm, rv), (dp, dg, dm, dv, p0) = _run_gc(dev, n, 9, emit_score=score)
    assert torch.equal(dm, rm) and torch.equal(dv, rv)
    assert same_bits(dg, rg)            # the emitted score, division and square root included
    assert same_bits(dp, rp)
    # dual-lr split: m/v/score mask-blind, p == w - where(mask, lr, lr*s)*update
    if score == "update":
        mask = (torch.rand(n, generator=torch.Generator().manual_seed(3)) < 0.5).to(torch.uint8)
        (sp, sg, sm, sv), (ep, eg, em, ev, _) = _run_gc(dev, n, 9, emit_score=score, mask=mask,
                                                     inactive_lr_scale=0.25)
        assert torch.equal(em, dm) and torch.equal(ev, dv) and torch.equal(eg, dg)
        p0 = _state(n, 9)[0]
        assert torch.equal(ep, p0 - torch.where(mask > 0, 1e-3, 1e-3 * 0.25) * eg)
        (_, _, _, _), (zp, _, _, _, _) = _run_gc(dev, n, 9, emit_score=score, mask=mask,
                                              inactive_lr_scale=0.0)
        assert torch.equal(zp[mask == 0], p0[mask == 0])


def test_grad_correct_adversarial_lanes(dev):
    from sga_amd import adamw as A
    n = 65_536
    p, g, m = adv(n, 1), adv(n, 2), adv(n, 3)
    v = adv(n, 4, nonneg=True)
    p, g, m, v = (t.clamp(-1e18, 1e18) for t in (p, g, m, v))
    ref = [t.clone() for t in (p, g, m, v)]
    OA.adamw_grad_correct(*ref, 1e-3, 0.9, 0.999, 1e-8, 0.01, 7)
    devt = [t.to(dev) for t in (p, g, m, v)]
    A.adamw_grad_correct(*devt, 1e-3, 0.9, 0.999, 1e-8, 0.01, 7)
    assert torch.equal(devt[2].cpu().view(torch.int32), ref[2].view(torch.int32))
    assert torch.equal(devt[3].cpu().view(torch.int32), ref[3].view(torch.int32))
    ok = torch.isfinite(ref[0])
    dp = devt[0].cpu()
    assert same_bits(dp[ok], ref[0][ok])
    assert torch.equal(torch.isnan(dp), torch.isnan(ref[0])) and torch.equal(torch.isinf(dp), torch.isinf(ref[0]))


@pytest.mark.parametrize("rec_start,n,dens,use_table", [
    (0, 4096, 0.05, False), (1, 5000, 0.05, True), (500, 1023, 1.0, True),
    (1000, 1024, 1.0, False), (1500, 1025, 1.0, True), (1023, 70_001, 0.3, True),
    (0, 300_000, 0.0, True), (777, 200_000, 0.01, False)])
@pytest.mark.parametrize("vdtype", [torch.float32, torch.bfloat16])
def test_compact_commit_matches_oracle(dev, rec_start, n, dens, use_table, vdtype):
    from sga_amd import adamw as A
    n_bucket = rec_start + n + 3000
    gen = torch.Generator().manual_seed(rec_start + n)
    buf = torch.randn(n_bucket, generator=gen) * 1e-3
    mask = (torch.rand(n_bucket, generator=gen) < dens).to(torch.uint8)
    idx = OK.compact_mask_u8(mask)
    vals = torch.empty(idx.numel(), dtype=vdtype)
    OK.pack_selected(buf, idx, vals, 1.0)
    p, m, v, _ = _state(n, 11)
    for kw in (dict(), dict(coeff=0.5), dict(fold=True, interval=4.0)):
        rb, rp, rm, rv = buf.clone(), p.clone(), m.clone(), v.clone()
        OA.adamw_grad_correct_compact(rp, rb[rec_start:rec_start + n], rm, rv, idx, vals,
                                      rec_start, 1e-3, 0.9, 0.95, 1e-8, 0.1, 4, **kw)
        db, dp, dm, dv = (t.to(dev) for t in (buf, p, m, v))
        table = A.build_dir_table(idx.to(dev), n_bucket) if use_table else None
        if use_table:
            assert torch.equal(table.cpu(), OA.build_dir_table(idx, n_bucket))
        A.adamw_grad_correct_compact(dp, db[rec_start:rec_start + n], dm, dv, idx.to(dev),
                                     vals.to(dev), rec_start, 1e-3, 0.9, 0.95, 1e-8, 0.1, 4,
                                     dir_table=table, **kw)
        assert torch.equal(dm.cpu(), rm) and torch.equal(dv.cpu(), rv), kw
        assert torch.equal(db.cpu(), rb), kw
        assert same_bits(dp, rp), kw


def test_dir_table_geometries(dev):
    from sga_amd import adamw as A
    gen = torch.Generator().manual_seed(4)
    n = 300_000
    masks = [torch.zeros(n, dtype=torch.uint8), torch.ones(n, dtype=torch.uint8),
             (torch.rand(n, generator=gen) < 0.05).to(torch.uint8)]
    short = torch.zeros(n, dtype=torch.uint8)
    short[:777] = 1
    runs = torch.zeros(n, dtype=torch.uint8)
    runs.view(-1, 100)[::7] = 1
    for m in masks + [short, runs]:
        idx = OK.compact_mask_u8(m)
        t = A.build_dir_table(idx.to(dev), n)
        assert t.dtype == torch.int32 and t.numel() == (n >> 10) + 2
        assert torch.equal(t.cpu(), OA.build_dir_table(idx, n))


@pytest.mark.parametrize("kw", [dict(), dict(mask=True), dict(mask=True, coeff=0.5, clear=True, fold=True, interval=4.0),
                                dict(emit_score="update"), dict(emit_score="coi"), dict(emit_score="abs_m"),
                                dict(mask=True, emit_score="abs_g", inactive_lr_scale=0.5)])
def test_adams_grad_correct(dev, kw):
    from sga_amd import adams as AS
    n = 90_001
    p, m, v, g = _state(n, 31)
    kw = dict(kw)
    mask = None
    if kw.pop("mask", False):
        mask = (torch.rand(n, generator=torch.Generator().manual_seed(2)) < 0.3).to(torch.uint8)
    ref = [t.clone() for t in (p, g, m, v)]
    OA.adams_grad_correct(*ref, 1e-3, 0.9, 0.95, 1e-8, 0.1, mask=mask, **kw)
    devt = [t.to(dev) for t in (p, g, m, v)]
    AS.adams_grad_correct(*devt, 1e-3, 0.9, 0.95, 1e-8, 0.1,
                          mask=None if mask is None else mask.to(dev), **kw)
    assert torch.equal(devt[2].cpu(), ref[2]) and torch.equal(devt[3].cpu(), ref[3])
    assert same_bits(devt[1], ref[1])          # cleared / folded gradient or the emitted score
    assert same_bits(devt[0], ref[0])


def test_adams_compact_equals_masked(dev):
    from sga_amd import adams as AS
    from sga_amd.adamw import build_dir_table
    from sga_amd.kernels import pack_selected
    from sga_amd.support import compact_mask_u8
    n = 70_001
    p, m, v, g = _state(n, 41)
    mask = (torch.rand(n, generator=torch.Generator().manual_seed(4)) < 0.2).to(torch.uint8)
    a = [t.to(dev) for t in (p, g, m, v)]
    AS.adams_grad_correct(*a, 1e-3, 0.9, 0.95, 1e-8, 0.1, mask=mask.to(dev), coeff=0.5, clear=True)
    b = [t.to(dev) for t in (p, g, m, v)]
    idx = compact_mask_u8(mask.to(dev))
    vals = torch.empty(idx.numel(), device=dev)
    pack_selected(b[1], idx, vals, 1.0)
    AS.adams_grad_correct_compact(b[0], b[1], b[2], b[3], idx, vals, 0, 1e-3, 0.9, 0.95, 1e-8, 0.1,
                                  coeff=0.5, dir_table=build_dir_table(idx, n))
    for x, y in zip(a, b):
        assert torch.equal(x, y)


@pytest.mark.parametrize("mode", ["sparse", "full_update", "full_split", "adams_sparse"])
def test_grad_correct_multi_equals_per_record_calls(dev, mode):
    """One launch over a ragged list of records == the per-record kernel calls,
    bit for bit, with per-record knobs (a record without a mask takes none)."""
    from sga_amd.adamw import adamw_grad_correct, adamw_grad_correct_multi
    gen = torch.Generator().manual_seed(17)
    sizes = [5, 4096, 4097, 12_289, 1, 100_003, 8192]
    adams = mode == "adams_sparse"
    recs_a, recs_b = [], []
    for j, n in enumerate(sizes):
        t = {k: (torch.randn(n + 1, generator=gen) * s).to(dev)[1 if j % 3 == 0 else 0:][:n]
             for k, s in (("p", 0.02), ("g", 1e-2), ("m", 1e-3))}
        t["v"] = (torch.rand(n + 1, generator=gen) * 1e-5).to(dev)[:n]
        mask = None if j == 4 else (torch.rand(n, generator=gen) < 0.3).to(torch.uint8).to(dev)
        hp = dict(lr=1e-3 * (1 + j), beta1=0.9, beta2=0.95 if j % 2 else 0.999, eps=1e-8,
                  weight_decay=0.1 if j % 2 else 0.0, step=3 + j)
        recs_a.append((dict((k, v.clone()) for k, v in t.items()), mask, hp))
        recs_b.append((dict((k, v.clone()) for k, v in t.items()), mask, hp))
    if mode in ("sparse", "adams_sparse"):
        emit, kn = None, dict(coeff=0.37, clear=True, fold=True, interval=4.0)
    elif mode == "full_update":
        emit, kn = "update", {}
    else:
        emit, kn = "abs_g", dict(inactive_lr_scale=0.25)
    table = []
    for t, mask, hp in recs_a:                    # reference: one call per record
        use = mask if mode != "full_update" else None
        kw = dict(kn) if use is not None else {}
        if use is None:
            kw.pop("inactive_lr_scale", None)
        adamw_grad_correct(t["p"], t["g"], t["m"], t["v"], hp["lr"], hp["beta1"], hp["beta2"],
                           hp["eps"], hp["weight_decay"], 1 if adams else hp["step"], mask=use,
                           emit_score=emit, _adams=adams, **kw)
    for t, mask, hp in recs_b:
        use = mask if mode != "full_update" else None
        table.append(dict(p=t["p"], g=t["g"], m=t["m"], v=t["v"], mask=use,
                          coeff_on=use is not None, clear=kn.get("clear", False) and use is not None,
                          fold=kn.get("fold", False) and use is not None,
                          inactive_lr_scale=kn.get("inactive_lr_scale", 1.0) if use is not None
                          else 1.0, **hp))
    adamw_grad_correct_multi(table, emit_score=emit, coeff=kn.get("coeff", 1.0),
                             interval=kn.get("interval", 1.0), _adams=adams)
    for (ta, _, _), (tb, _, _) in zip(recs_a, recs_b):
        for k in ("p", "g", "m", "v"):
            assert torch.equal(ta[k].view(torch.int32), tb[k].view(torch.int32)), (mode, k)
    with pytest.raises(ValueError, match="requires a sparse step"):
        adamw_grad_correct_multi([dict(table[0], mask=None, clear=True)], emit_score=None)


@pytest.mark.parametrize("vdtype,adams", [(torch.float32, False), (torch.bfloat16, False),
                                          (torch.float32, True)])
def test_grad_correct_compact_multi_equals_per_record_calls(dev, vdtype, adams):
    """One merge-join launch over every record of a bucket == the per-record
    compact calls, bit for bit (with and without the directory table)."""
    from sga_amd.adamw import (adamw_grad_correct_compact, adamw_grad_correct_compact_multi,
                               build_dir_table)
    gen = torch.Generator().manual_seed(23)
    sizes = [1500, 4096, 5, 70_001, 8193, 1023]
    n_total = sum(sizes)
    mask = torch.rand(n_total, generator=gen) < 0.07
    idx = mask.nonzero().reshape(-1).to(torch.int32).to(dev)
    values = (torch.randn(idx.numel(), generator=gen) * 1e-2).to(vdtype).to(dev)
    table = build_dir_table(idx, n_total)
    for use_table in (True, False):
        sets = []
        for _ in range(2):
            g2 = torch.Generator().manual_seed(5)
            recs, off = [], 0
            for j, n in enumerate(sizes):
                recs.append(dict(
                    p=(torch.randn(n, generator=g2) * 0.02).to(dev),
                    g=(torch.randn(n, generator=g2) * 1e-2).to(dev),
                    m=(torch.randn(n, generator=g2) * 1e-3).to(dev),
                    v=(torch.rand(n, generator=g2) * 1e-5).to(dev),
                    rec_start=off, lr=1e-3 * (j + 1), beta1=0.9, beta2=0.95, eps=1e-8,
                    weight_decay=0.1 if j % 2 else 0.0, step=4 + j))
                off += n
            sets.append(recs)
        tb = table if use_table else None
        for r in sets[0]:
            adamw_grad_correct_compact(r["p"], r["g"], r["m"], r["v"], idx, values, r["rec_start"],
                                       r["lr"], r["beta1"], r["beta2"], r["eps"],
                                       r["weight_decay"], 1 if adams else r["step"], coeff=0.6,
                                       fold=True, interval=8.0, dir_table=tb, _adams=adams)
        adamw_grad_correct_compact_multi(
            [dict(r, idx=idx, values=values, dir_table=tb) for r in sets[1]], coeff=0.6,
            fold=True, interval=8.0, _adams=adams)
        for a, b in zip(*sets):
            for k in ("p", "g", "m", "v"):
                assert torch.equal(a[k].view(torch.int32), b[k].view(torch.int32)), (use_table, k)
