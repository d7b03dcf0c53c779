"""GPU parity of the replay kernels: score formulas, in-place AdamW/AdamS
commit (dual-lr, label accumulation) and the fused group step vs the CPU
oracle.  Masks, thresholds, scores, m, v, w and the labels are bit-exact (the
same chain of correctly rounded operations, FMAs where the reference's in-place
ops have one); clip norms are double sums whose order differs: the
reference's 1e-6 reordering band."""
import pytest
import torch

from oracle import replay as OR
from oracle import scores as OS
from oracle import select as SEL
from tests.util import adv, same_bits, student_t

pytestmark = pytest.mark.gpu


def _state(n, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g) * 0.02, torch.randn(n, generator=g) * 1e-3,
            torch.rand(n, generator=g) * 1e-6 + 1e-12, torch.randn(n, generator=g) * 1e-3)


@pytest.mark.parametrize("opt", ["adamw", "adams"])
@pytest.mark.parametrize("name", ["update", "abs_g", "abs_m", "coi"])
def test_score_formulas(dev, name, opt):
    from sga_amd import replay_kernels as K
    from sga_amd.replay import score_formula
    from sga_amd.scores import get_score_spec
    b1, b2, eps, wd, step = 0.9, 0.95, 1e-8, 1e-2, 7
    bc1, bc2 = 1 - b1 ** step, 1 - b2 ** step
    w, m, v, g = _state(100_003, 3)
    ref = OS.score_formula(name, w, m, v, g, b1, b2, eps, wd, bc1, bc2, opt,
                           update_includes_wd=True)
    got = score_formula(name, *(t.to(dev) for t in (w, m, v, g)), b1, b2, eps, wd, bc1, bc2,
                        opt, update_includes_wd=True).cpu()
    assert same_bits(got, ref)
    if opt == "adamw":
        spec = get_score_spec(name).formula(*(t.to(dev) for t in (w, m, v, g)), b1, b2, eps, wd,
                                            bc1, bc2)
        assert torch.equal(spec.cpu(), got)
        assert torch.equal(K.formula(name)(*(t.to(dev) for t in (w, m, v, g)), b1, b2, eps, wd,
                                           bc1, bc2).cpu(), got)


@pytest.mark.parametrize("opt", ["adamw", "adams"])
def test_update_without_weight_decay_term(dev, opt):
    """update_includes_wd=False returns U(g) itself (scores.py:227-230), not
    0*w + U(g): lanes whose w is Inf / NaN or whose U is -0 keep U's bits."""
    from sga_amd.replay import score_formula
    b1, b2, eps, wd, step = 0.9, 0.95, 1e-8, 1e-2, 7
    bc1, bc2 = 1 - b1 ** step, 1 - b2 ** step
    w, m, v, g = _state(10_007, 5)
    w[:4] = torch.tensor([float("inf"), float("-inf"), float("nan"), -1.0])
    m[4:8] = torch.tensor([-0.0, 0.0, -0.0, 0.0])
    g[4:8] = torch.tensor([-0.0, -0.0, 0.0, 0.0])              # U = -0 / +0 lanes
    ref = OS.score_formula("update", w, m, v, g, b1, b2, eps, wd, bc1, bc2, opt,
                           update_includes_wd=False)
    got = score_formula("update", *(t.to(dev) for t in (w, m, v, g)), b1, b2, eps, wd, bc1, bc2,
                        opt, update_includes_wd=False)
    assert bool(torch.isfinite(ref[:4]).all()) and same_bits(got, ref)


@pytest.mark.parametrize("opt", ["adamw", "adams"])
@pytest.mark.parametrize("lr,wd,count", [(1e-3, .01, 7), (3e-4, .01, 1), (1e-3, 0.0, 100)])
def test_opt_step_inplace(dev, opt, lr, wd, count):
    from sga_amd import replay_kernels as K
    from sga_amd.replay import _opt_step_inplace
    b1, b2, eps = 0.9, 0.999, 1e-8
    n = 70_001
    for adversarial in (False, True):
        if adversarial:
            q, m, w = (adv(n, s).clamp(-1e15, 1e15) for s in (1, 2, 3))
            v = adv(n, 4, nonneg=True).clamp(0, 1e30)
        else:
            w, m, v, q = _state(n, count)
        bc1, bc2 = OR.bc_pair(opt, count, b1, b2)
        inactive = torch.rand(n, generator=torch.Generator().manual_seed(3)) < 0.5
        for ina, lri, with_lab in ((None, None, True), (inactive, lr * 0.3, False)):
            rm, rv, rw = m.clone(), v.clone(), w.clone()
            rlab = torch.zeros(n) if with_lab else None
            OR.opt_step_inplace(q, rm, rv, rw, rlab, lr, wd, b1, b2, bc1, bc2, eps,
                                optimizer=opt, inactive=ina, lr_inactive=lri)
            dm, dv, dw = (t.to(dev) for t in (m, v, w))
            dlab = torch.zeros(n, device=dev) if with_lab else None
            _opt_step_inplace(q.to(dev), dm, dv, dw, dlab, lr, wd, b1, b2, bc1, bc2, eps,
                              optimizer=opt, inactive=None if ina is None else ina.to(dev),
                              lr_inactive=lri)
            assert torch.equal(dm.cpu().view(torch.int32), rm.view(torch.int32))
            assert torch.equal(dv.cpu().view(torch.int32), rv.view(torch.int32))
            ok = torch.isfinite(rw)
            assert same_bits(dw.cpu()[ok], rw[ok]), adversarial
            assert torch.equal(torch.isfinite(dw.cpu()), ok)
            if with_lab and not adversarial:
                assert same_bits(dlab, rlab)
    with pytest.raises(ValueError, match="come as a pair"):
        K.opt_step_inplace(q.to(dev), dm, dv, dw, None, lr, wd, b1, b2, bc1, bc2, eps,
                           inactive=inactive.to(dev))


_RAGGED = [600_000, 130, 37, 500_000, 3, 1024, 100_001, 5, 250]   # > 2^20: the one-sweep select


def _fixture(n_sizes, W, seed=2026, bf16=False, vary=False):
    n = sum(n_sizes)
    gen = torch.Generator().manual_seed(seed)
    w0 = torch.randn(n, generator=gen) * 0.02
    m0 = torch.randn(n, generator=gen) * 1e-3
    v0 = torch.rand(n, generator=gen) * 1e-6
    grads = []
    for s in range(W):
        g = student_t(n, seed + s, scale=1e-2 * (1 + 0.05 * s))
        if s in (2, 3):
            g[n_sizes[0]:n_sizes[0] + n_sizes[1]] = 0.0      # a param absent from the payload
        grads.append(g.to(torch.bfloat16) if bf16 else g)
    entries, off = [], 0
    for i, s in enumerate(n_sizes):
        entries.append({"a": off, "n": s, "b1": 0.9, "b2": 0.95, "eps": 1e-8,
                        "wd": 0.1 if i % 2 == 0 else 0.0})
        if vary:     # every hyper-parameter changes from tensor to tensor
            entries[-1].update(b1=(0.9, 0.8, 0.95)[i % 3], b2=(0.95, 0.99)[i % 2],
                               eps=(1e-8, 1e-6, 1e-10)[(i + 1) % 3])
        off += s
    return n, w0, m0, v0, grads, entries


def _run_group(dev, cfg_specs, clip, W=9, bf16=False, t0=10, sizes=(400_000, 300_000, 170_000),
               semantics="topk", p_offs=None):
    from sga_amd.replay_group import Config, ReplayGroup
    n, w0, m0, v0, grads, entries = _fixture(list(sizes), W, bf16=bf16)
    if p_offs is not None:
        for e, po in zip(entries, p_offs):
            e["p_off"] = po
    lr = 5e-5
    norms = [float(g.float().norm()) * 1.3 for g in grads]
    metas = [{"clip_grad": clip, "grad_norm": norms[i], "lr": lr} for i in range(W)]
    ocfg = [OR.Config(*c) for c in cfg_specs]
    dcfg = [Config(*c) for c in cfg_specs]
    sel0 = []
    for c in ocfg:
        g0 = grads[0].float()
        sc = OS.step_score(c.score, w0, m0, v0, g0, g0, 0.9, 0.95, 1e-8, 0.1,
                           *OR.bc_pair(c.optimizer, t0 + 1, 0.9, 0.95), c.optimizer)
        if semantics == "topk":
            sel0.append(SEL.select_topk_flat(sc, SEL.replay_k(n, c.ratio))[0])
        else:
            sel0.append(SEL.shard_select_balanced(sc, SEL.replay_k(n, c.ratio), entries)[0])
    grp = ReplayGroup(entries, w0.to(dev), m0.to(dev), v0.to(dev), [s.to(dev) for s in sel0],
                      dcfg, t0, W, selection_semantics=semantics)
    dev_coefs, dev_qn2 = {}, {}
    for si in range(W):
        grp.step(grads[si].to(dev), metas[si])
        cf, q2 = grp.coef_d.cpu().tolist(), grp.qn2.cpu().tolist()
        for ci in range(len(dcfg)):
            dev_coefs[(si, ci)], dev_qn2[(si, ci)] = cf[ci], q2[ci]
    trace = []
    out = OR.group_replay(entries, w0, m0, v0, sel0, ocfg, grads, metas, t0,
                          coef_hook=lambda si, ci, c: dev_coefs[(si, ci)], trace=trace,
                          selection_semantics=semantics)
    for si, ci, qn2, coef in trace:             # clip norms: 1e-6 reordering band
        assert abs(dev_qn2[(si, ci)] - qn2) <= 1e-6 * max(qn2, 1e-30), (si, ci)
        assert abs(dev_coefs[(si, ci)] - coef) <= 1e-6 * coef, (si, ci)
    return grp, out, w0


def test_group_step_no_clip_bitwise(dev):
    specs = [("abs_g", 1.0, 1), ("abs_g", 10.0, 4), ("abs_m", 1.0, 4), ("abs_g", 0.1, 3, "adams"),
             ("abs_g", 1.0, 4, "adamw", True), ("abs_g", 1.0, 4, "adamw", False, 0.25),
             ("abs_g", 1.0, 16)]
    grp, out, w0 = _run_group(dev, specs, clip=0.0, bf16=True)
    for ci, o in enumerate(out):
        s = grp.state[ci]
        assert torch.equal(s["sel"].cpu().bool(), o["sel"]), ci
        assert torch.equal(s["res"].cpu().view(torch.int32), o["res"].view(torch.int32)), ci
        assert torch.equal(s["m"].cpu(), o["m"]) and torch.equal(s["v"].cpu(), o["v"]), ci
        assert same_bits(s["w"], o["w"]), ci
    assert float(grp.state[0]["res"].abs().max()) == 0.0       # T = 1: no residual survives


def test_group_step_one_sweep_select(dev):
    """More than 2^20 elements over ragged tensors: every boundary
    re-selection of the group runs the one-sweep select and the commits go
    through chunks that straddle tensors."""
    specs = [("abs_g", 1.0, 1), ("abs_g", 10.0, 2), ("abs_m", 1.0, 2), ("abs_g", 0.1, 3, "adams")]
    grp, out, w0 = _run_group(dev, specs, clip=0.0, W=5, bf16=True, sizes=_RAGGED)
    assert grp.last_select().path == 1
    for ci, o in enumerate(out):
        s = grp.state[ci]
        assert torch.equal(s["sel"].cpu().bool(), o["sel"]), ci
        assert torch.equal(s["res"].cpu().view(torch.int32), o["res"].view(torch.int32)), ci
        assert torch.equal(s["m"].cpu(), o["m"]) and torch.equal(s["v"].cpu(), o["v"]), ci
        assert same_bits(s["w"], o["w"]), ci


def test_group_step_with_clip(dev):
    specs = [("abs_g", 1.0, 1), ("abs_g", 10.0, 4), ("abs_g", 1.0, 4, "adams", True),
             ("abs_m", 0.1, 3, "adamw", False, 2.0)]
    grp, out, w0 = _run_group(dev, specs, clip=0.3, bf16=False)
    for ci, o in enumerate(out):
        s = grp.state[ci]
        assert torch.equal(s["sel"].cpu().bool(), o["sel"]), ci
        assert torch.equal(s["res"].cpu().view(torch.int32), o["res"].view(torch.int32)), ci
        assert torch.equal(s["m"].cpu(), o["m"]) and torch.equal(s["v"].cpu(), o["v"]), ci
        assert same_bits(s["w"], o["w"]), ci


@pytest.mark.parametrize("sizes,vary,path", [([300_000, 1024, 200_000], False, 0),
                                             (_RAGGED, True, 1)])
@pytest.mark.parametrize("score", ["update", "coi"])
def test_reselect_adam_scores(dev, score, sizes, vary, path):
    """Adam-normalised scores: the boundary re-selection equals the oracle
    selector on the oracle's own scores (division and square root included,
    the device runs the same correctly rounded chain).  The ragged set runs the
    one-sweep select, whose slabs hold several unaligned tensor boundaries with
    different hyper-parameters on either side."""
    from sga_amd.replay_group import Config, ReplayGroup
    n, w0, m0, v0, grads, entries = _fixture(sizes, 3, vary=vary)
    t0, lr = 5, 1e-4
    cfg = Config(score, 1.0, 1)
    k = SEL.replay_k(n, 1.0)
    sel0 = torch.zeros(n, dtype=torch.bool)
    grp = ReplayGroup(entries, w0.to(dev), m0.to(dev), v0.to(dev), [sel0.to(dev)], [cfg], t0, 3)
    grp.step(grads[0].to(dev), {"clip_grad": 0.0, "lr": lr})
    s = grp.state[0]
    w1, m1, v1 = (s[x].cpu().clone() for x in ("w", "m", "v"))
    grp.step(grads[1].to(dev), {"clip_grad": 0.0, "lr": lr})     # si = 1: reselects
    count = t0 + 2
    sc = torch.empty(n)
    q = grads[1]                                                   # res == 0 at T = 1, coef == 1
    for e in entries:
        a, b = e["a"], e["a"] + e["n"]
        sc[a:b] = OS.score_formula(score, w1[a:b], m1[a:b], v1[a:b], q[a:b], e["b1"], e["b2"],
                                   e["eps"], e["wd"], 1 - e["b1"] ** count, 1 - e["b2"] ** count,
                                   "adamw", update_includes_wd=True).abs()
    ref, th = SEL.select_topk_flat(sc, k)
    assert torch.equal(s["sel"].cpu().bool(), ref)
    assert grp.last_select().thresh == th
    assert grp.last_select().path == path


def _assert_group_equal(grp, out, specs):
    for ci, o in enumerate(out):
        s = grp.state[ci]
        assert torch.equal(s["sel"].cpu().bool(), o["sel"]), (ci, specs[ci])
        assert same_bits(s["res"], o["res"]) and same_bits(s["m"], o["m"]), (ci, specs[ci])
        assert same_bits(s["v"], o["v"]) and same_bits(s["w"], o["w"]), (ci, specs[ci])


@pytest.mark.parametrize("opt", ["adamw", "adams"])
@pytest.mark.parametrize("clip", [0.0, 0.3])
def test_group_adam_scores_live_residual(dev, opt, clip):
    """Boundary re-selection by the Adam-normalised scores with a LIVE residual
    (T > 1), a clip coefficient below one, a dense-run coefficient below one
    (the recorded norm is finite), fold and dual-lr arms, under AdamW and AdamS
    (v := m*m, bc := 1: replay.py:486-505): score = |formula(w, m, v,
    (g / coef_dense + res) * coef)| as replay_fused.py:1752-1825 forms it.  The
    oracle selects on its own scores; masks and state must agree bit for bit."""
    specs = [("update", 1.0, 2, opt), ("coi", 10.0, 4, opt), ("update", 0.1, 4, opt, True),
             ("coi", 1.0, 2, opt, False, 0.25), ("update", 10.0, 3, opt, True, 2.0),
             ("coi", 0.1, 3, opt)]
    grp, out, w0 = _run_group(dev, specs, clip=clip, W=9, bf16=True)
    assert float(grp.state[5]["res"].abs().max()) > 0.0          # T = 3 ends two steps past a boundary
    _assert_group_equal(grp, out, specs)


@pytest.mark.parametrize("opt", ["adamw", "adams"])
def test_group_adam_scores_one_sweep_long_cycle(dev, opt):
    """The same cell above 2^20 elements on ragged tensors (one-sweep select,
    slabs that straddle tensors) with a T = 16 arm that re-selects at si = 16
    after 15 masked steps of residual accumulation, f32 gradients, clip on."""
    specs = [("update", 1.0, 16, opt), ("coi", 1.0, 4, opt), ("update", 0.1, 2, opt, True, 0.25)]
    grp, out, w0 = _run_group(dev, specs, clip=0.3, W=18, bf16=False, sizes=_RAGGED)
    assert grp.last_select().path == 1
    _assert_group_equal(grp, out, specs)


@pytest.mark.parametrize("sizes,p_offs", [((400_000, 300_000, 170_000), None),
                                          (tuple(_RAGGED), [3, 0, 13, 8005, 1, 0, 6, 2, 7])])
def test_group_step_balanced_histogram_semantics(dev, sizes, p_offs):
    """The group step under the `balanced-histogram` selection semantics
    (replay_fused.py:1340-1344, 1805-1809): every boundary re-selects with the
    online engine's approximate tier -- stride-8 subsample on each tensor's
    own grid (non-zero param-relative phases in the ragged case), integer
    crossing bin, the whole bin selected -- on scores formed on the fly.  All
    registry scores, AdamS, fold and dual-lr arms, a live residual, clipping;
    masks and state bit for bit against the oracle's loop under the same
    semantics, and the masks differ from the exact top-k's."""
    specs = [("abs_g", 1.0, 2), ("update", 10.0, 4), ("coi", 1.0, 3, "adams"),
             ("abs_m", 1.0, 2), ("update", 0.1, 2, "adamw", True, 0.25),
             ("abs_g_blind", 1.0, 4), ("abs_g", 10.0, 3, "adams", True)]
    grp, out, w0 = _run_group(dev, specs, clip=0.3, W=9, bf16=True, sizes=sizes,
                              semantics="balanced-histogram", p_offs=p_offs)
    _assert_group_equal(grp, out, specs)
    res = grp.last_select()
    assert res.path == 3 and res.status == 0 and res.nonfinite == 0
    assert res.thresh_bits & 0xFFFF == 0                       # a bin's lower edge
    n = sum(sizes)
    for ci, c in enumerate(specs):
        cnt = int(out[ci]["sel"].sum())
        assert abs(cnt - SEL.replay_k(n, c[1])) < 0.005 * n + 64, (ci, cnt)
    assert int(out[0]["sel"].sum()) != SEL.replay_k(n, 1.0)     # approximate by construction


def test_shard_select_balanced_twin_with_param_phases(dev):
    """`sga_amd.replay_fused.shard_select_balanced` (one histogram call per
    entry, param-relative phase) against the oracle's twin on the geometry
    fixture of tests/test_selection_semantics_switch.py:176-186 with shard
    slices that start inside their parameters (p_off != 0)."""
    from sga_amd.replay_fused import shard_select_balanced
    sizes, p_offs = [40001, 7, 65536, 100009], [3, 13, 0, 8005]
    gen = torch.Generator().manual_seed(7)
    score = torch.rand(sum(sizes), generator=gen) ** 4
    ent, off = [], 0
    for sz, po in zip(sizes, p_offs):
        ent.append({"a": off, "n": sz, "p_off": po})
        off += sz
    score[ent[2]["a"]:ent[2]["a"] + sizes[2]] = 0.25
    n = score.numel()
    for k in (1, n // 100, 3 * n // 10, n - 1, n):
        ref_mask, ref_th = SEL.shard_select_balanced(score, k, ent)
        mask, th = shard_select_balanced(score.to(dev), k, None, ent)
        assert th == ref_th and torch.equal(mask.cpu(), ref_mask), k
    # whole views (no p_off key) are phase 0
    plain = [{"a": e["a"], "n": e["n"]} for e in ent]
    ref_mask, ref_th = SEL.shard_select_balanced(score, n // 100, plain)
    mask, th = shard_select_balanced(score.to(dev), n // 100, None, plain)
    assert th == ref_th and torch.equal(mask.cpu(), ref_mask)
    bad = score.clone()
    bad[5] = float("inf")
    with pytest.raises(ValueError, match="finite"):
        shard_select_balanced(bad.to(dev), 10, None, ent)


def test_group_benchmark_scores_outside_the_registry(dev):
    """Replay arms ranked by the two build-side scores (residual-blind |g| and
    |g + r| / sqrt(v + eps)): no reference counterpart, parity UNPINNED; checked
    bit for bit against the closed form in the oracle's group loop, with a live
    residual, clipping, AdamS and above the one-sweep select's size."""
    specs = [("abs_g_blind", 1.0, 2), ("abs_gr_over_sqrt_v", 1.0, 4), ("abs_g_blind", 10.0, 3, "adams"),
             ("abs_gr_over_sqrt_v", 0.1, 2, "adams", True), ("abs_g", 1.0, 2)]
    grp, out, w0 = _run_group(dev, specs, clip=0.3, W=7, bf16=True, sizes=_RAGGED)
    assert grp.last_select().path == 1
    _assert_group_equal(grp, out, specs)
    # the blind arm really ignores the residual: it differs from the |g + r| arm of the same shape
    assert not torch.equal(grp.state[0]["sel"], grp.state[4]["sel"])


@pytest.mark.parametrize("seed", range(6))
def test_randomized_groups(dev, seed):
    """Seeded random groups: ragged tensor sizes around 2^20 elements, 1..5
    configs drawn over score x ratio x cycle length x optimizer x fold x
    dual-lr, window length, gradient dtype, with and without clipping (the
    device's clip coefficient is handed to the oracle) -- end state bit for bit."""
    import random
    rng = random.Random(100 + seed)
    total = rng.choice([200_000, 900_000, 1_200_000, 1_500_007])
    sizes, left = [], total
    while left > 0:
        sz = min(left, rng.choice([3, 37, 128, 130, 1024, 4099, 100_000, 400_001]))
        sizes.append(sz)
        left -= sz
    if len(sizes) < 2:
        sizes = [sizes[0] - 1000, 1000]
    rng.shuffle(sizes)
    specs = [(rng.choice(["abs_g", "abs_m", "update", "coi"]), rng.choice([0.1, 1.0, 10.0]),
              rng.choice([1, 2, 3, 4]), rng.choice(["adamw", "adams"]), rng.choice([False, True]),
              rng.choice([1.0, 0.25, 2.0])) for _ in range(rng.randint(1, 5))]
    grp, out, w0 = _run_group(dev, specs, clip=rng.choice([0.0, 0.3]), W=rng.choice([4, 6, 9]),
                              bf16=rng.choice([True, False]), sizes=tuple(sizes))
    for ci, o in enumerate(out):
        s = grp.state[ci]
        assert torch.equal(s["sel"].cpu().bool(), o["sel"]), (ci, specs[ci])
        assert same_bits(s["res"], o["res"]) and same_bits(s["m"], o["m"]), (ci, specs[ci])
        assert same_bits(s["v"], o["v"]) and same_bits(s["w"], o["w"]), (ci, specs[ci])
