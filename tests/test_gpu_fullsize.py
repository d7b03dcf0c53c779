"""Full-size runs of the benchmark configurations checked through
size-independent properties (the CPU oracle would take minutes at these
sizes): exactly k selected, selected scores dominate unselected ones, ties
form an index prefix, idx sorted and consistent with the mask, values are the
rounded pre-step buffer, the residual is the buffer with selected coordinates
zeroed, m/v follow the closed form evaluated with torch on the device."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _student_t(n, seed, dev, scale=1e-3):
    gen = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(n, device=dev)
    step = 1 << 26
    for a in range(0, n, step):
        b = min(n, a + step)
        z = torch.randn(b - a, generator=gen, device=dev)
        chi = sum(torch.randn(b - a, generator=gen, device=dev).pow_(2) for _ in range(3))
        out[a:b] = z / torch.sqrt(chi / 3) * scale
    return out


def _check_select(score, mask, k, thresh):
    assert int(mask.sum()) == k
    sel_min = float(score[mask].min())
    assert sel_min == thresh
    if k < score.numel():
        assert float(score[~mask].max()) <= sel_min
    # ties at the threshold: the selected ones are the lowest-index ones
    ties = torch.nonzero(score == thresh).reshape(-1)
    taken = mask[ties]
    n_taken = int(taken.sum())
    assert bool(taken[:n_taken].all()) and not bool(taken[n_taken:].any())


def test_stress_1e9_global_topk_and_commit(dev):
    """Config 5: one contiguous 1.0e9-element fp32 buffer, heavy tails with 5 %
    duplicated magnitudes, exact global top-k at 0.01 % and 1 %, then the
    fused residual-aware AdamW step."""
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.replay import select_topk_flat
    n = 1_000_000_000
    g = _student_t(n, 7, dev)
    gen = torch.Generator(device=dev).manual_seed(1)
    dup = torch.randint(0, n, (n // 20,), generator=gen, device=dev)
    g[dup] = g[dup.roll(1)]                     # duplicated magnitudes -> tie layers
    del dup
    score = g.abs()
    for ratio in (0.01, 1.0):
        k = k_for(n, ratio)
        mask, th = select_topk_flat(score, k)
        _check_select(score, mask, k, th)
        del mask
    del score
    segs = [dict(start=0, n=n, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.1)]
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    r = torch.zeros(n, device=dev)
    k = k_for(n, 1.0)
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, max_k=k, want_mask=True)
    idx, vals = fs.step(g, r, p, m, v, 1, k=k)
    res = fs.read_result()
    assert res.status == 0 and res.n_selected == k and res.nonfinite == 0
    mask = fs.mask.bool()
    _check_select(g.abs(), mask, k, res.thresh)
    assert torch.equal(idx.long(), torch.nonzero(mask).reshape(-1))
    assert torch.equal(vals, g[mask])
    assert torch.equal(r, torch.where(mask, torch.zeros((), device=dev), g))
    assert torch.equal(m, torch.where(mask, g * (1.0 - 0.9), torch.zeros((), device=dev)))
    gq = torch.where(mask, g, torch.zeros((), device=dev))
    assert torch.equal(v, (gq * (1.0 - 0.95)) * gq)


@pytest.mark.parametrize("ratio", [0.1, 1.0, 10.0])
def test_llama1b_set_index_layout(dev, ratio):
    """Config 3: Llama-3.2-1B set, bf16 Student-t grads, int32 + bf16 pack."""
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.shapes import llama32_1b, segments_for
    segs, n = segments_for(llama32_1b())
    assert n == 1_235_814_400 and len(segs) == 146
    g = _student_t(n, 3, dev).to(torch.bfloat16)
    gen = torch.Generator(device=dev).manual_seed(2)
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m = torch.randn(n, generator=gen, device=dev) * 1e-4
    v = torch.rand(n, generator=gen, device=dev) * 1e-8
    r = _student_t(n, 4, dev, scale=3e-4)
    buf = r + g.float()
    m0 = m.clone()
    k = k_for(n, ratio)
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, max_k=k, want_mask=True)
    idx, vals = fs.step(g, r, p, m, v, 5, k=k)
    res = fs.read_result()
    assert res.status == 0 and res.n_selected == k and res.path == 1
    mask = fs.mask.bool()
    _check_select(buf.abs(), mask, k, res.thresh)
    assert idx.dtype == torch.int32 and vals.dtype == torch.bfloat16
    assert torch.equal(idx.long(), torch.nonzero(mask).reshape(-1))
    assert torch.equal(vals, buf[mask].to(torch.bfloat16))
    assert torch.equal(r, torch.where(mask, torch.zeros((), device=dev), buf))
    gq = torch.where(mask, buf.to(torch.bfloat16).float(), torch.zeros((), device=dev))
    assert torch.equal(m, m0 * 0.9 + gq * (1.0 - 0.9))


def test_qwen06b_set_mask_layout_per_bucket(dev):
    """Config 2: Qwen3-0.6B set, bf16 Gaussian grads with per-tensor std
    log-uniform in [1e-5, 1e-2], per-bucket top-k at 1 %, mask layout."""
    from sga_amd import backends
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    assert n == 596_049_920 and len(segs) == 310
    gen = torch.Generator(device=dev).manual_seed(5)
    g = torch.empty(n, dtype=torch.bfloat16, device=dev)
    cpu_gen = torch.Generator().manual_seed(5)
    for s in segs:
        std = 10 ** (-5 + 3 * float(torch.rand(1, generator=cpu_gen)))
        g[s["start"]:s["start"] + s["n"]] = (torch.randn(s["n"], generator=gen, device=dev)
                                             * std).to(torch.bfloat16)
    # buckets: the embedding, then groups of 4 layers, as contiguous flat ranges
    cuts = [0, segs[1]["start"]] + [segs[1 + 11 * j]["start"] for j in range(4, 28, 4)] + [n]
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m, v, r = (torch.zeros(n, device=dev) for _ in range(3))
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        bsegs = [dict(s, start=s["start"] - lo) for s in segs if lo <= s["start"] < hi]
        nb = hi - lo
        k = k_for(nb, 1.0)
        fs = FusedSparseStep(nb, bsegs, dev, values_dtype=torch.float32, max_k=k, want_mask=True)
        buf = g[lo:hi].float()
        idx, vals = fs.step(g[lo:hi], r[lo:hi], p[lo:hi], m[lo:hi], v[lo:hi], 1, k=k)
        res = fs.read_result()
        assert res.status == 0 and res.n_selected == k
        _check_select(buf.abs(), fs.mask.bool(), k, res.thresh)
        # mask layout of the reference's torch_pipelined_mask: 2 slices at N//2,
        # payload = ordered compaction of the (pre-step) buffer
        payloads, idx2 = backends.mask_layout_pack(buf, fs.mask, factor=1.0, slices=2)
        assert torch.equal(idx2, idx)
        assert torch.equal(torch.cat(payloads), vals)
        split = int((idx < nb // 2).sum())
        assert payloads[0].numel() == split
        dst = torch.zeros(nb, device=dev)
        backends.mask_layout_unpack(dst, idx2, payloads)
        assert torch.equal(dst, torch.where(fs.mask.bool(), buf, torch.zeros((), device=dev)))


def test_qwen06b_set_mask_layout_buckets_in_one_call(dev):
    """Config 2 through `sga_fused_sparse_step_multi`: the eight buckets of the
    Qwen3-0.6B set stepped by ONE call (their short select kernels batched)
    give, bucket by bucket, the bits of eight separate calls over two steps."""
    from sga_amd.fused_step import FusedSparseStep, fused_step_multi, k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    grads = [_qwen_log_uniform_grads(dev, segs, n, 5 + i) for i in range(2)]
    cuts = [0, segs[1]["start"]] + [segs[1 + 11 * j]["start"] for j in range(4, 28, 4)] + [n]
    spans = list(zip(cuts[:-1], cuts[1:]))
    gen = torch.Generator(device=dev).manual_seed(5)
    p0 = torch.randn(n, generator=gen, device=dev) * 0.02
    state = [[torch.zeros(n, device=dev), p0.clone(), torch.zeros(n, device=dev),
              torch.zeros(n, device=dev)] for _ in range(2)]                 # r, p, m, v
    steppers = []
    for which in range(2):
        row = []
        for lo, hi in spans:
            bsegs = [dict(s, start=s["start"] - lo) for s in segs if lo <= s["start"] < hi]
            row.append(FusedSparseStep(hi - lo, bsegs, dev, values_dtype=torch.float32,
                                       max_k=k_for(hi - lo, 1.0), want_mask=True))
        steppers.append(row)
    ks = [k_for(hi - lo, 1.0) for lo, hi in spans]
    for step in (1, 2):
        g = grads[step - 1]
        for b, (lo, hi) in enumerate(spans):
            steppers[0][b].step(g[lo:hi], *[t[lo:hi] for t in state[0]], step, k=ks[b])
        fused_step_multi(steppers[1], [g[lo:hi] for lo, hi in spans],
                         *[[state[1][a][lo:hi] for lo, hi in spans] for a in range(4)], step,
                         ks=ks)
        for b in range(len(spans)):
            a, c = steppers[0][b], steppers[1][b]
            ra, rc = a.read_result(), c.read_result()
            assert rc.status == 0 and rc.n_selected == ks[b] and rc.path == 1, (step, b, vars(rc))
            assert vars(ra) == vars(rc), (step, b)
            assert torch.equal(a.idx[:ks[b]], c.idx[:ks[b]]) and torch.equal(a.mask, c.mask)
            assert torch.equal(a.values[:ks[b]].view(torch.int32),
                               c.values[:ks[b]].view(torch.int32))
        for x, y in zip(state[0], state[1]):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), step


def _dev_scalar(x, dev):
    return torch.tensor(x, dtype=torch.float32, device=dev)


def _update_score_torch(segs, p, m, v, q, step):
    """|wd*p + U(q)| with plain torch ops on the device, one separately rounded
    fp32 kernel per operation in the order of scores.py:183-226.  Divisions go
    through 0-dim device tensors: torch divides a device tensor by a Python
    scalar as a multiplication by the reciprocal, by a tensor as a division."""
    dev = q.device
    out = torch.empty_like(q)
    for s in segs:
        a = s["start"] if "start" in s else s["a"]
        b = a + s["n"]
        b1, b2 = s["b1"], s["b2"]
        sa = (m[a:b] * b1 + q[a:b] * (1.0 - b1)) / _dev_scalar(1.0 - b1 ** step, dev)
        sb = (v[a:b] * b2 + (q[a:b] * (1.0 - b2)) * q[a:b]) / _dev_scalar(1.0 - b2 ** step, dev)
        out[a:b] = (s["wd"] * p[a:b] + sa / (torch.sqrt(sb) + s["eps"])).abs()
    return out


@pytest.mark.parametrize("ratio", [0.1, 1.0, 10.0])
def test_llama1b_set_update_score(dev, ratio):
    """Config 3 as worded: Llama-3.2-1B set, bf16 Student-t grads, the
    Adam-normalised score (`update`, scores.py:202-231) at 0.1 / 1 / 10 %,
    index pack int32 + bf16.  The score is rebuilt with torch ops on the device
    from the pre-step state; the one-sweep select scores slabs that straddle
    the 146 tensors with per-tensor weight decay."""
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.shapes import llama32_1b, segments_for
    segs, n = segments_for(llama32_1b())
    step = 5
    g = _student_t(n, 3, dev).to(torch.bfloat16)
    gen = torch.Generator(device=dev).manual_seed(2)
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m = torch.randn(n, generator=gen, device=dev) * 1e-4
    v = torch.rand(n, generator=gen, device=dev) * 1e-8
    r = _student_t(n, 4, dev, scale=3e-4)
    buf = r + g.float()
    score = _update_score_torch(segs, p, m, v, buf, step)
    m0 = m.clone()
    k = k_for(n, ratio)
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, max_k=k, want_mask=True)
    idx, vals = fs.step(g, r, p, m, v, step, k=k, score="update")
    res = fs.read_result()
    assert res.status == 0 and res.n_selected == k and res.path == 1 and res.nonfinite == 0
    mask = fs.mask.bool()
    _check_select(score, mask, k, res.thresh)
    assert torch.equal(idx.long(), torch.nonzero(mask).reshape(-1))
    assert torch.equal(vals, buf[mask].to(torch.bfloat16))
    assert torch.equal(r, torch.where(mask, torch.zeros((), device=dev), buf))
    gq = torch.where(mask, buf.to(torch.bfloat16).float(), torch.zeros((), device=dev))
    assert torch.equal(m, m0 * 0.9 + gq * (1.0 - 0.9))


@pytest.mark.parametrize("ratio", [0.1, 1.0, 10.0])
def test_llama1b_set_update_score_single_sweep(dev, ratio):
    """The same configuration through the single-sweep step (g / resid / p /
    m / v read once): the same properties against the torch rebuild of the
    score, and every output -- idx, values, mask, residual, p, m, v, threshold
    -- equal bit for bit to the two-sweep step run from the same state."""
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.shapes import llama32_1b, segments_for
    segs, n = segments_for(llama32_1b())
    step = 5
    g = _student_t(n, 3, dev).to(torch.bfloat16)
    gen = torch.Generator(device=dev).manual_seed(2)
    p = torch.randn(n, generator=gen, device=dev) * 0.02
    m = torch.randn(n, generator=gen, device=dev) * 1e-4
    v = torch.rand(n, generator=gen, device=dev) * 1e-8
    r = _student_t(n, 4, dev, scale=3e-4)
    k = k_for(n, ratio)
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, max_k=k, want_mask=True)
    r2, p2, m2, v2 = r.clone(), p.clone(), m.clone(), v.clone()
    idx, vals = fs.step(g, r2, p2, m2, v2, step, k=k, score="update")
    ref = fs.read_result()
    idx2, vals2, mask2 = idx.clone(), vals.clone(), fs.mask.clone()
    assert ref.status == 0 and ref.path == 1
    idx, vals = fs.step(g, r, p, m, v, step, k=k, score="update", single_sweep=True)
    res = fs.read_result()
    assert res.status == 0 and res.n_selected == k and res.path == 2 and res.nonfinite == 0
    assert (res.thresh_bits, res.need, res.n_gt, res.n_eq) == (ref.thresh_bits, ref.need, ref.n_gt,
                                                              ref.n_eq)
    assert torch.equal(idx, idx2) and torch.equal(fs.mask, mask2)
    assert torch.equal(vals.view(torch.int16), vals2.view(torch.int16))
    for a, b in ((r, r2), (p, p2), (m, m2), (v, v2)):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))


def test_llama1b_set_single_sweep_seeded_configs(dev):
    """Seeded draws of score, ratio (0.01 - 25 %), gradient and value dtype and
    the commit knobs on the full 1.24 B-element set, three steps each from a
    shared start: the single-sweep step and the two-sweep step agree in every
    output bit.  At this size the record lists, their overflow list and the
    dense pack all carry millions of entries."""
    import random
    from sga_amd.fused_step import FusedSparseStep, k_for
    from sga_amd.shapes import llama32_1b, segments_for
    segs, n = segments_for(llama32_1b())
    rnd = random.Random(7)
    gen = torch.Generator(device=dev).manual_seed(0)
    p0 = torch.randn(n, generator=gen, device=dev) * 0.02
    grads = [_student_t(n, 10 + i, dev) for i in range(2)]
    for cfg in range(5):
        score = rnd.choice(["abs_g", "update", "coi", "abs_g_blind", "abs_gr_over_sqrt_v"])
        ratio = rnd.choice([0.01, 0.1, 1.0, 3.2, 10.0, 25.0])
        vdt = rnd.choice([torch.bfloat16, torch.float32])
        gdt = rnd.choice([torch.bfloat16, torch.float32])
        knobs = rnd.choice([{}, dict(optimizer="adams"), dict(fold=True, interval=3.0),
                            dict(factor=0.5, coeff=0.25)])
        what = (cfg, score, ratio, vdt, gdt, knobs)
        k = k_for(n, ratio)
        state = [[p0.clone()] + [torch.zeros(n, device=dev) for _ in range(3)] for _ in range(2)]
        fs = [FusedSparseStep(n, segs, dev, values_dtype=vdt, max_k=k, want_mask=True)
              for _ in range(2)]
        for step in range(1, 4):
            g = grads[step % 2].to(gdt)
            outs = []
            for which in range(2):
                pp, mm, vv, rr = state[which]
                idx, vals = fs[which].step(g, rr, pp, mm, vv, step, k=k, score=score,
                                           single_sweep=bool(which), **knobs)
                res = fs[which].read_result()
                assert res.status == 0 and res.n_selected == k, (what, step, which, vars(res))
                outs.append((idx, vals, fs[which].mask, res))
            a, b = outs[0][3], outs[1][3]
            assert (a.thresh_bits, a.need, a.n_eq) == (b.thresh_bits, b.need, b.n_eq), (what, step)
            assert torch.equal(outs[0][0], outs[1][0]), (what, step)
            assert torch.equal(outs[0][2], outs[1][2]), (what, step)
            it = torch.int16 if vdt == torch.bfloat16 else torch.int32
            assert torch.equal(outs[0][1].view(it), outs[1][1].view(it)), (what, step)
            for x, y in zip(state[0], state[1]):
                assert torch.equal(x.view(torch.int32), y.view(torch.int32)), (what, step)
        del fs, state
        torch.cuda.empty_cache()


def _both_steps_agree(dev, segs, n, grads, score, k, what, steps=2, p_seed=3):
    """The single-sweep step against the two-sweep step from the same state
    over `steps` steps: every output bit (idx, values, mask, residual, p, m,
    v, threshold, tie counts), and the single sweep must have gone ahead
    (path 2) and ended with status 0."""
    from sga_amd.fused_step import FusedSparseStep
    gen = torch.Generator(device=dev).manual_seed(p_seed)
    p0 = torch.randn(n, generator=gen, device=dev) * 0.02
    state = [[p0.clone()] + [torch.zeros(n, device=dev) for _ in range(3)] for _ in range(2)]
    del p0
    fs = [FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, max_k=k, want_mask=True)
          for _ in range(2)]
    for step in range(1, steps + 1):
        g = grads[(step - 1) % len(grads)]
        outs = []
        for which in range(2):
            pp, mm, vv, rr = state[which]
            idx, vals = fs[which].step(g, rr, pp, mm, vv, step, k=k, score=score,
                                       single_sweep=bool(which), check=False)
            res = fs[which].read_result()
            assert res.status == 0 and res.n_selected == k, (what, step, which, vars(res))
            outs.append((idx, vals, fs[which].mask, res))
        a, b = outs[0][3], outs[1][3]
        assert b.path == 2, (what, step, vars(b))
        assert (a.thresh_bits, a.need, a.n_gt, a.n_eq) == (b.thresh_bits, b.need, b.n_gt, b.n_eq), (
            what, step)
        assert torch.equal(outs[0][0], outs[1][0]), (what, step)
        assert torch.equal(outs[0][2], outs[1][2]), (what, step)
        assert torch.equal(outs[0][1].view(torch.int16), outs[1][1].view(torch.int16)), (what, step)
        for x, y in zip(state[0], state[1]):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), (what, step)
    del fs, state
    torch.cuda.empty_cache()


def _qwen_log_uniform_grads(dev, segs, n, seed):
    """bf16 Gaussian gradients with a per-tensor std log-uniform in [1e-5, 1e-2]."""
    gen = torch.Generator(device=dev).manual_seed(seed)
    cpu_gen = torch.Generator().manual_seed(seed)
    g = torch.empty(n, dtype=torch.bfloat16, device=dev)
    for s in segs:
        std = 10 ** (-5 + 3 * float(torch.rand(1, generator=cpu_gen)))
        g[s["start"]:s["start"] + s["n"]] = (torch.randn(s["n"], generator=gen, device=dev)
                                             * std).to(torch.bfloat16)
    return g


@pytest.mark.parametrize("score", ["abs_g", "update"])
def test_qwen06b_log_uniform_scales_single_sweep_one_bucket(dev, score):
    """The single-sweep step on per-tensor scales three decades apart (config
    2's gradient distribution), the whole 596 M-element set as ONE bucket: the
    sampled bracket has to hold although a few tensors own the whole top 1 %."""
    from sga_amd.fused_step import k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    grads = [_qwen_log_uniform_grads(dev, segs, n, 5 + i) for i in range(2)]
    _both_steps_agree(dev, segs, n, grads, score, k_for(n, 1.0), ("one bucket", score))


def test_qwen06b_log_uniform_scales_single_sweep_per_bucket(dev):
    """The same distribution stepped as config 2 words it: the embedding and
    seven buckets of four layers, each with its own top 1 %."""
    from sga_amd.fused_step import k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    grads = [_qwen_log_uniform_grads(dev, segs, n, 5 + i) for i in range(2)]
    cuts = [0, segs[1]["start"]] + [segs[1 + 11 * j]["start"] for j in range(4, 28, 4)] + [n]
    for b, (lo, hi) in enumerate(zip(cuts[:-1], cuts[1:])):
        bsegs = [dict(s, start=s["start"] - lo) for s in segs if lo <= s["start"] < hi]
        _both_steps_agree(dev, bsegs, hi - lo, [g[lo:hi] for g in grads], "update",
                          k_for(hi - lo, 1.0), ("bucket", b))


@pytest.mark.parametrize("score", ["abs_g", "update"])
def test_single_sweep_when_the_last_tensors_have_no_gradient(dev, score):
    """Absent parameters: the last fifth of the set (whole tensors) has an
    all-zero gradient, so the tail of the bucket scores unlike the rest."""
    from sga_amd.fused_step import k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    cut = next(s["start"] for s in segs if s["start"] >= n - n // 5)
    grads = []
    for i in range(2):
        g = _student_t(n, 20 + i, dev).to(torch.bfloat16)
        g[cut:] = 0
        grads.append(g)
    _both_steps_agree(dev, segs, n, grads, score, k_for(n, 1.0), ("absent tail", score))


@pytest.mark.parametrize("ratio", [1.0, 0.3])
def test_single_sweep_when_the_last_percent_scores_100x(dev, ratio):
    """The last 1 % of the coordinates carries gradients 100 times larger than
    the rest: a sample that under-covered the end of the bucket would put the
    bracket in the wrong place (k = 1 %: the k-th key lies right where the two
    populations meet; k = 0.3 %: entirely inside the tail)."""
    from sga_amd.fused_step import k_for
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    grads = []
    for i in range(2):
        g = _student_t(n, 30 + i, dev)
        g[n - n // 100:] *= 100.0
        grads.append(g.to(torch.bfloat16))
    _both_steps_agree(dev, segs, n, grads, "update", k_for(n, ratio), ("hot tail", ratio))


def _select_ok(score, mask, k):
    """Exact-k, dominance and lowest-index ties of a mask against a score."""
    assert int(mask.sum()) == k
    th = float(score[mask].min())
    _check_select(score, mask, k, th)


def test_qwen06b_replay_group_full_window(dev):
    """Config 4 at full size: Qwen3-0.6B shapes (596,049,920 elements, 310
    tensors), G = 8 configs over score x ratio x cycle length, window of 32
    recorded bf16 steps, clip 1.0.  Size-independent properties:
    * every config's mask holds exactly k coordinates at every step end checked;
    * T = 1 configs never keep a residual;
    * off a boundary the residual is zero on the mask and the running fp32 sum
      of the recorded gradient since the last boundary elsewhere;
    * the re-selection at si = 16 of the T = 16 arm (15 masked steps of
      residual behind it), at si = 28 of a T = 4 `update` arm and at si = 24 of
      a T = 4 residual-blind arm equal the exact top-k of the score rebuilt,
      with plain torch ops on the device, from the state just before that step;
    * with clipping off, a T = 1 arm is the dense reference trajectory
      (sga_dense_replay_step) bit for bit."""
    from sga_amd.replay import select_topk_flat
    from sga_amd.replay_dense import DenseReplay
    from sga_amd.replay_group import Config, ReplayGroup
    from sga_amd.shapes import qwen3_06b, segments_for
    segs, n = segments_for(qwen3_06b())
    assert n == 596_049_920 and len(segs) == 310
    W, t0, lr = 32, 100, 1e-4
    entries = [{"a": s["start"], "n": s["n"], "b1": s["b1"], "b2": s["b2"], "eps": s["eps"],
                "wd": s["wd"]} for s in segs]
    specs = [("abs_g", 1.0, 1), ("abs_g", 0.1, 4), ("abs_g", 10.0, 16), ("update", 1.0, 4),
             ("update", 10.0, 1), ("coi", 1.0, 16), ("abs_g_blind", 1.0, 4), ("update", 0.1, 16)]
    cfgs = [Config(*sp) for sp in specs]
    gen = torch.Generator(device=dev).manual_seed(1)
    w0 = torch.randn(n, generator=gen, device=dev) * 0.02
    m0 = torch.randn(n, generator=gen, device=dev) * 1e-4
    v0 = torch.rand(n, generator=gen, device=dev) * 1e-8
    window = [_student_t(n, 500 + s, dev, scale=1e-3 * (1.0 + 0.02 * s)).to(torch.bfloat16)
              for s in range(W)]
    ks = [max(1, int(round(c.ratio / 100.0 * n))) for c in cfgs]
    base = window[0].float().abs()
    sel0 = [select_topk_flat(base, k)[0] for k in ks]
    del base
    grp = ReplayGroup(entries, w0, m0, v0, sel0, cfgs, t0, W)
    del sel0
    meta = {"clip_grad": 1.0, "grad_norm": float("nan"), "lr": lr}
    probes = {16: 2, 24: 6, 28: 3}                # si -> config whose re-selection is rebuilt
    for si in range(W):
        pre = None
        if si in probes:
            s = grp.state[probes[si]]
            pre = {x: s[x].clone() for x in ("w", "m", "v", "res")}
        grp.step(window[si], meta)
        if pre is not None:
            ci = probes[si]
            c = cfgs[ci]
            coef = grp.coef_f[ci:ci + 1]
            assert 0.0 < float(coef) < 1.0                     # the clip is live
            q = (window[si].float() + pre["res"]) * coef       # coef_dense == 1 (no recorded norm)
            assert float(pre["res"].abs().max()) > 0.0         # a live residual behind the boundary
            if c.score == "abs_g":
                score = q.abs()
            elif c.score == "abs_g_blind":
                score = (window[si].float() * coef).abs()      # the residual takes no part
            else:
                assert c.score == "update"
                score = _update_score_torch(entries, pre["w"], pre["m"], pre["v"], q,
                                            t0 + si + 1)
            _select_ok(score, grp.state[ci]["sel"].bool(), ks[ci])
            del pre, q, score
    for ci, c in enumerate(cfgs):
        s = grp.state[ci]
        mask = s["sel"].bool()
        assert int(mask.sum()) == ks[ci], ci
        res = s["res"]
        if c.T == 1:
            assert float(res.abs().max()) == 0.0, ci
            continue
        last_b = ((W - 1) // c.T) * c.T                        # res was zeroed there
        acc = torch.zeros(n, device=dev)
        for si in range(last_b + 1, W):
            acc += window[si].float()
        assert torch.equal(res, torch.where(mask, torch.zeros((), device=dev), acc)), ci
        del acc
    del grp
    torch.cuda.empty_cache()
    # clipping off: a T = 1 arm IS the dense trajectory
    steps = 6
    sel = torch.zeros(n, dtype=torch.bool, device=dev)
    grp = ReplayGroup(entries, w0, m0, v0, [sel], [Config("abs_g", 1.0, 1)], t0, steps)
    dense = DenseReplay(entries, w0, m0, v0, t0)
    for si in range(steps):
        grp.step(window[si], {"clip_grad": 0.0, "lr": lr})
        dense.step(t0 + si, window[si], {"clip_grad": 0.0, "lr": [lr]})
    s = grp.state[0]
    for name, ref in (("w", dense.w), ("m", dense.m), ("v", dense.v)):
        assert torch.equal(s[name].view(torch.int32), ref.view(torch.int32)), name
