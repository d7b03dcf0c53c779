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
