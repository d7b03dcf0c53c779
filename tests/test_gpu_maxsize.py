"""The largest bucket the boundary admits, n = 2^31 - 1 (indices are int32;
an odd length, so the last chunk and the last quad are ragged).  The CPU
oracle cannot run this size in seconds, so the selection is checked through
its defining properties with torch ops on the device, the two step variants
against each other bit for bit, and the commit against the oracle's own
pack + commit on windows at the two ends of the index range and across a
tensor boundary, given the device's selection."""
import pytest
import torch

from oracle import adamw as A
from oracle import kernels as K
from tests.test_gpu_fullsize import _student_t
from tests.util import same_bits

pytestmark = pytest.mark.gpu

N = (1 << 31) - 1
HALVES = ((0, 1 << 30), (1 << 30, N))       # torch's own ops are kept below 2^31 - 1 elements


def _check_select_halves(score, mask, k, thresh):
    """exactly k selected; min over the selected == thresh >= max over the
    rest; the ties at thresh that are taken are the lowest-index ones"""
    count, sel_min, rest_max, ties = 0, float("inf"), -float("inf"), []
    for a, b in HALVES:
        s, mk = score[a:b], mask[a:b]
        count += int(mk.sum())
        if bool(mk.any()):
            sel_min = min(sel_min, float(s[mk].min()))
        if not bool(mk.all()):
            rest_max = max(rest_max, float(s[~mk].max()))
        ties.append(torch.nonzero(s == thresh).reshape(-1) + a)
    assert count == k
    assert sel_min == thresh and rest_max <= thresh
    ties = torch.cat(ties)
    taken = mask[ties]
    n_taken = int(taken.sum())
    assert bool(taken[:n_taken].all()) and not bool(taken[n_taken:].any())


def _plant_ends(x, big):
    """Coordinates at both ends of the index range that any selection takes."""
    x[:3] = big
    x[N - 3:] = big
    x[N - 1025] = big                         # last coordinate of the last whole chunk


def test_select_topk_flat_at_the_largest_n(dev):
    from sga_amd.fused_step import k_for
    from sga_amd.replay import select_topk_flat
    score = _student_t(N, 21, dev).abs_()
    gen = torch.Generator(device=dev).manual_seed(3)
    dup = torch.randint(0, N, (N // 64,), generator=gen, device=dev)
    score[dup] = score[dup.roll(1)]          # duplicated magnitudes: tie layers at any threshold
    del dup
    _plant_ends(score, 1.0)
    for ratio in (1.0, 0.001):
        k = k_for(N, ratio)
        mask, th = select_topk_flat(score, k)
        _check_select_halves(score, mask, k, th)
        assert bool(mask[:3].all()) and bool(mask[N - 3:].all()) and bool(mask[N - 1025])
        del mask


def _segments():
    """Five tensors with their own hyper-parameters; boundaries off every
    alignment, one inside the last chunk."""
    cuts = [0, 400_000_003, 1_000_000_001, 1_600_000_130, N - 700, N]
    hp = [(1e-4, 0.9, 0.95, 1e-8, 0.1), (3e-4, 0.8, 0.99, 1e-6, 0.0), (1e-3, 0.9, 0.999, 1e-8, 0.01),
          (5e-5, 0.95, 0.9, 1e-7, 0.05), (2e-4, 0.85, 0.98, 1e-8, 0.2)]
    return [dict(start=a, n=b - a, lr=h[0], b1=h[1], b2=h[2], eps=h[3], wd=h[4])
            for a, b, h in zip(cuts[:-1], cuts[1:], hp)]


def _oracle_window(a, b, segs, step, g, r0, p0, m0, v0, idx, values_dtype):
    """The oracle's pack + compact commit on coordinates [a, b) alone, given
    the device's selection ``idx`` (ascending): returns (values, r, p, m, v)."""
    lo = int(torch.searchsorted(idx, a))
    hi = int(torch.searchsorted(idx, b))
    local = (idx[lo:hi].long() - a).cpu().to(torch.int32)
    buf = r0[a:b].cpu() + g[a:b].cpu().float()
    p, m, v = p0[a:b].cpu().clone(), m0[a:b].cpu().clone(), v0[a:b].cpu().clone()
    values = torch.empty(local.numel(), dtype=values_dtype)
    K.pack_selected(buf, local, values, 1.0)
    for s in segs:
        sa, sb = max(a, s["start"]), min(b, s["start"] + s["n"])
        if sa >= sb:
            continue
        A.adamw_grad_correct_compact(
            p[sa - a:sb - a], buf[sa - a:sb - a], m[sa - a:sb - a], v[sa - a:sb - a], local,
            values, sa - a, s["lr"], s["b1"], s["b2"], s["eps"], s["wd"], step)
    return (lo, hi), values, buf, p, m, v


@pytest.mark.parametrize("score", ["abs_g", "update"])
def test_fused_step_at_the_largest_n(dev, score):
    """Two-sweep step in place on a copy, single-sweep step out of place from
    the original state: equal bit for bit; windows at both ends of the index
    range and across the boundary inside the last chunk equal the oracle's
    pack + commit; for |g + r| the selection's defining properties hold."""
    from sga_amd.fused_step import FusedSparseStep, k_for
    segs, step = _segments(), 3
    g = _student_t(N, 31, dev)
    _plant_ends(g, 1.0)
    g = g.to(torch.bfloat16)
    gen = torch.Generator(device=dev).manual_seed(9)
    p0 = torch.randn(N, generator=gen, device=dev) * 0.02
    m0 = torch.randn(N, generator=gen, device=dev) * 1e-4
    v0 = torch.rand(N, generator=gen, device=dev) * 1e-8
    r0 = _student_t(N, 32, dev, scale=3e-4)
    k = k_for(N, 1.0)
    fs = FusedSparseStep(N, segs, dev, values_dtype=torch.bfloat16, max_k=k, want_mask=True)

    two = [t.clone() for t in (r0, p0, m0, v0)]
    idx, vals = fs.step(g, *two, step, k=k, score=score)
    res2 = fs.read_result()
    assert res2.status == 0 and res2.n_selected == k and res2.nonfinite == 0, vars(res2)
    idx2, vals2, mask2 = idx.clone(), vals.clone(), fs.mask.clone()
    if score == "abs_g":
        buf = torch.empty(N, device=dev)
        for a, b in HALVES:
            buf[a:b] = r0[a:b] + g[a:b].float()
        _check_select_halves(buf.abs_(), mask2.bool(), k, res2.thresh)
        del buf
    if score == "abs_g":                     # the planted coordinates: both ends of the int32 range
        assert int(idx2[0]) == 0 and int(idx2[-1]) == N - 1
    assert bool((idx2[1:] > idx2[:-1]).all())
    for a, b in HALVES:                      # idx is the mask, compacted
        lo, hi = int(torch.searchsorted(idx2, a)), int(torch.searchsorted(idx2, b))
        assert torch.equal(idx2[lo:hi].long(), torch.nonzero(mask2[a:b]).reshape(-1) + a)

    one = [torch.empty(N, device=dev) for _ in range(4)]
    idx, vals = fs.step(g, r0, p0, m0, v0, step, k=k, score=score, single_sweep=True, out=one)
    res1 = fs.read_result()
    assert res1.status == 0 and res1.path == 2 and not res1.redone, vars(res1)
    assert res1.thresh_bits == res2.thresh_bits and res1.n_selected == k
    assert torch.equal(idx, idx2) and torch.equal(vals.view(torch.int16), vals2.view(torch.int16))
    assert torch.equal(fs.mask, mask2)
    for t1, t2 in zip(one, two):
        assert torch.equal(t1.view(torch.int32), t2.view(torch.int32))
    del one, mask2

    span = 1 << 18
    for a, b in ((0, span), (N - span - 3, N), (400_000_003 - 777, 400_000_003 + span)):
        (lo, hi), values, r, p, m, v = _oracle_window(a, b, segs, step, g, r0, p0, m0, v0, idx2,
                                                      torch.bfloat16)
        assert hi > lo
        assert torch.equal(vals2[lo:hi].cpu().view(torch.int16), values.view(torch.int16)), (a, b)
        for dev_t, ref in zip(two, (r, p, m, v)):
            assert same_bits(dev_t[a:b], ref), (a, b)
