"""GPU parity of the exact top-k select (both tie semantics), the balanced /
fast histogram tiers and the replay select building blocks vs the CPU
oracle.  Masks, indices, counts and thresholds are bit-exact."""
import json
import os

import pytest
import torch

from oracle import select as SEL
from tests.test_oracle_select import adversarial
from tests.util import adv, student_t

pytestmark = pytest.mark.gpu
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "select_kats.json")))


@pytest.mark.parametrize("kat", KATS["tie_fill"], ids=lambda k: k["name"])
def test_tie_fill_kats(dev, kat):
    from sga_amd.replay import select_topk_flat
    t = torch.tensor(kat["t"], dtype=torch.float32, device=dev)
    mask, th = select_topk_flat(t, kat["k"])
    assert mask.dtype == torch.bool
    assert mask.cpu().to(torch.int64).tolist() == kat["mask"] and th == kat["thresh"]


@pytest.mark.parametrize("kat", KATS["rejections"])
def test_rejections(dev, kat):
    from sga_amd.replay import select_topk_flat
    t = torch.tensor([float(x) for x in kat["t"]], dtype=torch.float32, device=dev)
    with pytest.raises(ValueError) as ei:
        select_topk_flat(t, kat["k"])
    assert kat["substr"] in str(ei.value)


def test_adversarial_families_bitwise(dev):
    from sga_amd.replay import select_topk_flat
    gen = torch.Generator().manual_seed(20260912)
    n = 200_000
    for name, sc in adversarial(n, gen).items():
        npos = max(8, n // 1000)
        ks = sorted({1, n // 100, 3 * n // 10, n - 1, n})
        if name == "zero-heavy":
            ks = sorted(set(ks) | {max(1, npos // 2), min(n, npos * 4)})
        sd = sc.to(dev)
        for k in ks:
            m_ref, t_ref = SEL.select_topk_flat(sc, k)
            m_dev, t_dev = select_topk_flat(sd, k)
            assert t_dev == t_ref, (name, k)
            assert torch.equal(m_dev.cpu(), m_ref), (name, k)


@pytest.mark.parametrize("n", [1, 5, 1023, 1024, 1025, 4097, 1_000_003])
def test_sizes_and_random_bit_patterns(dev, n):
    from sga_amd.replay import select_topk_flat
    sc = adv(n, n, nonneg=True)
    for k in sorted({1, max(1, n // 100), max(1, n // 2), n}):
        m_ref, t_ref = SEL.select_topk_flat(sc, k)
        m_dev, t_dev = select_topk_flat(sc.to(dev), k)
        assert t_dev == t_ref and torch.equal(m_dev.cpu(), m_ref), (n, k)


def test_heavy_tail_with_duplicates(dev):
    """Stress-config shape at reduced size: heavy-tailed magnitudes with 5 %
    duplicated values, ratios 0.01 % and 1 %."""
    from sga_amd.replay import select_topk_flat
    n = 3_000_000
    sc = student_t(n, 3).abs()
    gen = torch.Generator().manual_seed(1)
    dup = torch.randint(0, n, (n // 20,), generator=gen)
    sc[dup] = sc[dup.roll(1)]
    for ratio in (0.01, 1.0):
        k = SEL.k_for(n, ratio)
        m_ref, t_ref = SEL.select_topk_flat(sc, k)
        m_dev, t_dev = select_topk_flat(sc.to(dev), k)
        assert t_dev == t_ref and torch.equal(m_dev.cpu(), m_ref)


def test_online_ties_all_views(dev):
    """Distribution families of the reference's xp-capability test: exact
    histogram tier == kthvalue masks, ties all selected, over split views."""
    from sga_amd.selection import select_masks_exact_kthvalue, select_masks_histogram
    N = 4097
    g = torch.Generator().manual_seed(1234)
    ds = [torch.randn(N, generator=g) * 1e-3,
          (torch.randn(N, generator=g) * 1e3).round() / 1e3,
          torch.randn(N, generator=g).exp() * torch.sign(torch.randn(N, generator=g)),
          torch.full((N,), 0.5), torch.randn(N, generator=g) * 1e-3,
          torch.randn(N, generator=g) * 1e-3]
    ds[4][::3] = 0.0
    ds[5][::7] *= 1e30
    for x in ds:
        views = [x[:N // 2].contiguous(), x[N // 2:].contiguous()]
        dviews = [v.to(dev) for v in views]
        for k in (1, 2, N // 10, N // 2, N - 1, N):
            t_ref, m_ref = SEL.select_masks_histogram(views, k, mode="exact")
            t_dev, m_dev = select_masks_histogram(dviews, k, None, mode="exact")
            assert t_dev == t_ref
            for a, b in zip(m_dev, m_ref):
                assert a.dtype == torch.uint8 and torch.equal(a.cpu(), b)
            t_e, m_e = select_masks_exact_kthvalue(dviews, k, None)
            assert t_e == t_ref and all(torch.equal(a.cpu(), b) for a, b in zip(m_e, m_ref))


@pytest.mark.parametrize("mode", ["balanced", "fast"])
def test_balanced_and_fast_tiers(dev, mode):
    from sga_amd.selection import HistogramSelect, TopkSelection
    from types import SimpleNamespace
    g = torch.Generator().manual_seed(5)
    views = [torch.randn(40001, generator=g), torch.full((7,), 0.25),
             torch.randn(65536, generator=g) * 3, torch.randn(100009, generator=g)]
    n_total = sum(v.numel() for v in views)
    k = SEL.k_for(n_total, 5.0)
    t_ref, m_ref = SEL.select_masks_histogram(views, k, mode=mode)
    t_dev, m_dev = HistogramSelect(mode).select([v.to(dev) for v in views], k, None)
    assert t_dev == t_ref
    for a, b in zip(m_dev, m_ref):
        assert torch.equal(a.cpu(), b)
    from sga_amd.config import set_args
    set_args(SimpleNamespace(sga_selection_method="histogram", sga_selection_ratio_percent=5.0,
                             sga_selection_histogram_mode=mode))
    sel = TopkSelection()
    masks = sel.select(SimpleNamespace(grad_views=[v.to(dev) for v in views]))
    assert sel.k_for(n_total) == k and sel.last_threshold == t_ref
    assert all(torch.equal(a.cpu(), b) for a, b in zip(masks, m_ref))


def test_replay_select_building_blocks(dev):
    from sga_amd import replay_kernels as K
    n = 250_007
    sc = student_t(n, 4).abs()
    sc[1000:1300] = sc[999]
    sd = sc.to(dev)
    hist, nf = K.hist_top16(sd)
    assert nf == 0 and hist.dtype == torch.int64 and hist.numel() == 32769
    top = SEL.abs_bit_top(sc)
    assert torch.equal(hist, torch.bincount(top, minlength=32769))
    b = int(top[999])
    cand = K.cand_extract(sd, b)
    assert torch.equal(cand, sc[top == b])
    th = float(sc[999])
    gt, eq, counts = K.gt_eq_counts(sd, th)
    assert gt.dtype == torch.bool and torch.equal(gt.cpu(), sc > th)
    assert torch.equal(eq.cpu(), sc == th)
    assert counts.tolist() == [int((sc > th).sum()), int((sc == th).sum())]
    # views that start off the 16-byte grid take the scalar paths of the same kernels
    for off in (1, 3):
        hv, _ = K.hist_top16(sd[off:])
        assert torch.equal(hv, torch.bincount(top[off:], minlength=32769))
        gv, ev, cv = K.gt_eq_counts(sd[off:], th)
        assert torch.equal(gv.cpu(), sc[off:] > th) and torch.equal(ev.cpu(), sc[off:] == th)
        assert cv.tolist() == [int((sc[off:] > th).sum()), int((sc[off:] == th).sum())]
    bad = sc.clone()
    bad[5] = float("nan")
    bad[6] = float("inf")
    assert K.hist_top16(bad.to(dev))[1] == 2
    assert K.arm(True, torch.float32) and not K.arm(False, torch.float32)
    assert K.formula("update") is not None and K.formula("nope") is None


def test_sampled_bracket_path_and_fallback(dev):
    """n >= 2^20 arms the sampled-bracket path; heavy-tailed data must take
    it (path == 1), tie-saturated data must fall back to the radix passes on
    the device (path == 0); both bit-exact vs the oracle."""
    from sga_amd import _lib as L
    from sga_amd.selection import read_result, select_exact_device
    n = (1 << 21) + 777
    gen = torch.Generator().manual_seed(99)
    fams = adversarial(n, gen)
    fams["student-t"] = student_t(n, 5).abs()
    fams["gauss"] = torch.randn(n, generator=gen).abs()
    seen = set()
    for name, sc in fams.items():
        sd = sc.to(dev)
        for k in sorted({1, n // 1000, n // 100, n // 10, n - 1}):
            m_ref, t_ref = SEL.select_topk_flat(sc, k)
            mask = torch.empty(n, dtype=torch.uint8, device=dev)
            res, _ = select_exact_device([sd], k, L.TIE_LOWEST_INDEX, masks=[mask])
            r = read_result(res)
            assert r.status == 0 and r.n_selected == k, (name, k, vars(r))
            assert r.thresh == t_ref, (name, k)
            assert torch.equal(mask.cpu().bool(), m_ref), (name, k)
            seen.add((name, r.path))
            # ties-all mode through the same path
            res2, (m2,) = select_exact_device([sd], k, L.TIE_ALL)
            assert torch.equal(m2.cpu().bool(), sc >= t_ref), (name, k)
    assert ("student-t", 1) in seen and ("gauss", 1) in seen
    assert ("all-equal", 0) in seen


def test_bracket_path_partial_ties(dev):
    """bf16-quantised magnitudes: the k-th value sits on a plateau of ties of
    which only the first few (by index) are selected, while the sampled
    bracket still holds -- the mask is settled from the sweep's bit planes
    and the candidate list."""
    from sga_amd import _lib as L
    from sga_amd.selection import read_result, select_exact_device
    n = (1 << 22) + 4321
    sc = student_t(n, 3).abs().to(torch.bfloat16).float()
    sd = sc.to(dev)
    partial = 0
    for k in (n // 1000, n // 100, n // 100 + 17, n // 10, n // 10 + 5, n // 3):
        m_ref, t_ref = SEL.select_topk_flat(sc, k)
        mask = torch.full((n,), 7, dtype=torch.uint8, device=dev)
        res, _ = select_exact_device([sd], k, L.TIE_LOWEST_INDEX, masks=[mask])
        r = read_result(res)
        assert r.status == 0 and r.n_selected == k and r.thresh == t_ref, (k, vars(r))
        assert torch.equal(mask.cpu().bool(), m_ref) and int(mask.max()) == 1, k
        partial += int(r.path == 1 and r.need < r.n_eq)
        res2, (m2,) = select_exact_device([sd], k, L.TIE_ALL)
        assert torch.equal(m2.cpu().bool(), sc >= t_ref), k
    assert partial >= 3


@pytest.mark.parametrize("x,reduce", [(4, "max"), (64, "max"), (1024, "max"), (8, "mean")])
def test_block_granular_selection(dev, x, reduce):
    from sga_amd.selection import HistogramSelect, block_reduce_views
    from sga_amd.support import block_idx_from_mask
    g = torch.Generator().manual_seed(x)
    views = [torch.randn(40001, generator=g), torch.randn(7, generator=g),
             torch.randn(65536, generator=g) * 3, torch.randn(100009, generator=g)]
    dviews = [v.to(dev) for v in views]
    n_total = sum(v.numel() for v in views)
    k = SEL.k_for(n_total, 5.0)
    bv_ref = SEL.block_reduce_views(views, x, reduce)
    bv_dev = block_reduce_views(dviews, x, reduce)
    for a, b in zip(bv_dev, bv_ref):
        if reduce == "max":
            assert torch.equal(a.cpu(), b)
        else:                      # fp32 summation order differs: tolerance class
            torch.testing.assert_close(a.cpu(), b, rtol=1e-6, atol=0)
    if reduce == "max":
        th_ref, m_ref = SEL.select_masks_blocks(views, k, x, reduce)
        th_dev, m_dev = HistogramSelect("exact", block_size=x, block_reduce=reduce).select(
            dviews, k, None)
        assert th_dev == th_ref
        for a, b in zip(m_dev, m_ref):
            assert torch.equal(a.cpu(), b)
        mask = torch.cat(m_ref)
    else:
        mask = (torch.rand(n_total, generator=g) < 0.01).to(torch.uint8)
    spans, off = [], 0
    for v in views:
        spans.append((off, off + v.numel()))
        off += v.numel()
    got = block_idx_from_mask(mask.to(dev), spans, x)
    assert got.dtype == torch.int32
    assert torch.equal(got.cpu(), SEL.block_idx_from_mask(mask, spans, x))
    # the block gather moves exactly the set bytes of every listed block
    from sga_amd.kernels import gather_selected_blocks, scatter_selected_blocks
    flat = torch.cat(views)
    vals = torch.empty(got.numel() * x, device=dev)
    gather_selected_blocks(flat.to(dev), mask.to(dev), got, vals, x, 1.0)
    dst = torch.zeros(n_total, device=dev)
    scatter_selected_blocks(dst, mask.to(dev), got, vals, x)
    assert torch.equal(dst.cpu(), torch.where(mask.bool(), flat, torch.zeros(())))


def test_adaptive_threshold_masks(dev):
    from sga_amd.selection import adapt_threshold, threshold_masks
    g = torch.Generator().manual_seed(11)
    views = [torch.randn(100_003, generator=g), torch.randn(5, generator=g),
             torch.randn(65_536, generator=g) * 2]
    views[0][7] = float("nan")
    tau = 1.25
    masks, cnt = threshold_masks([v.to(dev) for v in views], tau)
    ref = [(v.abs() >= tau).to(torch.uint8) for v in views]
    for a, b in zip(masks, ref):
        assert torch.equal(a.cpu(), b)
    assert cnt == sum(int(m.sum()) for m in ref)
    big = torch.randn(1_000_003, generator=g)          # several trips of the unrolled loop, ragged end
    for off in (0, 1):
        mk, c = threshold_masks([big.to(dev)[off:]], tau)
        assert torch.equal(mk[0].cpu(), (big[off:].abs() >= tau).to(torch.uint8))
        assert c == int((big[off:].abs() >= tau).sum())
    assert adapt_threshold(2.0, 0.105, 0.10) == 2.0
    assert adapt_threshold(2.0, 0.4, 0.10) == 2.0 * 1.15
    assert abs(adapt_threshold(2.0, 0.12, 0.10, band=0.0) - 2.0 * 1.2 ** 0.5) < 1e-12


def test_adaptive_tau_trajectory_matches_oracle(dev):
    """Bootstrap, gated warmup, tau feedback and collapse re-bootstrap over a
    drifting gradient scale: thresholds, masks and controller state track
    the oracle's state machine cycle by cycle."""
    from types import SimpleNamespace

    from oracle import select as OS
    from sga_amd.config import set_args
    from sga_amd.selection import TopkSelection
    set_args(SimpleNamespace(sga_selection_method="adaptive", sga_selection_ratio_percent=10.0,
                             sga_selection_adaptive_warmup_syncs=2,
                             sga_selection_adaptive_warmup_mode="fast"))
    sel = TopkSelection()
    ref = OS.AdaptiveTau(10.0, 2, "fast")
    assert sel.warmup_sync_target(0, 4) == ref.warmup_sync_target(0, 4) == 1
    gen = torch.Generator().manual_seed(5)
    scales = [1.0, 1.0, 1.0, 1.3, 1.3, 0.7, 0.7, 1e-6, 1.0, 1.0]
    for cyc, sc in enumerate(scales):
        grads = [torch.randn(50_000, generator=gen) * sc, torch.randn(1_237, generator=gen) * sc]
        k = OS.k_for(51_237, 10.0)
        thr_r, m_r = ref.select(grads, k, 2)
        ctx = SimpleNamespace(grad_views=[g.to(dev) for g in grads], comm_group=None,
                              warmup_target=2)
        m_d = sel.select(ctx)
        assert sel.last_threshold == thr_r, (cyc, sel.last_threshold, thr_r)
        assert sel.tau == ref.tau and sel.warmup_passed == ref.warmup_passed, cyc
        for a, b in zip(m_d, m_r):
            assert torch.equal(a.cpu(), b), cyc
    # zero-tau latch re-bootstraps to the smallest positive bin edge
    sel._impl.tau = 0.0
    sel._impl.warmup_passed = 5
    sel.select(SimpleNamespace(grad_views=[torch.zeros(64, device=dev)], comm_group=None,
                               warmup_target=0))
    assert sel.tau == OS.bin_edge_float(1, 19)


def test_adjacent_views_take_the_flat_path(dev):
    """Per-param views that are back-to-back slices of one buffer are selected
    as one flat array (one sweep) in place; scattered tensors are staged into
    one buffer first.  Both give the oracle's masks; explicit mask buffers keep
    the per-view passes, which must agree too."""
    from sga_amd import _lib as L
    from sga_amd.selection import read_result, select_exact_device, select_masks_histogram
    sizes = [300_001, 7, 1 << 20, 65_536, 1023]
    n = sum(sizes)
    flat = student_t(n, 4).to(torch.bfloat16).float()          # quantised: ties at the cut
    buf = flat.to(dev)
    views, clones, off = [], [], 0
    for s in sizes:
        views.append(buf[off:off + s])
        clones.append(buf[off:off + s].clone())
        off += s
    for k in (n // 1000, n // 100, n // 7):
        for tie in (L.TIE_LOWEST_INDEX, L.TIE_ALL):
            ra, ma = select_exact_device(views, k, tie)
            rb, mb = select_exact_device(clones, k, tie)
            a, b = read_result(ra), read_result(rb)
            assert a.path == 1 and b.path == 1             # both end up as one flat sweep
            assert (a.thresh_bits, a.n_selected) == (b.thresh_bits, b.n_selected)
            for x, y in zip(ma, mb):
                assert torch.equal(x, y)
        m_ref, t_ref = SEL.select_topk_flat(flat.abs(), k)
        assert torch.equal(torch.cat(select_exact_device(views, k, L.TIE_LOWEST_INDEX)[1]).cpu().bool(),
                           m_ref)
        own = [torch.empty(s, dtype=torch.uint8, device=dev) for s in sizes]
        rc, mc = select_exact_device(clones, k, L.TIE_LOWEST_INDEX, masks=own)
        assert read_result(rc).path == 0 and torch.equal(torch.cat(mc).cpu().bool(), m_ref)
        th, masks = select_masks_histogram(views, k, mode="exact")
        assert th == t_ref and torch.equal(torch.cat(masks).cpu().bool(), flat.abs() >= t_ref)


@pytest.mark.parametrize("n", [1000, 300_000, (1 << 20) + 4097, 3_000_001])
def test_negative_score_is_rejected_by_the_select_itself(dev, n):
    """``sga/replay.py:545-547`` rejects a score below zero.  The select's own
    sweep reports it (no extra pass): one negative anywhere, first / last /
    mid element, in an aligned or a scalar-path view, on the radix path (small
    n) and the one-sweep path (n >= 2^20).  -0.0 is not negative there
    (``(t < 0).any()``), and is not here."""
    from sga_amd.replay import select_topk_flat
    base = student_t(n, 11 + n).abs()
    k = max(1, n // 100)
    for pos in (0, n // 2 + 1, n - 1):
        t = base.clone()
        t[pos] = -1.0e-30
        with pytest.raises(ValueError, match="non-negative"):
            select_topk_flat(t.to(dev), k)
        with pytest.raises(ValueError, match="non-negative"):
            select_topk_flat(torch.cat([torch.zeros(1), t]).to(dev)[1:], k)
        select_topk_flat(t.to(dev), k, check=False)      # the unchecked form ranks magnitudes
    t = base.clone()
    t[n // 3] = -0.0
    m_ref, t_ref = SEL.select_topk_flat(t, k)
    m_dev, t_dev = select_topk_flat(t.to(dev), k)
    assert t_dev == t_ref and torch.equal(m_dev.cpu(), m_ref)
