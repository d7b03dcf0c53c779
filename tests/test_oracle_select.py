"""Pins the selection oracle against the reference's known-answer vectors
(tests/golden/select_kats.json), torch.kthvalue, and a stable sort."""
import json
import os

import pytest
import torch

from oracle import kernels as OK
from oracle import select as SEL

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                   "select_kats.json")))


def _f(x):
    return float(x)


def adversarial(n, gen):
    """Tie-heavy families of tests/test_replay_fused.py:2059-2074 (shape of
    the data, regenerated here with our own generator)."""
    plateau = torch.ones(n)
    plateau[: int(0.4 * n)] = 2.0
    npos = max(8, n // 1000)
    zh = torch.zeros(n)
    zh[:npos] = torch.rand(npos, generator=gen) + 0.5
    return {
        "all-equal": torch.full((n,), 1.0),
        "boundary-plateau": plateau,
        "quantized": torch.rand(n, generator=gen).mul(1000).round().div(1000),
        "zero-heavy": zh,
        "uniform": torch.rand(n, generator=gen) + 1e-6,
    }


def sort_topk_mask(t, k):
    """Independent statement of the contract: stable descending sort, the
    first k win (ties therefore go to the lowest index)."""
    order = torch.sort(t, descending=True, stable=True).indices
    m = torch.zeros(t.numel(), dtype=torch.bool)
    m[order[:k]] = True
    return m


@pytest.mark.parametrize("kat", KATS["tie_fill"], ids=lambda k: k["name"])
def test_tie_fill_kats(kat):
    t = torch.tensor(kat["t"], dtype=torch.float32)
    mask, th = SEL.select_topk_flat(t, kat["k"])
    assert mask.to(torch.int64).tolist() == kat["mask"]
    assert th == kat["thresh"]


@pytest.mark.parametrize("kat", KATS["rejections"])
def test_rejections(kat):
    t = torch.tensor([_f(x) for x in kat["t"]], dtype=torch.float32)
    with pytest.raises(ValueError) as ei:
        SEL.select_topk_flat(t, kat["k"])
    assert kat["substr"] in str(ei.value)


def test_injected_tie_layer_random():
    g = torch.Generator().manual_seed(8)
    t = torch.rand(200, generator=g)
    k = 50
    v = float(torch.kthvalue(t, t.numel() - k + 1).values)
    t[100:160] = v
    mask, th = SEL.select_topk_flat(t, k)
    assert th == v
    assert torch.equal(mask, sort_topk_mask(t, k))
    t7 = torch.rand(7, generator=g)
    mask, th = SEL.select_topk_flat(t7, 7)
    assert bool(mask.all()) and th == float(t7.min())


def test_exact_k_equals_stable_sort_on_adversarial_sets():
    gen = torch.Generator().manual_seed(20260912)
    n = 20000
    for name, sc in adversarial(n, gen).items():
        for k in sorted({1, n // 100, 3 * n // 10, n - 1, n, 10, 80}):
            mask, th = SEL.select_topk_flat(sc, k)
            assert int(mask.sum()) == k
            assert th == float(torch.kthvalue(sc, n - k + 1).values), name
            assert torch.equal(mask, sort_topk_mask(sc, k)), (name, k)


def test_threshold_is_kthvalue_all_distributions():
    """Distribution families of tests/test_xp_capability.py:61-91."""
    N = 4097
    g = torch.Generator().manual_seed(1234)
    ds = [torch.randn(N, generator=g) * 1e-3,
          (torch.randn(N, generator=g) * 1e3).round() / 1e3,
          torch.randn(N, generator=g).exp() * torch.sign(torch.randn(N, generator=g)),
          torch.full((N,), 0.5),
          torch.randn(N, generator=g) * 1e-3,
          torch.randn(N, generator=g) * 1e-3]
    ds[4][::3] = 0.0
    ds[5][::7] *= 1e30
    for x in ds:
        views = [x[:N // 2].contiguous(), x[N // 2:].contiguous()]
        for k in (1, 2, N // 10, N // 2, N - 1, N):
            ref = torch.kthvalue(x.abs(), N - k + 1).values.item()
            assert SEL.select_threshold_views(views, k) == ref
            th, masks = SEL.select_masks_histogram(views, k, mode="exact")
            te, me = SEL.select_masks_exact_kthvalue(views, k)
            assert th == ref == te
            for gv, m, m2 in zip(views, masks, me):
                assert torch.equal(m, (gv.abs() >= ref).to(torch.uint8))
                assert torch.equal(m, m2)
            assert sum(int(m.sum()) for m in masks) >= k


def test_balanced_closed_form_and_edges():
    g = torch.Generator().manual_seed(5)
    views = [torch.randn(40001, generator=g), torch.full((7,), 0.25),
             torch.randn(65536, generator=g) * 3, torch.randn(100009, generator=g)]
    n_total = sum(v.numel() for v in views)
    k = SEL.k_for(n_total, 5.0)
    th, masks = SEL.select_masks_histogram(views, k, mode="balanced")
    bits = torch.tensor(th, dtype=torch.float32).view(torch.int32).item()
    assert bits & 0xFFFF == 0
    # brute-force restatement of the integer closed form
    keys = torch.cat([SEL.abs_bit_top(v)[::8] for v in views]).tolist()
    keys.sort()
    n_s = len(keys)
    r = max(1, round(n_s * (n_total - k + 1) / n_total))
    b = keys[r - 1]              # smallest bin whose cumulative count >= r
    assert bits >> 16 == b
    n_sel = sum(int(m.sum()) for m in masks)
    n_exact = sum(int(m.sum()) for m in SEL.select_masks_histogram(views, k)[1])
    assert abs(n_sel - n_exact) / n_total < 0.005
    th_f, m_f = SEL.select_masks_histogram(views, k, mode="fast")
    bits_f = torch.tensor(th_f, dtype=torch.float32).view(torch.int32).item()
    assert bits_f & 0x7FFFF == 0
    # replay twin with p_off = 0 is the same mask
    flat = torch.cat(views).abs()
    ent, off = [], 0
    for v in views:
        ent.append({"a": off, "n": v.numel(), "p_off": 0})
        off += v.numel()
    m2, t2 = SEL.shard_select_balanced(flat, k, ent)
    assert t2 == th and torch.equal(m2.to(torch.uint8), torch.cat(masks))


def test_shard_select_balanced_param_relative_phase():
    """The replay twin on shard slices that start inside a parameter
    (``p_off`` != 0, replay_fused.py:420-432): the sample keeps the
    parameter's own stride-8 grid, i.e. local element j is sampled when
    ``(p_off + j) % 8 == 0``.  Brute force from that wording, on the geometry
    fixture of tests/test_selection_semantics_switch.py:176-186 (sizes 40001,
    7, 65536, 100009, a constant middle view)."""
    sizes, p_offs = [40001, 7, 65536, 100009], [3, 13, 0, 8 * 1000 + 5]
    gen = torch.Generator().manual_seed(7)
    score = torch.rand(sum(sizes), generator=gen) ** 4
    ent, off = [], 0
    for sz, po in zip(sizes, p_offs):
        ent.append({"a": off, "n": sz, "p_off": po})
        off += sz
    score[ent[2]["a"]:ent[2]["a"] + sizes[2]] = 0.25           # one constant view
    n = score.numel()
    top = SEL.abs_bit_top(score)
    for k in (1, n // 100, 3 * n // 10, n - 1):
        sample = []
        for e in ent:
            sample += [int(top[e["a"] + j]) for j in range(e["n"]) if (e["p_off"] + j) % 8 == 0]
        sample.sort()
        r = max(1, round(len(sample) * (n - k + 1) / n))
        mask, th = SEL.shard_select_balanced(score, k, ent)
        assert torch.equal(mask, top >= sample[r - 1]), k
        bits = torch.tensor(th, dtype=torch.float32).view(torch.int32).item()
        assert bits == sample[r - 1] << 16


@pytest.mark.parametrize("kat", KATS["k_for"])
def test_k_formulas(kat):
    assert SEL.k_for(kat["n"], kat["ratio"]) == kat["k"]
    assert SEL.replay_k(kat["n"], kat["ratio"]) == kat["k"]


def test_k_bankers_rounding():
    assert SEL.k_for(250, 1.0) == 2      # 2.5 -> 2
    assert SEL.k_for(350, 1.0) == 4      # 3.5 -> 4
    assert SEL.k_for(10, 0.001) == 1     # floor at 1


def test_compact_mask_kats():
    for kat in KATS["compact_mask"]:
        m = torch.tensor(kat["mask"], dtype=torch.uint8)
        idx = OK.compact_mask_u8(m)
        assert idx.dtype == torch.int32 and idx.tolist() == kat["idx"]
        assert int(torch.searchsorted(idx, m.numel() // 2)) == kat["split_at_mid"]
    g = torch.Generator().manual_seed(4)
    m = (torch.rand(300000, generator=g) < 0.4).to(torch.uint8)
    assert OK.compact_mask_u8(m).tolist() == [i for i, b in enumerate(m.tolist()) if b]


def test_layout_oracles_against_element_loops():
    """The two sparse-sync layouts of the oracle against plain Python loops on
    small inputs: mask layout = per slice [i*(n//s), ...) the set coordinates
    in index order times factor, written back in place; index layout = gather,
    scale, zero, with the bucket-midpoint split for two slices (the KAT's
    split_at_mid) and the even split otherwise."""
    g = torch.Generator().manual_seed(9)
    for n, s in ((11, 2), (11, 3), (10, 1), (7, 4), (1, 2)):
        grad = torch.randn(n, generator=g)
        mask = (torch.rand(n, generator=g) < 0.5).to(torch.uint8)
        cuts = [i * (n // s) for i in range(s)] + [n]
        want = [[grad[i].item() * 0.5 for i in range(a, b) if mask[i]]
                for a, b in zip(cuts[:-1], cuts[1:])]
        got = OK.mask_layout_pack(grad, mask, 0.5, s)
        assert [p.tolist() for p in got] == want
        back = torch.zeros(n)
        OK.mask_layout_unpack(back, mask, got, s)
        assert back.tolist() == [grad[i].item() * 0.5 if mask[i] else 0.0 for i in range(n)]
        idx = OK.compact_mask_u8(mask)
        k = idx.numel()
        bounds = OK.index_layout_bounds(idx, n, s)
        if s == 2:
            n0 = sum(1 for i in idx.tolist() if i < n // 2)
            assert bounds == [(0, n0), (n0, k)]
        else:
            assert bounds == [(i * k // s, (i + 1) * k // s) for i in range(s)]
        g2, vals = grad.clone(), torch.empty(k)
        assert OK.index_layout_pack(g2, idx, vals, 0.5, s) == bounds
        assert vals.tolist() == [grad[i].item() * 0.5 for i in idx.tolist()]
        assert g2.tolist() == [0.0 if mask[i] else grad[i].item() for i in range(n)]
    kat = KATS["compact_mask"][0]
    idx = torch.tensor(kat["idx"], dtype=torch.int32)
    assert OK.index_layout_bounds(idx, len(kat["mask"]), 2)[0][1] == kat["split_at_mid"]


def test_block_helpers_kats():
    """Literal block KATs: ANY rule, short tail blocks, x == 1 == compaction."""
    m = torch.tensor([0, 1, 0, 0, 0, 0, 1, 1, 0, 0, 1], dtype=torch.uint8)
    assert SEL.block_idx_from_mask(m, [(0, 6), (6, 11)], 4).tolist() == [0, 6, 10]
    assert SEL.block_idx_from_mask(m, [(0, 11)], 1).tolist() == OK.compact_mask_u8(m).tolist()
    g = torch.tensor([1.0, -3.0, 2.0, 0.0, 5.0])
    assert SEL.block_reduce_views([g], 2, "max")[0].tolist() == [3.0, 2.0, 5.0]
    assert SEL.block_reduce_views([g], 2, "mean")[0].tolist() == [2.0, 1.0, 5.0]
    th, masks = SEL.select_masks_blocks([g], 2, 2, "max")
    assert masks[0].tolist() == [0, 0, 0, 0, 1] and th == 5.0


def test_adaptive_threshold_reference_vectors():
    # known answers held by the reference's own unit test
    # (tests/test_plugins_unit.py:603-616)
    f = SEL.adapt_threshold
    assert f(1.0, 0.105, 0.10) == 1.0 and f(1.0, 0.095, 0.10) == 1.0
    assert f(1.0, 0.13, 0.10) == 1.3 ** 0.5
    assert f(1.0, 0.085, 0.10) == 0.85 ** 0.5
    assert f(1.0, 0.20, 0.10) == 1.15
    assert f(1.0, 0.0001, 0.10) == 0.9


def test_adaptive_warmup_anchor_reference_vectors():
    # tests/test_plugins_unit.py:346-362
    a = SEL.AdaptiveTau(40.0, 5, "fast")
    assert a.warmup_sync_target(0, 4) == 4
    assert a.warmup_sync_target(6, 4) == (20 - 1 - 6) // 4
    assert a.warmup_sync_target(25, 4) == 0
    assert SEL.AdaptiveTau(40.0, None, "fast").warmup_sync_target(0, 4) is None


def test_adaptive_lifecycle_oracle():
    # the phases the reference's lifecycle test walks
    # (tests/test_plugins_unit.py:619-677)
    torch.manual_seed(12)
    grads = [torch.randn(4096), torch.randn(1000)]
    k = SEL.k_for(5096, 10.0)
    a = SEL.AdaptiveTau(10.0, None, "fast")
    thr, _ = a.select(grads, k, 3)
    bits = torch.tensor(thr, dtype=torch.float32).view(torch.int32).item()
    assert bits & ((1 << 19) - 1) == 0 and a.tau == thr and a.warmup_passed in (0, 1)
    a.warmup_passed = 0
    thr, _ = a.select(grads, k, 3)
    assert a.tau == thr
    a.warmup_passed = 3
    tau = a.tau
    thr, masks = a.select(grads, k, 3)
    assert thr == tau
    for g, m in zip(grads, masks):
        assert torch.equal(m, (g.abs() >= tau).to(torch.uint8))
    a.tau = 1e30
    _, masks = a.select(grads, k, 3)
    assert a.tau < 1e30 and any(int(m.sum()) for m in masks)
    # zero-tau latch: an all-zero input bootstraps to bin 0 -> floor edge
    a.warmup_passed = 5
    a.tau = 0.0
    a.select([torch.zeros(64)], 6, 0)
    assert a.tau == SEL.bin_edge_float(1, 19) and a.tau > 0.0
