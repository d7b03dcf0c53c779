"""GPU parity of the fused per-rank sparse step vs the CPU oracle driver on
the same seeded inputs, every output bit for bit: threshold, idx, mask,
values, residual, m, v and p -- for the Adam-normalised scores too (the oracle
selects on its own scores; the device evaluates the same correctly rounded
chain)."""
import pytest
import torch

from oracle import fused_step as OF
from oracle import select as SEL
from tests.util import same_bits, student_t

pytestmark = pytest.mark.gpu


def _segments(sizes, wd_every=2, vary=False):
    segs, off = [], 0
    for i, s in enumerate(sizes):
        seg = dict(start=off, n=s, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8,
                   wd=0.1 if i % wd_every == 0 else 0.0)
        if vary:     # every hyper-parameter changes from tensor to tensor
            seg.update(lr=1e-4 * (1 + i % 3), b1=(0.9, 0.8, 0.95)[i % 3], b2=(0.95, 0.99)[i % 2],
                       eps=(1e-8, 1e-6, 1e-10)[(i + 1) % 3])
        segs.append(seg)
        off += s
    return segs, off


def _run(dev, sizes, steps, ratio, gdtype, vdtype, score="abs_g", seed0=0, vary=False,
         expect_path=None, **knobs):
    from sga_amd.fused_step import FusedSparseStep
    segs, n = _segments(sizes, vary=vary)
    gen = torch.Generator().manual_seed(1234)
    p = torch.randn(n, generator=gen) * 0.02
    m, v, r = torch.zeros(n), torch.zeros(n), torch.zeros(n)
    dp, dm, dv, dr = (t.to(dev) for t in (p, m, v, r))
    fs = FusedSparseStep(n, segs, dev, values_dtype=vdtype, want_mask=True)
    k = SEL.k_for(n, ratio)
    for step in range(1, steps + 1):
        g = student_t(n, seed0 + step - 1).to(gdtype)
        idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
            g, r, p, m, v, segs, step, k=k, score=score, values_dtype=vdtype, **knobs)
        idx, vals = fs.step(g.to(dev), dr, dp, dm, dv, step, k=k, score=score, **knobs)
        res = fs.read_result()
        assert res.status == 0 and res.nonfinite == 0 and res.n_selected == k
        assert expect_path is None or res.path == expect_path
        assert res.thresh == th_ref, (step, res.thresh, th_ref)
        assert torch.equal(idx.cpu(), idx_ref), step
        assert torch.equal(fs.mask.cpu().bool(), mask_ref), step
        it = torch.int16 if vdtype == torch.bfloat16 else torch.int32
        assert torch.equal(vals.cpu().view(it), val_ref.view(it)), step
        # the device state is never re-synchronised from the oracle between steps
        assert same_bits(dr, r) and same_bits(dm, m) and same_bits(dv, v), step
        assert same_bits(dp, p), step
    return n, k


def test_config1_flat_fp32_8_steps(dev):
    """2^22 fp32 Student-t(3)x1e-3 gradients, 8 seeded steps, ratio 1 %."""
    n, k = _run(dev, [1 << 22], 8, 1.0, torch.float32, torch.float32)
    assert k == 41943


def test_bf16_grads_bf16_values_multi_segment(dev):
    _run(dev, [400_000, 1024, 300_000, 128, 170_000, 2048], 4, 1.0, torch.bfloat16,
         torch.bfloat16)


@pytest.mark.parametrize("ratio", [0.1, 10.0])
def test_ratios(dev, ratio):
    _run(dev, [1_000_003], 3, ratio, torch.bfloat16, torch.bfloat16)


def test_ragged_unaligned_segments(dev):
    _run(dev, [1001, 7, 2999, 64_001], 3, 1.0, torch.float32, torch.bfloat16)


@pytest.mark.parametrize("score", ["update", "coi", "abs_m"])
def test_adam_normalised_scores(dev, score):
    _run(dev, [200_000, 1024, 100_000], 3, 1.0, torch.bfloat16, torch.bfloat16, score=score)


@pytest.mark.parametrize("score", ["update", "coi"])
def test_adam_scores_one_sweep_path_tensor_boundaries(dev, score):
    """Above 2^20 elements the select is the one-sweep path, which scores a
    256-element slab once per tensor that intersects it: tensors of 3..130
    elements put several boundaries into one slab, none of them aligned, and
    every hyper-parameter differs between neighbours."""
    sizes = [300_000, 128, 37, 700_000, 3, 1024, 250_001, 130, 5, 60_000]
    _run(dev, sizes, 2, 1.0, torch.bfloat16, torch.bfloat16, score=score, vary=True,
         expect_path=1)


@pytest.mark.parametrize("score", ["abs_g", "update", "coi"])
@pytest.mark.parametrize("knobs", [dict(optimizer="adams"),
                                   dict(optimizer="adamw", fold=True, interval=4.0),
                                   dict(optimizer="adams", fold=True, interval=3.0, coeff=0.5)])
def test_adams_and_fold_knobs(dev, score, knobs):
    """The fused step under AdamS (v rebuilt from the pre-commit m, no bias
    corrections: adams.py:87-213; the Adam-normalised scores through v := m*m,
    bc := 1: replay.py:486-505), with the residual-mean fold of the new
    residual (true division, adamw_torch.py:88-91; interval 3 is not a power
    of two) and a clip coefficient, below and above the one-sweep select's
    size, every output bit for bit over several steps."""
    _run(dev, [200_000, 1024, 100_000], 3, 1.0, torch.bfloat16, torch.bfloat16, score=score,
         **knobs)
    _run(dev, [600_000, 130, 37, 500_000, 3, 1024, 100_001], 2, 1.0, torch.float32, torch.float32,
         score=score, vary=True, expect_path=1, **knobs)


@pytest.mark.parametrize("opt", ["adamw", "adams"])
@pytest.mark.parametrize("score", ["abs_g_blind", "abs_gr_over_sqrt_v"])
def test_benchmark_scores_outside_the_registry(dev, score, opt):
    """The two build-side benchmark scores (the residual-blind |g| and the
    literal |g + r| / sqrt(v + eps)): NO reference implementation exists, so
    their parity is UNPINNED -- the device is compared with the closed form
    restated on the CPU (one fp32 add, a correctly rounded root, one divide),
    bit for bit, through the same exact-k selection, pack and commit."""
    _run(dev, [200_000, 1024, 100_000], 3, 1.0, torch.bfloat16, torch.bfloat16, score=score,
         optimizer=opt)
    _run(dev, [600_000, 130, 37, 500_000, 3, 1024, 100_001], 3, 10.0, torch.float32, torch.float32,
         score=score, vary=True, expect_path=1, optimizer=opt)


def test_fused_step_refuses_dual_lr_and_unknown_flags(dev):
    from sga_amd import _lib as L
    from sga_amd.fused_step import FusedSparseStep
    segs, n = _segments([4096])
    fs = FusedSparseStep(n, segs, dev)
    z = torch.zeros(n, device=dev)
    with pytest.raises(ValueError, match="requires a full step"):
        fs.step(z, z.clone(), z.clone(), z.clone(), z.clone(), 1, k=4, inactive_lr_scale=0.5)
    with pytest.raises(ValueError, match="interval"):
        fs.step(z, z.clone(), z.clone(), z.clone(), z.clone(), 1, k=4, fold=True, interval=0.0)
    lib = L.load()
    rc = lib.sga_fused_sparse_step(L.ptr(z), 0, L.ptr(z), L.ptr(z), L.ptr(z), L.ptr(z), n, 4,
                                   L.ptr(fs._seg_dev), 1, 1, L.ptr(fs.idx), L.ptr(fs.values), 1,
                                   None, 1.0, 1.0, 1, L.GC_LR_SPLIT, 1.0, None, L.ptr(fs.ws),
                                   fs.ws_bytes, L.stream())
    assert rc == -1 and b"requires a full step" in lib.sga_last_error()


def test_tie_heavy_gradients(dev):
    """Quantised gradients: many equal magnitudes at the threshold; ties must
    go to the lowest flat indices exactly like the oracle."""
    from sga_amd.fused_step import FusedSparseStep
    n = 500_000
    segs, _ = _segments([n])
    gen = torch.Generator().manual_seed(7)
    g = (torch.randn(n, generator=gen) * 4).round() / 1024
    p = torch.randn(n, generator=gen) * 0.02
    m, v, r = torch.zeros(n), torch.zeros(n), torch.zeros(n)
    dp, dm, dv, dr = (t.to(dev) for t in (p, m, v, r))
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, want_mask=True)
    for k in (1, 5000, 250_000, n):
        rr, pp, mm, vv = r.clone(), p.clone(), m.clone(), v.clone()
        idx_ref, val_ref, mask_ref, th = OF.fused_sparse_step(g, rr, pp, mm, vv, segs, 1, k=k)
        er, ep, em, ev = (t.clone() for t in (dr, dp, dm, dv))
        idx, vals = fs.step(g.to(dev), er, ep, em, ev, 1, k=k)
        assert fs.read_result().thresh == th
        assert torch.equal(idx.cpu(), idx_ref) and torch.equal(vals.cpu(), val_ref)
        assert torch.equal(er.cpu(), rr) and torch.equal(em.cpu(), mm)


def test_fast_and_radix_paths_agree(dev):
    """Same inputs through the sampled-bracket path and the plain radix
    passes: identical idx / values / state, and the fast path is really taken."""
    from sga_amd.fused_step import FusedSparseStep
    n = (1 << 21) + 4099
    segs, _ = _segments([1 << 20, 4099, 1 << 20])
    gen = torch.Generator().manual_seed(3)
    base = [torch.randn(n, generator=gen) * 0.02, torch.zeros(n), torch.zeros(n),
            student_t(n, 8) * 0.3]
    g = student_t(n, 9).to(torch.bfloat16).to(dev)
    outs = []
    for fast in (True, False):
        p, m, v, r = (t.to(dev).clone() for t in base)
        fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, want_mask=True)
        idx, vals = fs.step(g, r, p, m, v, 3, ratio_percent=1.0, fast=fast)
        res = fs.read_result()
        assert res.path == (1 if fast else 0) and res.status == 0
        outs.append((idx.clone(), vals.clone(), p, m, v, r, fs.mask.clone(), res.thresh))
    for a, b in zip(outs[0][:-1], outs[1][:-1]):
        assert torch.equal(a, b)
    assert outs[0][-1] == outs[1][-1]


@pytest.mark.parametrize("score,gdtype", [("abs_g", torch.bfloat16), ("update", torch.float32),
                                          ("abs_m", torch.bfloat16)])
def test_packed_state_is_bitwise_the_separate_layout(dev, score, gdtype):
    """The packed-state entry point runs the same arithmetic on interleaved
    64 KiB records: after unpacking, every output equals the separate-array
    entry point's bit for bit, over several steps, ragged sizes, both select
    paths (n below and above the sampled-bracket cut-in)."""
    from sga_amd.fused_step import FusedSparseStep, PackedState
    for sizes in ([4097, 3, 12_289, 1000], [1 << 20, 4099, (1 << 20) + 5]):
        segs, n = _segments(sizes)
        gen = torch.Generator().manual_seed(5)
        p0 = (torch.randn(n, generator=gen) * 0.02).to(dev)
        m0 = (torch.randn(n, generator=gen) * 1e-3).to(dev)
        v0 = (torch.rand(n, generator=gen) * 1e-5).to(dev)
        r0 = (student_t(n, 77) * 0.1).to(dev)
        p, m, v, r = (t.clone() for t in (p0, m0, v0, r0))
        st = PackedState(n, dev).pack(r0, p0, m0, v0)
        back = [torch.empty(n, device=dev) for _ in range(4)]
        st.unpack(*back)
        for a, b in zip(back, (r0, p0, m0, v0)):
            assert torch.equal(a, b)
        fa = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, want_mask=True)
        fb = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, want_mask=True)
        for step in range(1, 4):
            g = student_t(n, 100 + step).to(gdtype).to(dev)
            ia, va = fa.step(g, r, p, m, v, step, ratio_percent=1.0, score=score)
            ib, vb = fb.step_packed(g, st, step, ratio_percent=1.0, score=score)
            ra, rb = fa.read_result(), fb.read_result()
            assert (ra.thresh_bits, ra.need, ra.n_selected, ra.path) == \
                (rb.thresh_bits, rb.need, rb.n_selected, rb.path)
            assert torch.equal(ia, ib) and torch.equal(va.view(torch.int16), vb.view(torch.int16))
            assert torch.equal(fa.mask, fb.mask)
            st.unpack(*back)
            for a, b in zip(back, (r, p, m, v)):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (sizes, step)
    with pytest.raises(ValueError):
        fb.step_packed(g, PackedState(n + 1, dev), 1, ratio_percent=1.0)


@pytest.mark.parametrize("seed", range(8))
def test_randomized_configurations(dev, seed):
    """Seeded random draws of everything at once: tensor sizes (1 .. 700k
    elements, shuffled), per-tensor hyper-parameters (beta1 = 0 and eps = 1e-15
    included), score, gradient / value dtypes, ratio, and the magnitude of the
    gradients, moments and residual (1e-12 .. 10, some all zero), optimizer
    (AdamW / AdamS), fold and clip coefficient -- three steps each, every
    output bit for bit."""
    import random
    from sga_amd.fused_step import FusedSparseStep
    rng = random.Random(seed)
    total = rng.choice([70_001, 300_000, 1_100_000, 1_300_003])
    sizes, left = [], total
    while left > 0:
        sz = min(left, rng.choice([1, 3, 37, 128, 130, 1000, 1024, 4099, 50_000, 300_001, 700_000]))
        sizes.append(sz)
        left -= sz
    rng.shuffle(sizes)
    score = ["abs_g", "update", "coi", "abs_m"][seed % 4]
    gdtype = rng.choice([torch.bfloat16, torch.float32])
    vdtype = rng.choice([torch.bfloat16, torch.float32])
    gscale = 10.0 ** rng.uniform(-12, 1)
    segs, off = [], 0
    for sz in sizes:
        segs.append(dict(start=off, n=sz, lr=10 ** rng.uniform(-5, -2),
                         b1=rng.choice([0.9, 0.8, 0.95, 0.0]), b2=rng.choice([0.95, 0.99, 0.999]),
                         eps=rng.choice([1e-8, 1e-6, 1e-10, 1e-15]), wd=rng.choice([0.0, 0.1, 0.01])))
        off += sz
    n = off
    gen = torch.Generator().manual_seed(1000 + seed)
    p = torch.randn(n, generator=gen) * 0.02
    m = torch.randn(n, generator=gen) * gscale * rng.choice([0.0, 1.0, 1e-3])
    v = torch.rand(n, generator=gen) * gscale * gscale * rng.choice([0.0, 1.0, 1e-6])
    r = torch.randn(n, generator=gen) * gscale * rng.choice([0.0, 1.0])
    dp, dm, dv, dr = (t.to(dev) for t in (p, m, v, r))
    fs = FusedSparseStep(n, segs, dev, values_dtype=vdtype, want_mask=True)
    k = SEL.k_for(n, rng.choice([0.1, 1.0, 10.0]))
    knobs = dict(optimizer=rng.choice(["adamw", "adams"]), fold=rng.choice([False, True]),
                 interval=rng.choice([2.0, 3.0, 16.0]), coeff=rng.choice([1.0, 0.37]))
    for step in range(1, 4):
        g = (student_t(n, seed * 10 + step) * (gscale / 1e-3)).to(gdtype)
        idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
            g, r, p, m, v, segs, step, k=k, score=score, values_dtype=vdtype, **knobs)
        idx, vals = fs.step(g.to(dev), dr, dp, dm, dv, step, k=k, score=score, **knobs)
        res = fs.read_result()
        assert res.status == 0 and res.thresh == th_ref, (step, res.thresh, th_ref)
        assert torch.equal(idx.cpu(), idx_ref) and torch.equal(fs.mask.cpu().bool(), mask_ref), step
        it = torch.int16 if vdtype == torch.bfloat16 else torch.int32
        assert torch.equal(vals.cpu().view(it), val_ref.view(it)), step
        assert same_bits(dr, r) and same_bits(dm, m) and same_bits(dv, v) and same_bits(dp, p), step


@pytest.mark.parametrize("score,vdtype,knobs", [("abs_g", torch.float32, {}),
                                                ("update", torch.bfloat16, {}),
                                                ("coi", torch.bfloat16, dict(optimizer="adams")),
                                                ("abs_g", torch.bfloat16,
                                                 dict(fold=True, interval=3.0, coeff=0.5))])
def test_multi_bucket_step_equals_the_oracle_bucket_by_bucket(dev, score, vdtype, knobs):
    """`sga_fused_sparse_step_multi`: eleven buckets in one call -- more than
    one batch of eight, large ones (the sampled-bracket path, ragged tensors)
    mixed with buckets below 2^20 elements (the radix passes) and one of a
    single tensor of three elements -- each with its own k.  Three steps with
    the device state carried over; every bucket's idx, values, mask, residual,
    p, m, v and threshold equal the oracle's step of that bucket on its own."""
    from sga_amd.fused_step import FusedSparseStep, fused_step_multi
    layouts = [[1 << 20, 130, 37], [300_000, 1024, 100_001], [1_200_000], [3], [700_000, 5, 400_001],
               [65_536], [1 << 20], [999], [250_000, 250_000], [1_048_577, 7], [40_000, 3, 17]]
    ratios = [1.0, 10.0, 0.1, 50.0, 1.0, 0.5, 3.0, 1.0, 0.01, 1.0, 25.0]
    bk = []
    for b, sizes in enumerate(layouts):
        segs, n = _segments(sizes, vary=b % 2 == 1)
        gen = torch.Generator().manual_seed(100 + b)
        p = torch.randn(n, generator=gen) * 0.02
        host = [torch.zeros(n), p, torch.zeros(n), torch.zeros(n)]          # r, p, m, v
        bk.append(dict(segs=segs, n=n, k=SEL.k_for(n, ratios[b]), host=host,
                       devs=[t.to(dev) for t in host],
                       fs=FusedSparseStep(n, segs, dev, values_dtype=vdtype, want_mask=True)))
    it = torch.int16 if vdtype == torch.bfloat16 else torch.int32
    for step in (1, 2, 3):
        grads = [student_t(x["n"], 7 * step + b).to(torch.bfloat16) for b, x in enumerate(bk)]
        outs = fused_step_multi([x["fs"] for x in bk], [g.to(dev) for g in grads],
                                *[[x["devs"][a] for x in bk] for a in range(4)], step,
                                ks=[x["k"] for x in bk], score=score, **knobs)
        for b, x in enumerate(bk):
            r, p, m, v = x["host"]
            idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
                grads[b], r, p, m, v, x["segs"], step, k=x["k"], score=score, values_dtype=vdtype,
                **knobs)
            res = x["fs"].read_result()
            what = (step, b, vars(res))
            assert res.status == 0 and res.n_selected == x["k"] and res.thresh == th_ref, what
            assert res.path == (1 if x["n"] >= 1 << 20 else 0), what
            idx, vals = outs[b]
            assert torch.equal(idx.cpu(), idx_ref), what
            assert torch.equal(x["fs"].mask.cpu().bool(), mask_ref), what
            assert torch.equal(vals.cpu().view(it), val_ref.view(it)), what
            for d, h in zip(x["devs"], x["host"]):
                assert same_bits(d, h), what


def test_multi_bucket_step_refusals(dev):
    from sga_amd.fused_step import FusedSparseStep, fused_step_multi
    segs, n = _segments([5000])
    fs = [FusedSparseStep(n, segs, dev, values_dtype=torch.float32) for _ in range(2)]
    t = [torch.zeros(n, device=dev) for _ in range(2)]
    with pytest.raises(ValueError, match="one gradient"):
        fused_step_multi(fs, t, t, t, t, t[:1], 1, ratio_percent=1.0)
    with pytest.raises(ValueError, match="out of range"):
        fused_step_multi(fs, t, t, t, t, t, 1, ks=[10, n + 1])
    fs[1] = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="share the gradient and value dtypes"):
        fused_step_multi(fs, t, t, t, t, t, 1, ratio_percent=1.0)
