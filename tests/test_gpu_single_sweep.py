"""GPU parity of the single-sweep fused step (g / resid / p / m / v read once)
against the CPU oracle, every output bit for bit, and its stand-back routes."""
import pytest
import torch

from oracle import fused_step as OF
from oracle import select as SEL
from tests.test_gpu_fused import _segments
from tests.util import same_bits, student_t

pytestmark = pytest.mark.gpu


def _run(dev, sizes, steps, ratio, gdtype, vdtype, score="abs_g", seed0=0, vary=False,
         expect_path=2, packed=False, grads=None, out=False, **knobs):
    """``out``: run the out-of-place step on ping-pong state (the new state
    lands in the other set, the inputs must come back untouched)."""
    from sga_amd.fused_step import FusedSparseStep, PackedState
    segs, n = _segments(sizes, vary=vary)
    gen = torch.Generator().manual_seed(1234)
    p = torch.randn(n, generator=gen) * 0.02
    m, v, r = torch.zeros(n), torch.zeros(n), torch.zeros(n)
    dp, dm, dv, dr = (t.to(dev) for t in (p, m, v, r))
    st = PackedState(n, dev).pack(dr, dp, dm, dv) if packed else None
    if out:
        # poisoned, so that a coordinate the step failed to write shows
        st2 = PackedState(n, dev) if packed else None
        if packed:
            st2.data.fill_(float("nan"))
        other = [torch.full((n,), float("nan"), device=dev) for _ in range(4)]
    fs = FusedSparseStep(n, segs, dev, values_dtype=vdtype, want_mask=True)
    k = SEL.k_for(n, ratio)
    for step in range(1, steps + 1):
        g = (grads(n, seed0 + step - 1) if grads else student_t(n, seed0 + step - 1)).to(gdtype)
        idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
            g, r, p, m, v, segs, step, k=k, score=score, values_dtype=vdtype, **knobs)
        if out and packed:
            before = st.data.clone()
            idx, vals = fs.step_packed(g.to(dev), st, step, k=k, score=score, single_sweep=True,
                                       out=st2, **knobs)
            assert same_bits(st.data, before.cpu()), step
            st, st2 = st2, st
            st.unpack(dr, dp, dm, dv)
        elif out:
            before = [t.clone() for t in (dr, dp, dm, dv)]
            idx, vals = fs.step(g.to(dev), dr, dp, dm, dv, step, k=k, score=score,
                                single_sweep=True, out=other, **knobs)
            for t, b in zip((dr, dp, dm, dv), before):
                assert same_bits(t, b.cpu()), step
            (dr, dp, dm, dv), other = other, [dr, dp, dm, dv]
        elif packed:
            idx, vals = fs.step_packed(g.to(dev), st, step, k=k, score=score, single_sweep=True,
                                       **knobs)
            st.unpack(dr, dp, dm, dv)
        else:
            idx, vals = fs.step(g.to(dev), dr, dp, dm, dv, step, k=k, score=score,
                                single_sweep=True, **knobs)
        res = fs.read_result()
        assert res.status == 0 and res.nonfinite == 0 and res.n_selected == k, vars(res)
        assert expect_path is None or res.path == expect_path, vars(res)
        assert res.thresh == th_ref, (step, res.thresh, th_ref)
        assert torch.equal(idx.cpu(), idx_ref), step
        assert torch.equal(fs.mask.cpu().bool(), mask_ref), step
        it = torch.int16 if vdtype == torch.bfloat16 else torch.int32
        assert torch.equal(vals.cpu().view(it), val_ref.view(it)), step
        assert same_bits(dr, r) and same_bits(dm, m) and same_bits(dv, v), step
        assert same_bits(dp, p), step
    return n, k


@pytest.mark.parametrize("score", ["abs_g", "update", "coi", "abs_m", "abs_g_blind",
                                   "abs_gr_over_sqrt_v"])
def test_scores_ragged_tensors(dev, score):
    sizes = [300_000, 128, 37, 700_000, 3, 1024, 250_001, 130, 5, 60_000]
    # |m| is all zeros at the first step: one plateau, which the sweep stands back from
    _run(dev, sizes, 3, 1.0, torch.bfloat16, torch.bfloat16, score=score, vary=True,
         expect_path=None if score == "abs_m" else 2)


@pytest.mark.parametrize("ratio", [0.1, 10.0, 0.001])
def test_ratios(dev, ratio):
    _run(dev, [1_500_003], 3, ratio, torch.bfloat16, torch.bfloat16, score="update")


def test_fp32_grads_fp32_values_packed(dev):
    _run(dev, [1 << 21, 999, 300_001], 3, 1.0, torch.float32, torch.float32, packed=True)


@pytest.mark.parametrize("knobs", [dict(optimizer="adams"),
                                   dict(optimizer="adamw", fold=True, interval=3.0, coeff=0.5),
                                   dict(factor=0.125)])
def test_knobs(dev, knobs):
    _run(dev, [600_000, 130, 37, 500_000, 3, 1024, 100_001], 2, 1.0, torch.float32,
         torch.bfloat16, score="update", vary=True, **knobs)


def test_small_bucket_takes_the_two_sweep_step(dev):
    _run(dev, [200_000, 1024, 100_000], 2, 1.0, torch.bfloat16, torch.bfloat16, expect_path=None)


@pytest.mark.parametrize("sizes,k_ratio", [([1 << 20], 1.0), ([(1 << 20) + 1], 1.0),
                                           ([(1 << 20) - 3, 3, 1], 0.5), ([1 << 20], 1.0e-4)])
def test_buckets_at_the_size_where_the_single_sweep_starts(dev, sizes, k_ratio):
    """2^20 elements is the smallest bucket the sampled bracket takes: exactly
    that size, one element more (a ragged last chunk), a boundary three
    elements before the end, and k = 1."""
    _run(dev, sizes, 2, k_ratio, torch.bfloat16, torch.float32, score="update", vary=len(sizes) > 1,
         expect_path=None)


def test_wide_ratio_fills_the_small_segments(dev):
    """At 60 % a chunk holds ~50 bracket keys against 64 slots of its own
    segment: the chunks that do not fit go to the shared overflow list."""
    _run(dev, [1_200_000], 2, 60.0, torch.bfloat16, torch.bfloat16, expect_path=2)


def test_ratio_beyond_the_buffers_takes_the_two_sweep_step(dev):
    _run(dev, [1 << 24], 1, 45.0, torch.bfloat16, torch.bfloat16, expect_path=None)


def test_chunk_with_more_bracket_keys_than_lds_slots(dev):
    """600 neighbouring coordinates sit within a hair of the k-th magnitude
    (distinct values): their chunk overflows the wave's 256-slot buffer, is
    read again and recorded straight in the overflow list."""
    def grads(n, seed):
        g = student_t(n, seed)
        kth = g.abs().kthvalue(n - SEL.k_for(n, 1.0) + 1).values.item()
        run = torch.arange(600, dtype=torch.float32)
        g[500_000:500_600] = kth * (1.0 + (run - 300.0) * 1e-7)
        return g
    _run(dev, [1_400_000], 2, 1.0, torch.float32, torch.float32, grads=grads)
    _run(dev, [700_000, 700_000], 1, 1.0, torch.float32, torch.bfloat16, score="update",
         grads=grads, expect_path=None)


def test_plateau_inside_the_bracket_stands_back(dev):
    """Half of the coordinates share one magnitude that straddles the k-th
    key: the sample sees the plateau, the sweep stands back before touching
    anything and the radix passes do the step exactly."""
    def grads(n, seed):
        g = student_t(n, seed)
        gen = torch.Generator().manual_seed(seed + 99)
        flat = torch.rand(n, generator=gen) < 0.5
        g[flat] = 3e-3
        return g
    _run(dev, [1_300_000], 1, 30.0, torch.float32, torch.float32, expect_path=0, grads=grads)
    # out of place the key-forming final sweep writes the other set
    _run(dev, [1_300_000], 1, 30.0, torch.float32, torch.float32, expect_path=0, grads=grads, out=True)
    _run(dev, [1_300_000], 1, 30.0, torch.float32, torch.bfloat16, expect_path=0, grads=grads, out=True,
         packed=True)


def _mix32(x):
    x &= 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def _adversarial_grad(n, seed):
    """Magnitudes in [1, 2) in every quad the sample of ``seed`` reads (its
    offsets restated here), in [3, 4) everywhere else."""
    n_sv, n_vec = 16384, n // 4
    gen = torch.Generator().manual_seed(5)
    g = 3.0 + torch.rand(n, generator=gen)
    for j in range(n_sv):
        w0, w1 = j * n_vec // n_sv, (j + 1) * n_vec // n_sv
        vec = w0 + _mix32(j + seed * 0x9E3779B9) % (w1 - w0)
        g[4 * vec: 4 * vec + 4] = 1.0 + torch.rand(4, generator=gen)
    return g


def test_a_bracket_that_missed_is_reported(dev):
    """The one outcome the single sweep cannot repair: every quad the sample
    reads (its offsets restated here for the given seed) holds a magnitude in
    [1, 2), every other coordinate one in [3, 4).  The sample's bracket sits
    near 2, practically the whole bucket lies above it, and the check after
    the sweep reports status 3 instead of a selection.  With another seed the
    sample sees the real population and the same data gives the exact step."""
    from sga_amd.fused_step import FusedSparseStep
    n, seed = 1 << 21, 12345
    g = _adversarial_grad(n, seed)
    segs = [dict(start=0, n=n, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.0)]
    k = SEL.k_for(n, 1.0)

    def run(sd, check=False):
        p = torch.zeros(n, device=dev)
        m, v, r = torch.zeros(n, device=dev), torch.zeros(n, device=dev), torch.zeros(n, device=dev)
        fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, want_mask=True)
        idx, vals = fs.step(g.to(dev), r, p, m, v, 1, k=k, single_sweep=True, seed=sd,
                            check=check)
        return fs.read_result(), idx.cpu(), fs.mask.cpu().bool()

    res, _, _ = run(seed)
    assert res.status == 3 and res.path == 0, vars(res)
    # the wrapper's default waits for the step and refuses to hand back a pack that was not written
    from sga_amd.fused_step import SingleSweepLost
    with pytest.raises(SingleSweepLost, match="missed the k-th key"):
        run(seed, check=True)
    res, idx, mask = run(seed + 1, check=True)
    assert res.status == 0 and res.n_selected == k, vars(res)
    ref_mask, th = SEL.select_topk_flat(g.abs(), k)
    assert res.thresh == th and torch.equal(mask, ref_mask)
    assert torch.equal(idx.long(), torch.nonzero(ref_mask).reshape(-1))


@pytest.mark.parametrize("packed", [False, True])
def test_out_of_place_step_on_ping_pong_state(dev, packed):
    """The out-of-place step: new state in the other set, inputs untouched,
    every output equal to the oracle's over three steps (ragged tensors, a
    ragged last chunk), on both layouts; and a small bucket, which the
    two-sweep step does behind the same call, out of place as well."""
    sizes = [300_000, 128, 37, 700_000, 3, 1024, 250_001, 130, 5, 60_000]
    _run(dev, sizes, 3, 1.0, torch.bfloat16, torch.bfloat16, score="update", vary=True,
         packed=packed, out=True)
    _run(dev, [200_000, 1024, 100_001], 2, 1.0, torch.float32, torch.float32, packed=packed,
         out=True, expect_path=None, optimizer="adams", fold=True, interval=3.0)


@pytest.mark.parametrize("ratio", [0.001, 0.1, 10.0, 60.0])
def test_out_of_place_step_ratios(dev, ratio):
    """k = 15 up to 60 % of the bucket (the narrower bracket of the
    out-of-place step against segments that fill and the overflow list)."""
    _run(dev, [1_500_003], 2, ratio, torch.bfloat16, torch.bfloat16, score="update", out=True)
    _run(dev, [1_200_000, 77], 2, ratio, torch.float32, torch.float32, packed=True, out=True)


@pytest.mark.parametrize("packed", [False, True])
def test_out_of_place_step_redoes_a_missed_bracket(dev, packed):
    """The input of ``test_a_bracket_that_missed_is_reported`` through the
    out-of-place step: the sweep commits on the wrong bracket into the OUTPUT
    arrays, the check sees the miss, and the device redoes the step from the
    untouched inputs.  Status 0, ``redone`` set, every output equal to the
    oracle's."""
    from sga_amd.fused_step import FusedSparseStep, PackedState
    n, seed = 1 << 21, 12345
    g = _adversarial_grad(n, seed)
    segs = [dict(start=0, n=n, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.01)]
    k = SEL.k_for(n, 1.0)
    gen = torch.Generator().manual_seed(8)
    p = torch.randn(n, generator=gen) * 0.02
    r = torch.randn(n, generator=gen) * 1e-3
    m, v = torch.randn(n, generator=gen) * 1e-3, torch.rand(n, generator=gen) * 1e-6
    ins = [t.to(dev) for t in (r, p, m, v)]
    outs = [torch.full((n,), float("nan"), device=dev) for _ in range(4)]
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, want_mask=True)
    if packed:
        st, st2 = PackedState(n, dev).pack(*ins), PackedState(n, dev)
        st2.data.fill_(float("nan"))
        before = st.data.clone()
        idx, vals = fs.step_packed(g.to(dev), st, 1, k=k, single_sweep=True, seed=seed, out=st2)
        assert same_bits(st.data, before.cpu())
        st2.unpack(*outs)
    else:
        idx, vals = fs.step(g.to(dev), *ins, 1, k=k, single_sweep=True, seed=seed, out=outs)
        for t, b in zip(ins, (r, p, m, v)):
            assert same_bits(t, b)
    res = fs.read_result()
    assert res.status == 0 and res.redone and res.path == 0 and res.n_selected == k, vars(res)
    idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
        g, r, p, m, v, segs, 1, k=k, score="abs_g", values_dtype=torch.float32)
    assert res.thresh == th_ref
    assert torch.equal(idx.cpu(), idx_ref) and torch.equal(fs.mask.cpu().bool(), mask_ref)
    assert torch.equal(vals.cpu().view(torch.int32), val_ref.view(torch.int32))
    for t, ref in zip(outs, (r, p, m, v)):        # the oracle stepped r / p / m / v in place
        assert same_bits(t, ref)


def test_out_of_place_step_refuses_overlapping_state(dev):
    from sga_amd.fused_step import FusedSparseStep
    n = 4096
    segs = [dict(start=0, n=n, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.0)]
    fs = FusedSparseStep(n, segs, dev)
    buf = torch.zeros(10 * n, device=dev)
    g = torch.randn(n, device=dev)
    r, p, m, v = (buf[i * n:(i + 1) * n] for i in range(4))
    ok = [buf[(4 + i) * n:(5 + i) * n] for i in range(4)]
    with pytest.raises(RuntimeError, match="overlaps"):
        fs.step(g, r, p, m, v, 1, k=40, single_sweep=True, out=[r, ok[1], ok[2], ok[3]])
    with pytest.raises(RuntimeError, match="overlaps"):
        fs.step(g, r, p, m, v, 1, k=40, single_sweep=True,
                out=[ok[0], ok[1], buf[6 * n - 8:7 * n - 8], ok[3]])
    with pytest.raises(RuntimeError, match="overlaps"):          # ... or the gradient
        fs.step(buf[8 * n:9 * n], r, p, m, v, 1, k=40, single_sweep=True,
                out=[ok[0], ok[1], ok[2], buf[8 * n + 100:9 * n + 100]])
    with pytest.raises(ValueError, match="single-sweep"):
        fs.step(g, r, p, m, v, 1, k=40, out=ok)
    fs.step(g, r, p, m, v, 1, k=40, single_sweep=True, out=ok)
    assert fs.read_result().status == 0


@pytest.mark.parametrize("packed", [False, True])
def test_many_chunks_race_for_full_segments(dev, packed):
    """Record segments that fill up while several chunks reserve room in them
    at once.  1280 of the 65536 chunks hold magnitudes in [1, 2), the rest
    ~1e-6, and k sits in the middle of the large ones: about a quarter of the
    large values fall inside the sampled bracket, ~250 records per hot chunk.
    The hot chunks are the ones whose index is below 160 modulo 8192, i.e. the
    eight chunks c, c + 8192, ... of 160 segments of 256 slots each: one
    chunk's records fit a segment, the other seven find it full and go to the
    overflow list, and chunks over 256 records spill slab by slab.  Every
    output equals the two-sweep step's, bit for bit, on both state layouts."""
    from sga_amd.fused_step import FusedSparseStep, PackedState
    n = 1 << 26
    gen = torch.Generator().manual_seed(11)
    g = torch.rand(n, generator=gen) * 1e-6
    chunk = torch.arange(n // 1024)
    hot = ((chunk & 8191) < 160).repeat_interleave(1024)
    n_hot = int(hot.sum())
    g[hot] = 1.0 + torch.rand(n_hot, generator=gen)
    g *= torch.where(torch.rand(n, generator=gen) < 0.5, -1.0, 1.0)
    k = n_hot // 2
    segs = [dict(start=0, n=n, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8, wd=0.1)]
    gd = g.to(dev)
    p0 = (torch.randn(n, generator=gen) * 0.02).to(dev)
    outs = []
    for single in (False, True):
        r, m, v = (torch.zeros(n, device=dev) for _ in range(3))
        p = p0.clone()
        fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, max_k=k, want_mask=True)
        st = PackedState(n, dev).pack(r, p, m, v) if packed else None
        for step in (1, 2):
            if packed:
                idx, vals = fs.step_packed(gd, st, step, k=k, single_sweep=single)
            else:
                idx, vals = fs.step(gd, r, p, m, v, step, k=k, single_sweep=single)
            res = fs.read_result()
            assert res.status == 0 and res.n_selected == k, (single, step, vars(res))
            assert not single or res.path == 2, (step, vars(res))
        if packed:
            st.unpack(r, p, m, v)
        outs.append((res, idx.clone(), vals.clone(), fs.mask.clone(), r, p, m, v))
        del fs, st
    a, b = outs
    assert (a[0].thresh_bits, a[0].need, a[0].n_gt, a[0].n_eq) == (
        b[0].thresh_bits, b[0].need, b[0].n_gt, b[0].n_eq)
    assert a[0].thresh > 1.0          # the k-th key lies among the hot chunks
    assert torch.equal(a[1], b[1]) and torch.equal(a[3], b[3])
    for x, y in zip(a[2:], b[2:]):
        assert torch.equal(x.view(torch.int32) if x.dtype == torch.float32 else x,
                           y.view(torch.int32) if y.dtype == torch.float32 else y)


@pytest.mark.parametrize("active", [0.10, 0.004])
def test_out_of_place_step_on_row_sparse_gradients(dev, active):
    """Gradients that come in whole rows of 2048 coordinates, as an embedding's
    do: a row is either active (one scale for the row, drawn log-uniformly
    over two decades) or exactly zero.  The four coordinates of a sampled quad
    then fall into one row -- the sample's effective size is a quarter of its
    key count, which the out-of-place step's 6 sigma margins allow for only
    statistically.  Whatever a seed's sample does (bracket held, or missed and
    redone on the device), every output equals the two-sweep step's bit for
    bit; with 0.4 % of the rows active the top 1 % reaches into the zeros and
    the threshold is the zero plateau."""
    from sga_amd.fused_step import FusedSparseStep
    n, row = 1 << 25, 2048
    gen = torch.Generator().manual_seed(17)
    rows = n // row
    on = torch.rand(rows, generator=gen) < active
    scale = 10.0 ** (-4.0 + 2.0 * torch.rand(rows, generator=gen))
    g = (torch.randn(rows, row, generator=gen) * (scale * on)[:, None]).reshape(n).to(torch.bfloat16)
    segs = [dict(start=0, n=n, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8, wd=0.01)]
    k = SEL.k_for(n, 1.0)
    gd = g.to(dev)
    p0 = (torch.randn(n, generator=gen) * 0.02).to(dev)
    ref = [torch.zeros(n, device=dev), p0.clone(), torch.zeros(n, device=dev),
           torch.zeros(n, device=dev)]
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, max_k=k, want_mask=True)
    idx, vals = fs.step(gd, *ref, 1, k=k)
    r2 = fs.read_result()
    assert r2.status == 0 and r2.n_selected == k, vars(r2)
    idx2, vals2, mask2 = idx.clone(), vals.clone(), fs.mask.clone()
    ins = [torch.zeros(n, device=dev), p0, torch.zeros(n, device=dev), torch.zeros(n, device=dev)]
    redone = 0
    for seed in range(12):
        outs = [torch.full((n,), float("nan"), device=dev) for _ in range(4)]
        idx, vals = fs.step(gd, *ins, 1, k=k, single_sweep=True, seed=1000 + seed, out=outs)
        r1 = fs.read_result()
        what = (seed, vars(r1))
        assert r1.status == 0 and r1.n_selected == k, what
        assert (r1.thresh_bits, r1.need, r1.n_gt, r1.n_eq) == (r2.thresh_bits, r2.need, r2.n_gt, r2.n_eq), what
        redone += int(r1.redone)
        assert torch.equal(idx, idx2) and torch.equal(fs.mask, mask2), what
        assert torch.equal(vals.view(torch.int16), vals2.view(torch.int16)), what
        for x, y in zip(outs, ref):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), what
    print(f"active {active}: {redone} of 12 seeds redone, threshold {r2.thresh}")
    if active < 0.01:
        assert r2.thresh == 0.0


@pytest.mark.parametrize("ratio", [100.0, 99.9999, 50.0])
@pytest.mark.parametrize("out", [False, True])
def test_everything_or_nearly_everything_selected(dev, ratio, out):
    """k = n, k = n - 1 and k = n / 2: the bracket is open above or below (or
    too wide for the record lists), so the two-sweep step or the radix passes
    do the step behind the single-sweep call; against the oracle, two steps.
    With an all-zero gradient at the second step the buffer is the residual
    alone: zeros wherever the first step selected."""
    def grads(n, seed):
        return student_t(n, seed) if seed == 0 else torch.zeros(n)
    _run(dev, [1_100_000, 130, 100_001], 2, ratio, torch.float32, torch.float32, expect_path=None,
         grads=grads, out=out)


@pytest.mark.parametrize("variant", ["two_sweep", "single_sweep", "single_sweep_out"])
def test_non_finite_gradients_are_counted_and_rank_first(dev, variant):
    """NaN / Inf in the step's gradient (a loss spike): the reference's exact
    select refuses such scores after a pass of its own (replay.py:545-547);
    the fused step reports their number in the result block instead and the
    caller decides.  What the kernels do with them is defined all the same:
    a key is the magnitude's bit pattern, so every non-finite coordinate ranks
    above every finite one and is selected (k permitting), the finite part of
    the selection is the exact top of the finite scores, and the step ends
    normally on every route."""
    from sga_amd.fused_step import FusedSparseStep
    n = 1_200_003
    segs = [dict(start=0, n=n, lr=1e-4, b1=0.9, b2=0.95, eps=1e-8, wd=0.0)]
    g = student_t(n, 5)
    bad = [0, 1023, 1024, 500_001, 777_777, n - 2, n - 1]
    vals = [float("nan"), float("inf"), -float("inf"), float("nan"), float("inf"), -float("nan"),
            float("inf")]
    for i, x in zip(bad, vals):
        g[i] = x
    k = SEL.k_for(n, 1.0)
    score = g.abs()
    score[torch.tensor(bad)] = torch.finfo(torch.float32).max     # above every finite score
    mask_ref, _ = SEL.select_topk_flat(score, k)
    state = [torch.zeros(n, device=dev) for _ in range(4)]
    outs = [torch.empty(n, device=dev) for _ in range(4)]
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32, want_mask=True)
    idx, _v = fs.step(g.to(dev), *state, 1, k=k, single_sweep=variant != "two_sweep",
                      out=outs if variant.endswith("out") else None)
    res = fs.read_result()
    assert res.status == 0 and res.nonfinite == len(bad) and res.n_selected == k, vars(res)
    assert torch.equal(fs.mask.cpu().bool(), mask_ref)
    assert torch.equal(idx.cpu().long(), torch.nonzero(mask_ref).reshape(-1))
    new_r = (outs if variant.endswith("out") else state)[0].cpu()
    assert bool((new_r[torch.tensor(bad)] == 0.0).all())           # selected: residual cleared
    assert bool(torch.isfinite(new_r).all())


def test_randomized_single_sweep_equals_two_sweep(dev):
    """Seeded random draws of tensor layouts, hyper-parameters, scores, dtypes,
    ratios, knobs and magnitudes: the two-sweep step, the single-sweep step in
    place and the single-sweep step out of place run from the same state and
    must agree in every output bit (idx, values, mask, residual, p, m, v,
    threshold, tie counts) over several steps; on half of the fp32-gradient
    draws the single-sweep arms run without a separate gradient."""
    import random
    from sga_amd.fused_step import FusedSparseStep
    rnd = random.Random(2024)
    for draw in range(24):
        sizes = [rnd.choice([3, 37, 130, 1024, 4097, 60_000]) for _ in range(rnd.randrange(2, 7))]
        sizes.insert(rnd.randrange(len(sizes) + 1), rnd.randrange(1_100_000, 2_500_000))
        segs, n = _segments(sizes, vary=True)
        score = rnd.choice(["abs_g", "update", "coi", "abs_g_blind", "abs_gr_over_sqrt_v"])
        gdt = rnd.choice([torch.bfloat16, torch.float32])
        vdt = rnd.choice([torch.bfloat16, torch.float32])
        ratio = rnd.choice([0.05, 0.5, 1.0, 3.0, 12.0])
        knobs = rnd.choice([{}, dict(optimizer="adams"), dict(fold=True, interval=3.0),
                            dict(factor=0.5, coeff=0.25)])
        scale = 10.0 ** rnd.uniform(-8, 0)
        gen = torch.Generator().manual_seed(draw)
        p0 = (torch.randn(n, generator=gen) * 0.02).to(dev)
        # arm 0 the two-sweep step, arm 1 the single-sweep step in place, arm 2 the single-sweep
        # step out of place on ping-pong state; on some draws with fp32 gradients arms 1 and 2 run
        # on the single-buffer contract (the gradient is added to the buffer beforehand and the
        # step takes none)
        no_g = gdt == torch.float32 and score != "abs_g_blind" and rnd.random() < 0.5
        state = [[torch.zeros(n, device=dev), p0.clone(), torch.zeros(n, device=dev),
                  torch.zeros(n, device=dev)] for _ in range(3)]                  # r, p, m, v
        spare = [torch.full((n,), float("nan"), device=dev) for _ in range(4)]
        fs = [FusedSparseStep(n, segs, dev, values_dtype=vdt, want_mask=True) for _ in range(3)]
        k = SEL.k_for(n, ratio)
        for step in range(1, 4):
            g = (student_t(n, 100 * draw + step) * (scale / 1e-3)).to(gdt).to(dev)
            outs = []
            for which in range(3):
                gin = g
                if which and no_g:
                    state[which][0].add_(g)
                    gin = None
                out = spare if which == 2 else None
                idx, vals = fs[which].step(gin, *state[which], step, k=k, score=score,
                                           single_sweep=bool(which), out=out, **knobs)
                if which == 2:
                    state[2], spare = spare, state[2]
                res = fs[which].read_result()
                assert res.status == 0 and res.n_selected == k, (draw, step, which, vars(res))
                outs.append((idx, vals, fs[which].mask, res))
            what = (draw, step, score, ratio, knobs, no_g)
            it = torch.int16 if vdt == torch.bfloat16 else torch.int32
            for which in (1, 2):
                assert outs[which][3].path in (0, 1, 2), what
                assert (outs[0][3].thresh_bits, outs[0][3].need, outs[0][3].n_eq) == \
                       (outs[which][3].thresh_bits, outs[which][3].need, outs[which][3].n_eq), what
                assert torch.equal(outs[0][0], outs[which][0]), what
                assert torch.equal(outs[0][2], outs[which][2]), what
                assert torch.equal(outs[0][1].view(it), outs[which][1].view(it)), what
                for a, b in zip(state[0], state[which]):
                    assert torch.equal(a.view(torch.int32), b.view(torch.int32)), what
