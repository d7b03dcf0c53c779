"""The fused step on the reference's own buffer contract: backward has
already accumulated the step's gradient into the fp32 buffer that keeps the
residual (``sga/engine.py:453-470`` hands ``bs.grad_data`` itself to the
pack), so the step takes NO separate gradient (``g=None``) and the buffer is
used bit for bit as it stands.  Every variant of the step against the CPU
oracle run the same way, state carried over three steps."""
import pytest
import torch

from oracle import fused_step as OF
from oracle import select as SEL
from tests.test_gpu_fused import _segments
from tests.util import same_bits, student_t

pytestmark = pytest.mark.gpu

SIZES = [300_000, 128, 37, 700_000, 3, 1024, 250_001, 130, 5, 60_000]


def _start(n, seed):
    gen = torch.Generator().manual_seed(seed)
    p = torch.randn(n, generator=gen) * 0.02
    m = torch.randn(n, generator=gen) * 1e-4
    v = torch.rand(n, generator=gen) * 1e-8
    r = torch.randn(n, generator=gen) * 3e-4
    r[::977] = -0.0                          # stays -0.0 when the step's gradient there is -0.0
    return r, p, m, v


def _grad(n, seed):
    g = student_t(n, seed)
    g[::977] = -0.0
    return g


@pytest.mark.parametrize("variant", ["two_sweep", "single_sweep", "packed", "single_sweep_out",
                                     "packed_single_sweep_out"])
@pytest.mark.parametrize("score,knobs", [("abs_g", {}), ("update", {}), ("coi", dict(optimizer="adams")),
                                         ("abs_m", {}), ("abs_gr_over_sqrt_v", {}),
                                         ("update", dict(fold=True, interval=3.0, coeff=0.5))])
def test_buffer_that_already_holds_g_plus_r(dev, variant, score, knobs):
    from sga_amd.fused_step import FusedSparseStep, PackedState
    segs, n = _segments(SIZES, vary=True)
    host = list(_start(n, 77))
    devs = [t.to(dev) for t in host]
    other = [torch.full((n,), float("nan"), device=dev) for _ in range(4)]
    packed = variant.startswith("packed")
    st = PackedState(n, dev).pack(*devs) if packed else None
    st2 = PackedState(n, dev) if packed else None
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.bfloat16, want_mask=True)
    k = SEL.k_for(n, 1.0)
    single = "single_sweep" in variant
    for step in (1, 2, 3):
        g = _grad(n, 40 + step)
        host[0].add_(g)                       # backward's accumulation, on both sides
        if packed:
            st.unpack(resid=devs[0])
            devs[0].add_(g.to(dev))
            st.pack(resid=devs[0])
        else:
            devs[0].add_(g.to(dev))
        assert same_bits(devs[0], host[0])
        idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
            None, *host, segs, step, k=k, score=score, values_dtype=torch.bfloat16, **knobs)
        if variant == "packed_single_sweep_out":
            idx, vals = fs.step_packed(None, st, step, k=k, score=score, single_sweep=True, out=st2,
                                       **knobs)
            st, st2 = st2, st
        elif packed:
            idx, vals = fs.step_packed(None, st, step, k=k, score=score, **knobs)
        elif variant == "single_sweep_out":
            idx, vals = fs.step(None, *devs, step, k=k, score=score, single_sweep=True, out=other,
                                **knobs)
            devs, other = other, devs
        else:
            idx, vals = fs.step(None, *devs, step, k=k, score=score, single_sweep=single, **knobs)
        if packed:
            st.unpack(*devs)
        res = fs.read_result()
        what = (step, vars(res))
        assert res.status == 0 and res.n_selected == k and res.thresh == th_ref, what
        if single and score != "abs_m":       # |m| keeps a plateau the sweep stands back from
            assert res.path == 2, what
        assert torch.equal(idx.cpu(), idx_ref), what
        assert torch.equal(fs.mask.cpu().bool(), mask_ref), what
        assert torch.equal(vals.cpu().view(torch.int16), val_ref.view(torch.int16)), what
        for d, h in zip(devs, host):
            assert same_bits(d, h), what


def test_multi_bucket_step_with_and_without_a_separate_gradient(dev):
    """One call, five buckets: three whose buffer already holds g + r, two
    with an fp32 gradient of their own; each equals the oracle's step of that
    bucket run the same way."""
    from sga_amd.fused_step import FusedSparseStep, fused_step_multi
    layouts = [[1 << 20, 130, 37], [300_000, 1024, 100_001], [1_200_000], [999], [700_000, 5, 400_001]]
    own_g = [False, True, False, False, True]
    bk = []
    for b, sizes in enumerate(layouts):
        segs, n = _segments(sizes, vary=b % 2 == 1)
        host = list(_start(n, 100 + b))
        bk.append(dict(segs=segs, n=n, k=SEL.k_for(n, 1.0), host=host, devs=[t.to(dev) for t in host],
                       fs=FusedSparseStep(n, segs, dev, values_dtype=torch.float32, want_mask=True)))
    for step in (1, 2):
        grads = [_grad(x["n"], 9 * step + b) for b, x in enumerate(bk)]
        for b, x in enumerate(bk):
            if not own_g[b]:
                x["host"][0].add_(grads[b])
                x["devs"][0].add_(grads[b].to(dev))
        outs = fused_step_multi([x["fs"] for x in bk],
                                [grads[b].to(dev) if own_g[b] else None for b in range(len(bk))],
                                *[[x["devs"][a] for x in bk] for a in range(4)], step,
                                ks=[x["k"] for x in bk], score="update")
        for b, x in enumerate(bk):
            idx_ref, val_ref, mask_ref, th_ref = OF.fused_sparse_step(
                grads[b] if own_g[b] else None, *x["host"], x["segs"], step, k=x["k"], score="update",
                values_dtype=torch.float32)
            res = x["fs"].read_result()
            what = (step, b, vars(res))
            assert res.status == 0 and res.n_selected == x["k"] and res.thresh == th_ref, what
            idx, vals = outs[b]
            assert torch.equal(idx.cpu(), idx_ref), what
            assert torch.equal(vals.cpu().view(torch.int32), val_ref.view(torch.int32)), what
            for d, h in zip(x["devs"], x["host"]):
                assert same_bits(d, h), what


def test_no_gradient_refusals(dev):
    from sga_amd import _lib as L
    from sga_amd.fused_step import FusedSparseStep, fused_step_multi
    segs, n = _segments([5000])
    fs = FusedSparseStep(n, segs, dev, values_dtype=torch.float32)
    r, p, m, v = (torch.zeros(n, device=dev) for _ in range(4))
    with pytest.raises(ValueError, match="abs_g_blind"):
        fs.step(None, r, p, m, v, 1, k=50, score="abs_g_blind")
    fs._upload_segments(1)
    args = [L.ptr(r), L.ptr(p), L.ptr(m), L.ptr(v), n, 50, L.ptr(fs._seg_dev), 1, 0, L.ptr(fs.idx),
            L.ptr(fs.values), L.SGA_F32, None, 1.0, 1.0, 1, 0, 1.0, L.ptr(fs.result), L.ptr(fs.ws),
            fs.ws_bytes, L.stream()]
    with pytest.raises(RuntimeError, match="g may be NULL only with g_dtype SGA_F32"):
        L.call("sga_fused_sparse_step", None, L.SGA_BF16, *args)
    L.call("sga_fused_sparse_step", None, L.SGA_F32, *args)
    assert fs.read_result().status == 0
    two = [FusedSparseStep(n, segs, dev, values_dtype=torch.float32) for _ in range(2)]
    t = [torch.zeros(n, device=dev) for _ in range(2)]
    with pytest.raises(ValueError, match="goes with fp32"):
        fused_step_multi(two, [t[0].to(torch.bfloat16), None], t, t, t, t, 1, ratio_percent=1.0)
