"""Engine-ordered cycle through the plugin API on the device: full step
(score emission) -> TopkSelection -> compact_mask_u8 -> sparse steps (pack +
compact commit, or masked commit with fused clear/fold) -> reset, against the
same sequence driven through the CPU oracle (order of sga/engine.py:416-604)."""
from types import SimpleNamespace

import pytest
import torch

from oracle import adamw as OA
from oracle import kernels as OK
from oracle import select as SEL
from tests.util import same_bits, student_t

pytestmark = pytest.mark.gpu
HP = dict(lr=1e-3, beta1=0.9, beta2=0.95, eps=1e-8)


def _mk(dev, sizes, seed=0):
    from sga_amd.adamw import ParamRecord
    n = sum(sizes)
    gen = torch.Generator().manual_seed(seed)
    w = torch.randn(n, generator=gen) * 0.02
    bucket = SimpleNamespace(grad_data=torch.zeros(n, device=dev), active_mask_u8=None,
                             extra_main_grads=[], support_index=0)
    wd_dev = w.to(dev)
    recs, off = [], 0
    for i, s in enumerate(sizes):
        mp = SimpleNamespace(data=wd_dev[off:off + s], grad=bucket.grad_data[off:off + s])
        recs.append(ParamRecord(None, mp, bucket, off, off + s, weight_decay=0.1 if i % 2 == 0 else 0.0,
                                step=0, _state={}, **HP))
        off += s
    return n, w, bucket, recs


@pytest.mark.parametrize("compact", [True, False])
def test_full_then_sparse_cycle(dev, compact):
    from sga_amd.adamw import OptContext, SgaAdamW, build_dir_table
    from sga_amd.config import set_args
    from sga_amd.kernels import compact_norm_sq_contribution, pack_selected
    from sga_amd.selection import TopkSelection
    from sga_amd.support import compact_mask_u8
    sizes = [120_000, 1024, 77_777, 128]
    n, w, bucket, recs = _mk(dev, sizes)
    # the plugins read their flags from the args singleton, seeded once as the engine does
    set_args(SimpleNamespace(sga_score="abs_g", sga_optimizer_residual_mean=True,
                             sga_optimizer_compact_search="table",
                             sga_optimizer_full_sync_inactive_lr_scale=1.0,
                             sga_selection_method="histogram", sga_selection_ratio_percent=2.0,
                             sga_selection_histogram_mode="exact"))
    opt = SgaAdamW()
    sel = TopkSelection()
    # oracle-side state
    ow, og = w.clone(), torch.zeros(n)
    om, ov = torch.zeros(n), torch.zeros(n)
    period = 4
    omask = oidx = None
    for it in range(1, 2 * period + 1):
        g = student_t(n, 50 + it)
        bucket.grad_data.add_(g.to(dev))
        og.add_(g)
        full = (it - 1) % period == 0
        for r in recs:
            r.step = it
        if full:
            opt.full_step(OptContext(recs, "full", bucket_states=[bucket]))
            views = [r.grad for r in recs]
            masks = sel.select(SimpleNamespace(grad_views=views))
            # oracle: same order
            for r in recs:
                a, b = r.start, r.end
                OA.adamw_grad_correct(ow[a:b], og[a:b], om[a:b], ov[a:b], r.lr, r.beta1, r.beta2,
                                      r.eps, r.weight_decay, it, emit_score="abs_g")
            th, omasks = SEL.select_masks_histogram([og[r.start:r.end] for r in recs],
                                                    sel.k_for(n), mode="exact")
            assert sel.last_threshold == th
            for a, b in zip(masks, omasks):
                assert torch.equal(a.cpu(), b)
            opt.reset(OptContext(recs, "full", bucket_states=[bucket]), was_full=True)
            og.zero_()
            bucket.active_mask_u8 = torch.cat(masks)
            omask = torch.cat(omasks)
            idx = compact_mask_u8(bucket.active_mask_u8)
            oidx = OK.compact_mask_u8(omask)
            assert torch.equal(idx.cpu(), oidx)
            support = SimpleNamespace(buckets=[SimpleNamespace(
                idx=idx, dir_table=build_dir_table(idx, n))])
        else:
            nxt_full = it % period == 0
            coeff = 0.75
            if compact:
                vals = torch.empty(idx.numel(), device=dev)
                pack_selected(bucket.grad_data, idx, vals, 0.5)
                tot = torch.zeros((), device=dev)
                compact_norm_sq_contribution(vals, tot)
                ctx = OptContext(recs, "sparse", support=support, bucket_states=[bucket],
                                 fold_window=period, next_step_is_full=nxt_full,
                                 apply_coeff=coeff, compact_values={id(bucket): vals})
                opt.sparse_step(ctx)
                ovals = torch.empty(oidx.numel())
                OK.pack_selected(og, oidx, ovals, 0.5)
                otot = torch.zeros(())
                OK.compact_norm_sq_contribution(ovals, otot)
                assert abs(tot.item() - otot.item()) <= 1e-5 * abs(otot.item())
                for r in recs:
                    a, b = r.start, r.end
                    OA.adamw_grad_correct_compact(ow[a:b], og[a:b], om[a:b], ov[a:b], oidx, ovals,
                                                  a, r.lr, r.beta1, r.beta2, r.eps, r.weight_decay,
                                                  it, coeff=coeff, fold=nxt_full, interval=float(period))
            else:
                ctx = OptContext(recs, "sparse", bucket_states=[bucket], fold_window=period,
                                 next_step_is_full=nxt_full, apply_coeff=coeff, compact_values=None)
                opt.sparse_step(ctx)
                for r in recs:
                    a, b = r.start, r.end
                    OA.adamw_grad_correct(ow[a:b], og[a:b], om[a:b], ov[a:b], r.lr, r.beta1,
                                          r.beta2, r.eps, r.weight_decay, it, mask=omask[a:b],
                                          coeff=coeff, clear=True, fold=nxt_full,
                                          interval=float(period))
            opt.reset(ctx, was_full=False)
        dm = torch.cat([r.m for r in recs]).cpu()
        dv = torch.cat([r.v for r in recs]).cpu()
        assert torch.equal(dm, om) and torch.equal(dv, ov), it
        assert torch.equal(bucket.grad_data.cpu(), og), it
    dw = torch.cat([r.main_param.data for r in recs]).cpu()
    assert same_bits(dw, ow)
