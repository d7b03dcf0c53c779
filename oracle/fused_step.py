"""Oracle for the per-rank fused sparse step (test infrastructure; torch CPU).

The benchmark's per-step driver composes reference primitives in the order
the engine calls them (``sga/engine.py:416-604``):

    buf   <- residual + g_t          (backward's in-place accumulation)
    score <- registry formula on buf (scores.py)
    k     <- k_for                   (selection/topk.py:111-112)
    mask  <- exact-k, lowest-index   (replay.py:538-572)
    idx   <- compact_mask_u8         (support.py:57-99)
    pack_selected(buf, idx, values)  (kernels_torch.py:29-38) -> buf is the
                                      new residual
    sparse commit with (idx, values) (adamw.py:702-724, adamw_torch.py:31-93)
"""
import torch

from . import adamw as A
from . import kernels as K
from . import scores as S
from . import select as SEL


def fused_sparse_step(g, resid, p, m, v, segments, step, ratio_percent=None,
                      k=None, score="abs_g", values_dtype=torch.float32,
                      factor=1.0, coeff=1.0, optimizer="adamw", fold=False,
                      interval=1.0):
    """One step over a flat bucket.

    g        : flat gradient (bf16 or fp32), read only; None: ``resid``
               already holds g + r
    resid    : flat fp32 residual, updated in place (new residual)
    p, m, v  : flat fp32 state, updated in place
    segments : list of dicts {"start","n","lr","b1","b2","eps","wd"}
    score    : "abs_g" (= |g+r|), "update", "coi", "abs_m", or one of the two
               build-side benchmark scores of ``scores.EXTRA_SCORES``
    optimizer: "adamw" | "adams" -- AdamS scores through the replay-side
               routing v := m*m, bc := 1 (replay.py:486-505) and commits with
               ``adams_grad_correct`` (adams_torch.py:34-85)
    fold     : divide the new residual by ``interval`` (adamw_torch.py:88-91)
    Returns (idx int32[k], values[k], mask bool[N], thresh).
    """
    n = resid.numel()
    if g is None:
        # the reference's own buffer contract: backward has already accumulated
        # g into the buffer that keeps the residual (engine.py:453-470 hands
        # ``bs.grad_data`` itself to the pack); nothing is added here
        if score == "abs_g_blind":
            raise ValueError("the residual-blind score ranks the step's own gradient")
        gf = None
    else:
        gf = g.float()
        resid.add_(gf)                         # buf = r + g (one fp32 add)
    buf = resid
    if score == "abs_g":
        sc = buf.abs()
    else:
        sc = torch.empty(n)
        for s in segments:
            a, b = s["start"], s["start"] + s["n"]
            bc1 = 1.0 - s["b1"] ** step
            bc2 = 1.0 - s["b2"] ** step
            sc[a:b] = S.step_score(
                score, p[a:b], m[a:b], v[a:b], buf[a:b],
                None if gf is None else gf[a:b], s["b1"],
                s["b2"], s["eps"], s["wd"], bc1, bc2, optimizer)
    if k is None:
        k = SEL.k_for(n, ratio_percent)
    mask, thresh = SEL.select_topk_flat(sc, k)
    idx = K.compact_mask_u8(mask.to(torch.uint8))
    values = torch.empty(idx.numel(), dtype=values_dtype)
    K.pack_selected(buf, idx, values, factor)
    for s in segments:
        a, b = s["start"], s["start"] + s["n"]
        if optimizer == "adamw":
            A.adamw_grad_correct_compact(
                p[a:b], buf[a:b], m[a:b], v[a:b], idx, values, a, s["lr"],
                s["b1"], s["b2"], s["eps"], s["wd"], step, coeff=coeff,
                fold=fold, interval=interval)
        else:
            # the compact path's torch fallback (adams.py:507-654): scatter
            # the record's values into the pack-cleared buffer, masked commit
            seg_mask = mask[a:b].to(torch.uint8)
            lo = int(torch.searchsorted(idx, a))
            hi = int(torch.searchsorted(idx, b))
            if hi > lo:
                buf[a:b][idx[lo:hi].long() - a] = values[lo:hi].to(buf.dtype)
            A.adams_grad_correct(
                p[a:b], buf[a:b], m[a:b], v[a:b], s["lr"], s["b1"], s["b2"],
                s["eps"], s["wd"], mask=seg_mask, coeff=coeff, clear=True,
                fold=fold, interval=interval)
    return idx, values, mask, thresh
