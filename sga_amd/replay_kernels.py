"""Operator boundary of ``sga/replay_kernels.py`` on MI355X: same names and
return contracts (``replay_kernels.py:73-99, 330-414``)."""
import os

import torch

from . import _lib as L
from .scores import SCORE_MAP, device_formula

MODE = os.environ.get("REPLAY_FUSED_KERNEL", "auto")


def _check_contig(**ts):
    for name, t in ts.items():
        if t is not None and not t.is_contiguous():
            raise ValueError(f"replay_kernels requires contiguous tensors ({name} is "
                             "not); the fused call sites pass contiguous slices")


def arm(dev_is_cuda, dtype):
    """Run-level arm: killswitch auto + device tensor + fp32 (``:73-87``)."""
    if MODE != "auto":
        return False
    return bool(dev_is_cuda) and dtype == torch.float32


def arm_select(score):
    return arm(score.is_cuda, score.dtype) and score.is_contiguous()


def _mk_formula(name):
    sid = SCORE_MAP[name]

    def f(w, m, v, g, b1, b2, eps, wd, bc1c, bc2c):
        _check_contig(w=w, m=m, v=v, g=g)
        return device_formula(sid, w, m, v, g, b1, b2, eps, wd, bc1c, bc2c)
    return f


_FORMULAS = {n: _mk_formula(n) for n in SCORE_MAP}


def formula(name):
    """Kernel for a registered score name, or None (``:96-99``)."""
    return _FORMULAS.get(name)


def opt_step_inplace(q, m, v, w, lab, lr, wd, b1, b2, bc1c, bc2c, eps,
                     optimizer="adamw", inactive=None, lr_inactive=None):
    """In-place AdamW / AdamS commit with optional dual-lr split and label
    accumulation (``:330-369``)."""
    _check_contig(q=q, m=m, v=v, w=w, lab=lab, inactive=inactive)
    if (inactive is None) != (lr_inactive is None):
        raise ValueError(
            "opt_step_inplace: inactive and lr_inactive come as a pair "
            f"(got inactive={inactive is not None}, lr_inactive={lr_inactive!r})")
    L.require_dev(q, m, v, w, lab, inactive)
    for t in (q, m, v, w, lab):
        if t is not None and t.dtype != torch.float32:
            raise TypeError("opt_step_inplace: fp32 tensors")
    ina = None
    if inactive is not None:
        ina = inactive.view(torch.uint8) if inactive.dtype == torch.bool else inactive
    flags = ((L.RP_HAS_LAB if lab is not None else 0)
             | (L.RP_ADAMS if optimizer == "adams" else 0)
             | (L.RP_SPLIT if inactive is not None else 0))
    L.call("sga_opt_step_inplace", L.ptr(q), L.ptr(m), L.ptr(v), L.ptr(w), L.ptr(lab),
           L.ptr(ina), q.numel(), L.f32(b1), L.f32(1.0 - b1), L.f32(b2), L.f32(1.0 - b2),
           L.f32(bc1c), L.f32(bc2c), L.f32(eps), L.f32(1.0 - lr * wd), L.f32(-lr),
           L.f32(lr * lr), L.f32(lr),
           L.f32(lr_inactive if lr_inactive is not None else 0.0), L.f32(wd), flags,
           L.stream())


def adam_step_inplace(q, m, v, w, lab, lr, wd, b1, b2, bc1c, bc2c, eps):
    opt_step_inplace(q, m, v, w, lab, lr, wd, b1, b2, bc1c, bc2c, eps)


def hist_top16(score):
    """(int64 cpu histogram[32769], non-finite lane count) (``:372-381``)."""
    L.require_dev(score)
    _check_contig(score=score)
    s = score.reshape(-1)
    hist = torch.zeros(32769, dtype=torch.int64, device=s.device)
    nf = torch.zeros(1, dtype=torch.int32, device=s.device)
    L.call("sga_hist_topbits", L.ptr(s), s.numel(), 16, 1, 0, L.ptr(hist), 32769,
           L.ptr(nf), L.stream())
    return hist.cpu(), int(nf.cpu().item())


def cand_extract(score, b):
    """Bin ``b``'s candidates on cpu, ascending index order (``:384-399``)."""
    L.require_dev(score)
    _check_contig(score=score)
    s = score.reshape(-1)
    n = s.numel()
    counts = torch.empty(int(L.raw("sga_mask_chunks", n)), dtype=torch.int32,
                         device=s.device)
    total = torch.empty(1, dtype=torch.int64, device=s.device)
    L.call("sga_cand_extract_count", L.ptr(s), n, int(b), L.ptr(counts), L.ptr(total),
           L.stream())
    k = int(total.item())
    cand = torch.empty(k, dtype=torch.float32, device=s.device)
    if k:
        L.call("sga_cand_extract_fill", L.ptr(s), n, int(b), L.ptr(counts), L.ptr(cand),
               k, L.stream())
    return cand.cpu()


def gt_eq_counts(score, thresh):
    """(gt, eq bool device masks, int64 cpu counts pair) (``:402-414``)."""
    L.require_dev(score)
    _check_contig(score=score)
    s = score.reshape(-1)
    n = s.numel()
    gt = torch.empty(n, dtype=torch.bool, device=s.device)
    eq = torch.empty(n, dtype=torch.bool, device=s.device)
    cnts = torch.zeros(2, dtype=torch.int32, device=s.device)
    L.call("sga_gt_eq", L.ptr(s), n, L.f32(thresh), L.ptr(gt.view(torch.uint8)),
           L.ptr(eq.view(torch.uint8)), L.ptr(cnts), L.stream())
    c = cnts.cpu()
    return gt, eq, torch.tensor([int(c[0]), int(c[1])], dtype=torch.int64)
