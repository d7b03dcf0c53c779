"""Oracle for the residual-aware AdamW commit (test infrastructure; torch CPU).

Follows ``sga/plugins/optimizer/adamw_torch.py:31-93`` (the commit skeleton),
``sga/plugins/optimizer/adamw.py:502-634`` (wrapper semantics and refusals)
and ``adamw.py:702-724`` (the compact path's torch fallback).
"""
import math

import torch

from . import scores as S


def grad_correct(param, grad, m, v, lr, b1, b2, eps, wd, bc1, bc2, mask,
                 emit_score, coeff=1.0, clear=False, fold=False, interval=1.0,
                 inactive_lr_scale=1.0):
    """One fused commit on flat fp32 buffers, in place
    (adamw_torch.py:31-93).

    sparse (``emit_score is None``): ``g' = where(mask, grad*coeff, 0)``
    full   (score name): ``g' = grad`` everywhere, the score lands in ``grad``
    dual-lr (``inactive_lr_scale != 1``): full step, lr scaled off-mask.
    """
    if inactive_lr_scale != 1.0:
        g = grad
        lr_apply = torch.where(mask > 0, lr, lr * inactive_lr_scale)
    elif mask is not None:
        g = torch.where(mask > 0, grad, torch.zeros_like(grad))
        lr_apply = lr
    else:
        g = grad
        lr_apply = lr
    if coeff != 1.0:
        g = torch.where(mask > 0, g * coeff, g)
    upd = S.update(param, m, v, g, b1, b2, eps, wd, bc1, bc2)
    if emit_score is None:
        score = None
    elif emit_score == "update":
        score = upd
    else:
        score = S.get_formula(emit_score)(param, m, v, g, b1, b2, eps, wd,
                                          bc1, bc2)
    m_new = b1 * m + (1.0 - b1) * g
    v_new = b2 * v + (1.0 - b2) * g * g
    m.copy_(m_new)
    v.copy_(v_new)
    if emit_score is not None:
        grad.copy_(score)
    else:
        if clear and mask is not None:
            grad.masked_fill_(mask > 0, 0.0)
        if fold:
            grad.div_(interval)
    param.sub_(lr_apply * upd)


def check_knobs(mask, emit_score, coeff, clear, fold, inactive_lr_scale):
    """The wrapper's refusals, same substrings (adamw.py:554-592)."""
    if emit_score is not None and emit_score not in S.SCORE_IDS:
        raise ValueError(
            f"emit_score '{emit_score}' has no _grad_correct_kernel branch "
            f"(implemented: {sorted(S.SCORE_IDS)})")
    if ((coeff != 1.0) or clear or fold) and (emit_score is not None
                                              or mask is None):
        raise ValueError(
            f"grad-correct sparse fusion (coeff={coeff!r}, clear={clear!r}, "
            f"fold={fold!r}) requires a sparse step (emit_score=None) with "
            "a mask")
    if inactive_lr_scale != 1.0:
        if not (math.isfinite(inactive_lr_scale) and inactive_lr_scale >= 0.0):
            raise ValueError("grad-correct inactive_lr_scale must be a "
                             f"finite float >= 0.0 (got {inactive_lr_scale!r})")
        if emit_score is None or mask is None:
            raise ValueError(
                "grad-correct boundary dual-lr (inactive_lr_scale="
                f"{inactive_lr_scale!r}) requires a full step (emit_score "
                "set) with a mask")
    if (mask is not None and emit_score is not None
            and inactive_lr_scale == 1.0):
        raise ValueError("grad-correct masked-commit full step (mask + "
                         "emit_score with inactive_lr_scale=1.0) is refused")


def adamw_grad_correct(param, grad, m, v, lr, b1, b2, eps, wd, step,
                       mask=None, emit_score=None, coeff=1.0, clear=False,
                       fold=False, interval=1.0, inactive_lr_scale=1.0):
    """Wrapper with the Python-double bias corrections (adamw.py:552-553)."""
    check_knobs(mask, emit_score, coeff, clear, fold, inactive_lr_scale)
    if param.numel() == 0:
        return
    grad_correct(param, grad, m, v, lr, b1, b2, eps, wd,
                 1.0 - b1 ** step, 1.0 - b2 ** step, mask, emit_score,
                 coeff=coeff, clear=clear, fold=fold, interval=interval,
                 inactive_lr_scale=inactive_lr_scale)


def adamw_grad_correct_compact(param, grad, m, v, idx, values, rec_start, lr,
                               b1, b2, eps, wd, step, coeff=1.0, fold=False,
                               interval=1.0):
    """Compact commit: the record's slice of the sorted bucket ``(idx,
    values)`` is scattered into the pack-cleared grad buffer, then the masked
    commit runs with ``clear=True`` (adamw.py:702-724)."""
    n = param.numel()
    if n == 0:
        return
    k = idx.numel()
    lo = 0 if k == 0 else int(torch.searchsorted(idx, rec_start))
    hi = 0 if k == 0 else int(torch.searchsorted(idx, rec_start + n))
    mask = torch.zeros(n, dtype=torch.uint8)
    if hi > lo:
        local = idx[lo:hi].long() - rec_start
        mask[local] = 1
        grad[local] = values[lo:hi].to(grad.dtype)
    grad_correct(param, grad, m, v, lr, b1, b2, eps, wd,
                 1.0 - b1 ** step, 1.0 - b2 ** step, mask, None,
                 coeff=coeff, clear=True, fold=fold, interval=interval)


def build_dir_table(idx, total_n):
    """``table[j] = lower_bound(idx, j*1024)`` for ``(total_n>>10)+2`` entries
    (adamw.py:472-499; equals searchsorted-left per
    tests/test_kernels_gpu.py:690-710)."""
    n_table = (total_n >> 10) + 2
    keys = torch.arange(n_table, dtype=torch.int64) * 1024
    return torch.searchsorted(idx.long(), keys).to(torch.int32)


def adams_grad_correct(param, grad, m, v, lr, b1, b2, eps, wd, mask=None,
                       emit_score=None, coeff=1.0, clear=False, fold=False,
                       interval=1.0, inactive_lr_scale=1.0):
    """AdamS twin (``sga/plugins/optimizer/adams_torch.py:34-85``): v is
    rebuilt from the pre-commit m, no bias corrections."""
    check_knobs(mask, emit_score, coeff, clear, fold, inactive_lr_scale)
    if param.numel() == 0:
        return
    if inactive_lr_scale != 1.0:
        g = grad
        lr_apply = torch.where(mask > 0, lr, lr * inactive_lr_scale)
    elif mask is not None:
        g = torch.where(mask > 0, grad, torch.zeros_like(grad))
        lr_apply = lr
    else:
        g = grad
        lr_apply = lr
    if coeff != 1.0:
        g = torch.where(mask > 0, g * coeff, g)
    upd = S.update(param, m, v, g, b1, b2, eps, wd, 1.0, 1.0, optimizer="adams")
    score = None
    if emit_score == "update":
        score = upd
    elif emit_score is not None:
        score = S.get_formula(emit_score)(param, m, v, g, b1, b2, eps, wd, 1.0, 1.0,
                                          optimizer="adams")
    m_new = b1 * m + (1.0 - b1) * g
    v_new = b2 * (m * m) + (1.0 - b2) * g * g
    m.copy_(m_new)
    v.copy_(v_new)
    if emit_score is not None:
        grad.copy_(score)
    else:
        if clear and mask is not None:
            grad.masked_fill_(mask > 0, 0.0)
        if fold:
            grad.div_(interval)
    param.sub_(lr_apply * upd)
