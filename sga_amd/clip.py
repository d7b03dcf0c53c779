"""Masked gradient clipping (``sga/engine.py:1052-1218``,
``_masked_clip_grad_norm``) on the device.

Managed params contribute the raw accumulated gradient at their
support-masked coordinates (or, with compact emission, the communicated
values once per bucket); full steps and mask-less records contribute whole.
The squared norm is accumulated by deterministic two-stage reductions, so
the clip coefficient is run-to-run reproducible.
"""
import torch

from . import _lib as L
from .kernels import compact_norm_sq_contribution, masked_norm_sq_contribution


def scale_masked_(grad, mask, coeff):
    """``grad[mask > 0] *= coeff`` (``mask`` None: ``grad.mul_(coeff)``)."""
    g = grad.reshape(-1)
    L.require_dev(g)
    L.require_contig(grad=g)
    if g.dtype != torch.float32:
        raise TypeError("scale_masked_: fp32 grad")
    if mask is not None:
        L.require_dev(mask)
        if mask.numel() != g.numel() or mask.dtype != torch.uint8:
            raise ValueError("scale_masked_: mask must be uint8 with grad's length")
    L.call("sga_scale_masked", L.ptr(g), L.ptr(mask) if mask is not None else None,
           g.numel(), L.f32(coeff), L.stream())


def masked_clip_grad_norm(records, clip_grad, was_full, compact_values=None,
                          trace_dumps=False):
    """Returns ``(grad_norm, sparse_coeff)``.

    ``compact_values`` maps ``id(bucket_state)`` to that bucket's
    communicated fp32 values (compact emission, sparse steps only).  The
    coefficient is applied in place on full steps, on dump steps and on
    mask-less records; otherwise it is returned for the commit kernel's
    in-register multiply (``engine.py:1172-1217``).
    """
    live = [r for r in records if r.grad is not None]
    if not live:
        return 0.0, 1.0
    compact = compact_values if (not was_full and compact_values) else None
    total = torch.zeros(1, dtype=torch.float32, device=live[0].grad.device)
    seen = set()
    for rec in live:
        mask = None if was_full else rec.mask_u8()
        if compact is not None:
            if mask is None:
                raise RuntimeError("compact clip: record without an active mask")
            key = id(rec.bucket_state)
            if key not in compact:
                raise RuntimeError("compact clip: bucket state without a values entry")
            if key not in seen:
                seen.add(key)
                if compact[key].numel():
                    compact_norm_sq_contribution(compact[key], total)
            continue
        g = rec.grad.data.reshape(-1)
        if mask is None:
            compact_norm_sq_contribution(g, total)
        else:
            masked_norm_sq_contribution(g, mask, total)
    grad_norm = total.sqrt().item()
    sparse_coeff = 1.0
    if clip_grad > 0.0:
        coeff = clip_grad / (grad_norm + 1.0e-6)
        if coeff < 1.0:
            if was_full:
                for rec in live:
                    scale_masked_(rec.grad.data, None, coeff)
            elif compact is not None:
                if trace_dumps:
                    for vals in compact.values():
                        if vals.numel():
                            scale_masked_(vals, None, coeff)
                else:
                    sparse_coeff = float(coeff)
            elif trace_dumps:
                for rec in live:
                    scale_masked_(rec.grad.data, rec.mask_u8(), coeff)
            else:
                for rec in live:
                    if rec.mask_u8() is None:
                        scale_masked_(rec.grad.data, None, coeff)
                sparse_coeff = float(coeff)
    return grad_norm, sparse_coeff
