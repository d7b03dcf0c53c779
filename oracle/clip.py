"""Oracle for the masked clip service (test infrastructure; torch CPU).

Follows ``sga/engine.py:1052-1218`` at world size 1 with every record counted
locally.  Pinned by closed form: the norm is ``sqrt(sum of squares over the
contributing coordinates)`` (checked against fp64 in the tests), the
coefficient is ``clip / (norm + 1e-6)``, and each route multiplies exactly
the coordinates the reference multiplies.
"""
import torch


def masked_clip_grad_norm(records, clip_grad, was_full, compact_values=None,
                          trace_dumps=False):
    live = [r for r in records if r.grad is not None]
    compact = compact_values if (not was_full and compact_values) else None
    total = torch.zeros(1, dtype=torch.float32)
    seen = set()
    for rec in live:
        mask = None if was_full else rec.mask_u8()
        if compact is not None:
            key = id(rec.bucket_state)
            if key not in seen:
                seen.add(key)
                total += compact[key].float().pow(2).sum()
            continue
        g = rec.grad.data.reshape(-1).float()
        total += g.pow(2).sum() if mask is None else g[mask > 0].pow(2).sum()
    norm = total.sqrt().item()
    out = 1.0
    if clip_grad > 0.0:
        coeff = clip_grad / (norm + 1.0e-6)
        if coeff < 1.0:
            if was_full:
                for rec in live:
                    rec.grad.data.mul_(coeff)
            elif compact is not None:
                if trace_dumps:
                    for v in compact.values():
                        v.mul_(coeff)
                else:
                    out = float(coeff)
            elif trace_dumps:
                for rec in live:
                    m = rec.mask_u8()
                    if m is None:
                        rec.grad.data.mul_(coeff)
                    else:
                        rec.grad.data.view(-1)[m > 0] *= coeff
            else:
                for rec in live:
                    if rec.mask_u8() is None:
                        rec.grad.data.mul_(coeff)
                out = float(coeff)
    return norm, out
