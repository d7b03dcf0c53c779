"""Oracle for the scheme-agnostic masked ops (test infrastructure; torch CPU).

Follows ``sga/kernels_torch.py`` and ``sga/support.py:57-99`` of the
reference.  All data movement here is bitwise; the two norms are
tolerance-class reductions.
"""
import torch


def scatter_selected(dst, indices, src):
    """``dst[idx[i]] = src[i]`` (kernels_torch.py:21-26)."""
    dst[indices.long()] = src


def pack_selected(grad, indices, values, factor):
    """``values[i] = grad[idx[i]]*factor; grad[idx[i]] = 0``
    (kernels_torch.py:29-38).  The product is formed in fp32 and stored in
    ``values``' dtype (round-to-nearest-even for bf16)."""
    ix = indices.long()
    picked = grad[ix]
    if factor != 1.0:
        picked = picked * factor
    values.copy_(picked)
    grad[ix] = 0.0


def masked_norm_sq_contribution(grad, mask, total_norm_sq):
    """``total += sum(grad[mask]^2)`` (kernels_torch.py:13-18)."""
    total_norm_sq += grad.reshape(-1)[mask.reshape(-1).bool()].float().pow(2).sum()


def compact_norm_sq_contribution(values, total_norm_sq):
    """``total += sum(values^2)`` (kernels_torch.py:41-45)."""
    total_norm_sq += values.float().pow(2).sum()


def compact_mask_u8(mask_u8):
    """Ascending int32 positions of the set bytes (support.py:57-99)."""
    assert mask_u8.numel() < 2 ** 31
    return torch.nonzero(mask_u8.reshape(-1)).reshape(-1).to(torch.int32)


def _lanes(block_idx, x, n):
    pos = block_idx.long().unsqueeze(1) + torch.arange(x)
    return pos < n, pos.clamp_max(n - 1)


def gather_selected_blocks(grad, mask_u8, block_idx, values, x, factor):
    """Block gather: lane (j,i) reads ``grad[block_idx[j]+i]*factor`` when in
    bounds and mask-set, else 0 (kernels_torch.py:66-92)."""
    kb = block_idx.numel()
    if kb == 0:
        return
    inb, pos = _lanes(block_idx, x, grad.numel())
    act = inb & (mask_u8[pos] != 0)
    v = grad[pos]
    if factor != 1.0:
        v = v * factor
    values[:kb * x] = torch.where(act, v, torch.zeros((), dtype=v.dtype)).reshape(-1)


def scatter_selected_blocks(dst, mask_u8, block_idx, src, x):
    """Mirror of the block gather (kernels_torch.py:95-106)."""
    kb = block_idx.numel()
    if kb == 0:
        return
    inb, pos = _lanes(block_idx, x, dst.numel())
    act = inb & (mask_u8[pos] != 0)
    dst[pos[act]] = src[:kb * x].reshape(kb, x)[act]


def mask_layout_pack(grad, mask_u8, factor, slices=2):
    """Mask-layout payload: per slice ``[i*(N//slices), ...)`` the ordered
    compaction ``grad[s:e][mask]*factor``
    (``sga/backends/torch_pipelined_mask.py:91-116``).  Pure read."""
    n = grad.numel()
    bounds = [i * (n // slices) for i in range(slices)] + [n]
    out = []
    for s, e in zip(bounds[:-1], bounds[1:]):
        sel = grad[s:e][mask_u8[s:e].bool()]
        if factor != 1.0:
            sel = sel * factor
        out.append(sel)
    return out


def mask_layout_unpack(grad, mask_u8, payloads, slices=2):
    """``grad[s:e][mask] = payload`` (torch_pipelined_mask.py:117-138)."""
    n = grad.numel()
    bounds = [i * (n // slices) for i in range(slices)] + [n]
    for (s, e), p in zip(zip(bounds[:-1], bounds[1:]), payloads):
        grad[s:e][mask_u8[s:e].bool()] = p


def index_layout_bounds(idx, n, slices=2):
    """(lo, hi) ranges of the sorted idx per pipeline slice: bucket-midpoint
    split for the default two slices (``support.split``, support.py:345-351),
    even split of the selected set otherwise
    (``torch_pipelined_index.py:314-325``)."""
    k = idx.numel()
    if slices == 2:
        n0 = int((idx.long() < n // 2).sum())
        return [(0, n0), (n0, k)]
    return [(i * k // slices, (i + 1) * k // slices) for i in range(slices)]


def index_layout_pack(grad, idx, values, factor, slices=2):
    """Compact emission of the index backend: slice by slice
    ``pack_selected(grad, idx[lo:hi], values[lo:hi], factor)``
    (``torch_pipelined_index.py:508-520``)."""
    out = index_layout_bounds(idx, grad.numel(), slices)
    for lo, hi in out:
        if hi > lo:
            pack_selected(grad, idx[lo:hi], values[lo:hi], factor)
    return out
