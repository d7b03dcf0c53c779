"""Operator boundary of ``sga/kernels.py`` on MI355X: same function names,
argument order and refusals (reference ``sga/kernels.py:145-302``)."""
import torch

from . import _lib as L


def scatter_selected(dst, indices, src):
    """``dst[idx[i]] = src[i]`` in place (``sga/kernels.py:145-163``)."""
    n = indices.numel()
    if n == 0:
        return
    assert dst.numel() < 2 ** 31, (
        f"scatter_selected assumes < 2^31 bucket elements, got {dst.numel()}")
    L.require_dev(dst, indices, src)
    L.require_contig(dst=dst, indices=indices, src=src)
    if indices.dtype != torch.int32:
        indices = indices.to(torch.int32)
    if dst.dtype != torch.float32 or src.dtype != torch.float32:
        raise TypeError("scatter_selected: fp32 dst/src")
    L.call("sga_scatter_selected", L.ptr(dst), L.ptr(indices), L.ptr(src), n,
           dst.numel(), L.stream())


def pack_selected(grad, indices, values, factor):
    """``values[i] = grad[idx[i]]*factor; grad[idx[i]] = 0`` in one pass
    (``sga/kernels.py:166-187``).  ``values`` may be fp32 or bf16."""
    k = indices.numel()
    if k == 0:
        return
    assert grad.numel() < 2 ** 31, (
        f"pack_selected assumes < 2^31 bucket elements, got {grad.numel()}")
    L.require_dev(grad, indices, values)
    L.require_contig(grad=grad, indices=indices, values=values)
    if indices.dtype != torch.int32:
        indices = indices.to(torch.int32)
    if grad.dtype != torch.float32:
        raise TypeError("pack_selected: fp32 grad buffer")
    assert values.numel() >= k
    L.call("sga_pack_selected", L.ptr(grad), L.ptr(indices), L.ptr(values),
           L.dtype_code(values), L.f32(factor), k, grad.numel(), L.stream())


def _check_x(x):
    if not isinstance(x, int) or x < 1 or x > 1024 or x & (x - 1):
        raise ValueError(f"block size x must be a power of two in [1, 1024], got {x!r}")


def gather_selected_blocks(grad, mask_u8, block_idx, values, x, factor):
    """Mask-guarded block gather (``sga/kernels.py:190-221``)."""
    kb = block_idx.numel()
    if kb == 0:
        return
    assert grad.numel() < 2 ** 31, (
        f"gather_selected_blocks assumes < 2^31 bucket elements, got {grad.numel()}")
    assert values.numel() >= kb * x, (
        f"values buffer {values.numel()} < k_blocks*x {kb * x}")
    _check_x(x)
    L.require_dev(grad, mask_u8, block_idx, values)
    L.require_contig(grad=grad, mask_u8=mask_u8, block_idx=block_idx, values=values)
    L.call("sga_gather_selected_blocks", L.ptr(grad), L.ptr(mask_u8), L.ptr(block_idx),
           L.ptr(values), kb, x, L.f32(factor), grad.numel(), L.stream())


def scatter_selected_blocks(dst, mask_u8, block_idx, src, x):
    """Mirror of the block gather (``sga/kernels.py:224-249``)."""
    kb = block_idx.numel()
    if kb == 0:
        return
    assert dst.numel() < 2 ** 31, (
        f"scatter_selected_blocks assumes < 2^31 bucket elements, got {dst.numel()}")
    assert src.numel() >= kb * x, f"src buffer {src.numel()} < k_blocks*x {kb * x}"
    _check_x(x)
    L.require_dev(dst, mask_u8, block_idx, src)
    L.require_contig(dst=dst, mask_u8=mask_u8, block_idx=block_idx, src=src)
    L.call("sga_scatter_selected_blocks", L.ptr(dst), L.ptr(mask_u8), L.ptr(block_idx),
           L.ptr(src), kb, x, dst.numel(), L.stream())


def _partials(n, device):
    return torch.empty(int(L.raw("sga_norm_partials", n)), dtype=torch.float32,
                       device=device)


def compact_norm_sq_contribution(values, total_norm_sq):
    """``total += sum(values^2)``, deterministic two-stage reduction
    (``sga/kernels.py:252-268``)."""
    k = values.numel()
    if k == 0:
        return
    L.require_dev(values, total_norm_sq)
    v = values.reshape(-1)
    L.require_contig(values=v)
    if v.dtype != torch.float32 or total_norm_sq.dtype != torch.float32:
        raise TypeError("compact_norm_sq_contribution: fp32 values and total")
    L.call("sga_compact_norm_sq", L.ptr(v), k, L.ptr(_partials(k, v.device)),
           L.ptr(total_norm_sq), L.stream())


def use_fused_masked_op(grad, mask):
    """Same predicate as ``sga/kernels.py:271-281`` minus the Triton test."""
    return (grad.is_cuda and grad.dtype == torch.float32 and grad.is_contiguous()
            and mask.is_contiguous() and mask.element_size() == 1)


def masked_norm_sq_contribution(grad, mask, total_norm_sq):
    """``total += sum(grad[mask]^2)`` (``sga/kernels.py:284-302``); two-stage
    and run-to-run deterministic (the reference accumulates with a float
    atomic)."""
    g = grad.view(-1)
    mk = mask.view(-1)
    n = g.numel()
    if n == 0:
        return
    L.require_dev(g, mk, total_norm_sq)
    if not use_fused_masked_op(g, mk):
        raise TypeError("masked_norm_sq_contribution: needs contiguous fp32 grad "
                        "and a contiguous 1-byte mask on the device")
    if mk.dtype == torch.bool:
        mk = mk.view(torch.uint8)
    L.call("sga_masked_norm_sq", L.ptr(g), L.ptr(mk), n, L.ptr(_partials(n, g.device)),
           L.ptr(total_norm_sq), L.stream())


def _as_int(s):
    return int(s.item()) if torch.is_tensor(s) else int(s)


def _state_step(wrapper, group):
    """The per-param ``state['step']`` of the first parameter of ``group`` that
    has one (torch AdamW's counter style), or None."""
    for p in group['params']:
        st = wrapper.optimizer.state.get(p)
        if st is not None and 'step' in st:
            return _as_int(st['step'])
    return None


def sga_peek_step(wrapper, group):
    """The step number the NEXT optimizer commit will use, read without
    touching any counter (``sga/kernels.py:305-326``): the group counter + 1
    when the optimizer keeps one (TE / apex FusedAdam), else the first
    per-param state counter + 1 (torch AdamW), else 1."""
    if 'step' in group:
        return _as_int(group['step']) + 1
    s = _state_step(wrapper, group)
    return 1 if s is None else s + 1


def sga_advance_step(wrapper, group):
    """Advance the shared Adam step counter by one and return the new value as
    a Python int (``sga/kernels.py:329-367``).  A group without a counter is
    seeded ONCE per wrapper from the per-param state (0 when there is none);
    every group then starts from that seed."""
    if 'step' in group:
        group['step'] = _as_int(group['step']) + 1
        return group['step']
    if not getattr(wrapper, '_sga_step_seeded', False):
        s = _state_step(wrapper, group)
        wrapper._sga_step_seeded = True
        wrapper._sga_step_seed_value = 0 if s is None else s
    group['step'] = wrapper._sga_step_seed_value + 1
    return group['step']
