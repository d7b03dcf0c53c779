"""Support helpers of ``sga/support.py`` on MI355X: mask -> sorted int32 idx."""
from typing import Optional

import torch

from . import _lib as L

_GATHER_BUF_CHUNK = 4 << 20   # growth granularity, sga/support.py:29


class IndexPool:
    """Grow-only int32 buffer reused across cycles (``sga/support.py:32-54``)."""

    def __init__(self):
        self.buf: Optional[torch.Tensor] = None

    def get(self, k, device):
        if self.buf is None or self.buf.numel() < k or self.buf.device != device:
            cap = -(-k // _GATHER_BUF_CHUNK) * _GATHER_BUF_CHUNK
            if self.buf is not None and self.buf.device == device:
                cap = max(cap, self.buf.numel())
            self.buf = torch.empty(cap, dtype=torch.int32, device=device)
        return self.buf


def compact_mask_u8(mask_u8, pool: Optional[IndexPool] = None):
    """Ascending int32 positions of the non-zero bytes of ``mask_u8``
    (``sga/support.py:57-99``): one counting sweep, one host read of k (the
    reference syncs on the count too), one ordered fill sweep."""
    n = mask_u8.numel()
    assert n < 2 ** 31, f"int32 support indices assume < 2^31 elements, got {n}"
    L.require_dev(mask_u8)
    mk = mask_u8.reshape(-1)
    L.require_contig(mask_u8=mk)
    if mk.dtype == torch.bool:
        mk = mk.view(torch.uint8)
    if mk.dtype != torch.uint8:
        raise TypeError("compact_mask_u8: uint8/bool mask")
    dev = mk.device
    if n == 0:
        return torch.empty(0, dtype=torch.int32, device=dev)
    counts = torch.empty(int(L.raw("sga_mask_chunks", n)), dtype=torch.int32, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    L.call("sga_mask_count", L.ptr(mk), n, L.ptr(counts), L.ptr(total), L.stream())
    k = int(total.item())
    buf = pool.get(k, dev) if pool is not None else torch.empty(
        k, dtype=torch.int32, device=dev)
    if k:
        L.call("sga_mask_fill", L.ptr(mk), n, L.ptr(counts), L.ptr(buf), buf.numel(),
               L.stream())
    return buf[:k]


def block_idx_from_mask(mask_u8, spans, x):
    """int32 block-start index per x-element block that has ANY set byte, per
    span; blocks tile each span from its start, the tail block may be short
    (``sga/support.py:102-142``).  With x == 1 equals ``compact_mask_u8``."""
    assert mask_u8.numel() < 2 ** 31, (
        f"int32 block-start indices assume < 2^31 elements, got {mask_u8.numel()}")
    L.require_dev(mask_u8)
    mk = mask_u8.reshape(-1)
    if mk.dtype == torch.bool:
        mk = mk.view(torch.uint8)
    dev = mk.device
    prev_end, counts = 0, []
    for start, end in spans:
        assert start >= prev_end, (
            f"spans must be ascending and non-overlapping, got span starting at {start} "
            f"after one ending at {prev_end}")
        prev_end = end
        counts.append(-(-(end - start) // x))
    total = sum(counts)
    if total == 0:
        return torch.empty(0, dtype=torch.int32, device=dev)
    any_b = torch.empty(total, dtype=torch.uint8, device=dev)
    st = L.stream()
    off = 0
    for (start, end), nb in zip(spans, counts):
        if nb:
            L.call("sga_block_any", L.ptr(mk[start:end]), end - start, x,
                   L.ptr(any_b[off:off + nb]), st)
        off += nb
    ordinal = compact_mask_u8(any_b).long()        # selected block ordinals, ascending
    if ordinal.numel() == 0:
        return torch.empty(0, dtype=torch.int32, device=dev)
    first = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)[:-1]), device=dev)
    starts = torch.tensor([s for s, _ in spans], device=dev)
    owner = torch.searchsorted(first, ordinal, right=True) - 1
    return ((ordinal - first[owner]) * x + starts[owner]).to(torch.int32)
