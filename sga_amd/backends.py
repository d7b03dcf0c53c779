"""Pack / unpack data movement of the reference's two sparse-sync layouts
(``sga/backends/torch_pipelined_index.py``, ``torch_pipelined_mask.py``)
without the collective: what one rank hands to, and takes back from, the
all-reduce."""
import torch

from . import _lib as L
from . import kernels as K
from .support import compact_mask_u8


def index_layout_bounds(idx, n, slices=2):
    """Per-slice (lo, hi) ranges into the sorted ``idx``: with the default two
    slices the split sits at the bucket midpoint (``support.split`` =
    ``searchsorted(idx, n // 2)``, ``sga/support.py:345-351``), any other count
    splits the selected set evenly (``torch_pipelined_index.py:314-325``)."""
    k = idx.numel()
    if slices == 2:
        mid = torch.tensor([n // 2], dtype=idx.dtype, device=idx.device)
        n0 = int(torch.searchsorted(idx, mid).item())
        return [(0, n0), (n0, k)]
    return [(i * k // slices, (i + 1) * k // slices) for i in range(slices)]


def index_layout_pack(grad, idx, values, factor=1.0, slices=2):
    """Index layout: ``values[k]`` in ``grad``'s order of the sorted int32
    ``idx``, packed slice by slice as the reference pipelines it
    (``torch_pipelined_index.py:508-520``); the packed positions of ``grad``
    are zeroed.  Returns the per-slice (lo, hi) ranges of ``values``."""
    out = index_layout_bounds(idx, grad.numel(), slices)
    for lo, hi in out:
        if hi > lo:
            K.pack_selected(grad, idx[lo:hi], values[lo:hi], factor)
    return out


def index_layout_writeback(grad, idx, values):
    """Writeback emission: scatter the reduced values back
    (``torch_pipelined_index.py:483-501``)."""
    K.scatter_selected(grad, idx, values)


def mask_layout_pack(grad, mask_u8, factor=1.0, slices=2):
    """Mask layout: per slice ``[i*(N//slices), ...)`` the ordered compaction
    ``grad[s:e][mask] * factor`` (``torch_pipelined_mask.py:91-116``); a pure
    read of ``grad``.  Returns (payload list, idx) -- idx is kept so unpack
    does not recompute the compaction."""
    n = grad.numel()
    idx = compact_mask_u8(mask_u8)
    base = n // slices if slices > 1 else n
    cuts = [i * base for i in range(slices)] + [n]
    pos = torch.searchsorted(idx, torch.tensor(cuts, dtype=torch.int32, device=idx.device))
    pos = pos.tolist()
    payloads = []
    for lo, hi in zip(pos[:-1], pos[1:]):
        sel = torch.empty(hi - lo, dtype=torch.float32, device=grad.device)
        if hi > lo:
            L.call("sga_gather_selected_blocks", L.ptr(grad), L.ptr(mask_u8),
                   L.ptr(idx[lo:hi]), L.ptr(sel), hi - lo, 1, L.f32(factor),
                   n, L.stream())
        payloads.append(sel)
    return payloads, idx


def mask_layout_unpack(grad, idx, payloads):
    """``grad[s:e][mask] = payload`` per slice (``torch_pipelined_mask.py:117-138``)."""
    off = 0
    for p in payloads:
        if p.numel():
            K.scatter_selected(grad, idx[off:off + p.numel()], p)
        off += p.numel()
