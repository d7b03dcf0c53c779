"""Top-k selection plugin on MI355X (``sga/plugins/selection/topk.py``,
``_histogram.py``, ``_exact.py``): strict-ratio global top-k over per-param
score views, returning per-view uint8 masks.

The exact threshold is found on the device by a three-level radix descent
over the sign-stripped fp32 patterns (no host round trip, no candidate
gather); ``balanced`` / ``fast`` keep the reference's stride-8 subsample
histogram and crossing-bin rule so the masks are identical to its.
"""
import ctypes as C
from types import SimpleNamespace

import torch

from . import _lib as L
from .config import get_args

_HIST_MODES = {"exact": (16, 32769, 1), "balanced": (16, 32769, 8),
               "fast": (19, 4097, 8)}            # _histogram.py:68-72
_CHUNK = 1024


class SelectResult(C.Structure):
    """struct sga_select_result"""
    _fields_ = [(n, C.c_uint32) for n in
                ("thresh_bits", "need", "n_gt", "n_eq", "n_selected", "nonfinite",
                 "status", "path")]


def read_result(res_t):
    """Decode a device uint32[8] result block (one host sync)."""
    r = res_t.cpu().tolist()
    out = SimpleNamespace(thresh_bits=r[0], need=r[1], n_gt=r[2], n_eq=r[3],
                          n_selected=r[4], nonfinite=r[5], status=r[6], path=r[7] & 0xFF,
                          negative=bool(r[7] & 0x100), redone=bool(r[7] & 0x200))
    out.thresh = torch.tensor([r[0]], dtype=torch.int32).view(torch.float32).item()
    return out


def _bin_edge_float(b, shift):
    bits = (b << shift) & 0x7FFFFFFF
    return torch.tensor([bits], dtype=torch.int32).view(torch.float32).item()


def _sampled_count(n, stride, phase=0):
    return len(range(phase, n, stride))


def _flat_views(views):
    out = []
    for g in views:
        L.require_dev(g)
        f = g.reshape(-1)
        if f.dtype != torch.float32:
            raise TypeError("selection scores must be fp32")
        L.require_contig(view=f)
        out.append(f)
    return out


def _flat_span(views):
    """The views as ONE flat tensor when they are back-to-back slices of the
    same storage (a bucket's per-param views usually are), else None."""
    first = views[0]
    store = first.untyped_storage()
    end = first.data_ptr()
    for g in views:
        if g.untyped_storage().data_ptr() != store.data_ptr() or g.data_ptr() != end:
            return None
        end += g.numel() * 4
    total = sum(g.numel() for g in views)
    return torch.empty(0, dtype=torch.float32, device=first.device).set_(
        store, first.storage_offset(), (total,), (1,))


def select_exact_device(views, k, tie_mode, masks=None):
    """Exact top-k over a list of flat fp32 views; returns (result, masks).
    Views are laid out back to back in chunk space, each on a fresh
    1024-element chunk, so flat-index order == view order then in-view order
    (the reference's catalog order)."""
    views = _flat_views(views)
    dev = views[0].device
    bases, nt = [], 0
    for g in views:
        bases.append(nt)
        nt += -(-g.numel() // _CHUNK)
    n_total = sum(g.numel() for g in views)
    if not (1 <= k <= n_total):
        raise ValueError(f"k={k} > N={n_total}" if k > n_total else f"k={k} < 1")
    ws_bytes = int(L.raw("sga_select_workspace_bytes", nt * _CHUNK))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    res = torch.empty(8, dtype=torch.int32, device=dev)
    st = L.stream()
    flat = None
    if masks is None and len(views) > 1:
        flat = _flat_span(views)
        if flat is None and n_total >= (1 << 20):
            # scattered views: one staging copy (8 B/elem) buys the one-sweep
            # select (5 B/elem) instead of five per-view passes (21 B/elem
            # and five launches per view)
            flat = torch.cat(views)
    if flat is not None:
        # adjacent slices of one buffer: flat-index order is the view order, so
        # the whole list is one array for the single-call entry point
        fmask = torch.empty(n_total, dtype=torch.uint8, device=dev)
        L.call("sga_select_topk", L.ptr(flat), n_total, k, tie_mode, L.ptr(fmask), L.ptr(res),
               L.ptr(ws), ws_bytes, st)
        out, off = [], 0
        for g in views:
            out.append(fmask[off:off + g.numel()])
            off += g.numel()
        return res, out
    if masks is None:
        masks = [torch.empty(g.numel(), dtype=torch.uint8, device=dev) for g in views]
    if len(views) == 1:
        # one contiguous array: the single-call entry point (sampled bracket
        # with the radix passes as the on-device fallback)
        L.call("sga_select_topk", L.ptr(views[0]), n_total, k, tie_mode, L.ptr(masks[0]),
               L.ptr(res), L.ptr(ws), ws_bytes, st)
        return res, masks
    L.call("sga_sel_begin", k, L.ptr(ws), ws_bytes, st)
    for level in range(3):
        for g in views:
            L.call("sga_sel_hist", L.ptr(g), g.numel(), level, L.ptr(ws), ws_bytes, st)
        L.call("sga_sel_scan", level, L.ptr(ws), ws_bytes, st)
    for g, b in zip(views, bases):
        L.call("sga_sel_count", L.ptr(g), g.numel(), b, L.ptr(ws), ws_bytes, st)
    L.call("sga_sel_tile_scan", max(nt, 1), tie_mode, L.ptr(ws), ws_bytes, st)
    for g, b, m in zip(views, bases, masks):
        L.call("sga_sel_mask", L.ptr(g), g.numel(), b, tie_mode, L.ptr(m), L.ptr(ws),
               ws_bytes, st)
    L.call("sga_sel_result", L.ptr(res), L.ptr(ws), ws_bytes, st)
    return res, masks


def select_masks_histogram(grads, k, comm_group=None, mode="exact",
                           global_allreduce=True):
    """``_histogram.py:161-216`` at world size 1 (no collective in this
    build): returns (threshold, per-view uint8 masks), ties all selected."""
    try:
        shift, nbins, stride = _HIST_MODES[mode]
    except KeyError:
        raise ValueError(f"unknown histogram_mode: {mode!r}") from None
    if mode == "exact":
        res, masks = select_exact_device(grads, k, L.TIE_ALL)
        return read_result(res).thresh, masks
    views = _flat_views(grads)
    dev = views[0].device
    hist = torch.zeros(nbins, dtype=torch.int64, device=dev)
    nf = torch.zeros(1, dtype=torch.int32, device=dev)
    st = L.stream()
    for g in views:
        L.call("sga_hist_topbits", L.ptr(g), g.numel(), shift, stride, 0, L.ptr(hist),
               nbins, L.ptr(nf), st)
    n_total = sum(g.numel() for g in views)
    n_sampled = sum(_sampled_count(g.numel(), stride) for g in views)
    r = max(1, round(n_sampled * (n_total - k + 1) / n_total))
    b = int(torch.searchsorted(torch.cumsum(hist, 0), r).item())
    masks = []
    for g in views:
        m = torch.empty(g.numel(), dtype=torch.uint8, device=dev)
        L.call("sga_mask_topbits_ge", L.ptr(g), g.numel(), shift, b, L.ptr(m), st)
        masks.append(m)
    return _bin_edge_float(b, shift), masks


def select_masks_exact_kthvalue(grads, k, comm_group=None):
    """``_exact.py:12-41`` at world size 1: same threshold and masks as the
    exact histogram tier, produced by the same device select."""
    res, masks = select_exact_device(grads, k, L.TIE_ALL)
    return read_result(res).thresh, masks


class HistogramSelect:
    """``_histogram.py:254-307`` (element granularity)."""

    def __init__(self, mode="exact", block_size=1, block_reduce="mean",
                 global_allreduce=True):
        if mode not in _HIST_MODES:
            raise ValueError(f"unknown histogram_mode: {mode!r} "
                             f"(expected one of {sorted(_HIST_MODES)})")
        if (not isinstance(block_size, int) or isinstance(block_size, bool)
                or block_size < 1 or block_size > 1024 or block_size & (block_size - 1)):
            raise ValueError(
                f"block_size must be a power of two in [1, 1024], got {block_size!r}")
        if block_reduce not in ("mean", "max"):
            raise ValueError(f"block_reduce must be 'mean' or 'max', got {block_reduce!r}")
        self.mode, self.block_size = mode, block_size
        self.block_reduce, self.global_allreduce = block_reduce, global_allreduce

    def select(self, grads, k, comm_group, warmup_target=None):
        if self.block_size == 1:
            return select_masks_histogram(grads, k, comm_group, mode=self.mode,
                                          global_allreduce=self.global_allreduce)
        # block mode (_histogram.py:291-307): select over per-block scores,
        # then expand the block masks back to element masks
        x = self.block_size
        k_blocks = max(1, int(round(k / x)))
        bviews = block_reduce_views(grads, x, self.block_reduce)
        thresh, bmasks = select_masks_histogram(bviews, k_blocks, comm_group, mode=self.mode,
                                                global_allreduce=self.global_allreduce)
        masks = []
        st = L.stream()
        for bm, g in zip(bmasks, grads):
            m = torch.empty(g.numel(), dtype=torch.uint8, device=g.device)
            L.call("sga_expand_blocks", L.ptr(bm), x, g.numel(), L.ptr(m), st)
            masks.append(m)
        return thresh, masks


def block_reduce_views(grads, x, reduce):
    """Per-view block scores: |g| reduced (mean | max) over contiguous
    x-element blocks, the tail block over its real length
    (``_histogram.py:219-251``)."""
    out = []
    st = L.stream()
    for g in _flat_views(grads):
        nb = -(-g.numel() // x)
        o = torch.empty(nb, dtype=torch.float32, device=g.device)
        L.call("sga_block_reduce", L.ptr(g), g.numel(), x, 0 if reduce == "mean" else 1,
               L.ptr(o), st)
        out.append(o)
    return out


def count_on(mask_u8):
    """Number of set bytes of a device uint8 mask (``_adaptive.py:44-51``)."""
    n = mask_u8.numel()
    if n == 0:
        return 0
    L.require_dev(mask_u8)
    dev = mask_u8.device
    counts = torch.empty(int(L.raw("sga_mask_chunks", n)), dtype=torch.int32, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    L.call("sga_mask_count", L.ptr(mask_u8), n, L.ptr(counts), L.ptr(total), L.stream())
    return int(total.item())


def threshold_masks(grads, tau):
    """``|g| >= tau`` uint8 masks per view and their total set count in one
    sweep each (``_adaptive.py:44-66``: ``_threshold_masks`` + ``_count_on``)."""
    views = _flat_views(grads)
    dev = views[0].device
    count = torch.zeros(1, dtype=torch.int64, device=dev)
    masks = []
    st = L.stream()
    for g in views:
        m = torch.empty(g.numel(), dtype=torch.uint8, device=dev)
        L.call("sga_mask_abs_ge", L.ptr(g), g.numel(), L.f32(tau), L.ptr(m), L.ptr(count), st)
        masks.append(m)
    return masks, int(count.item())


def adapt_threshold(thresh, measured_ratio, target_ratio, gain=0.5, max_up=1.15,
                    max_down=0.9, band=0.01):
    """One multiplicative dead-band update of tau (``_adaptive.py:28-41``)."""
    if abs(measured_ratio - target_ratio) <= band:
        return thresh
    factor = (measured_ratio / target_ratio) ** gain
    return thresh * min(max(factor, max_down), max_up)


_ADAPT_BAND = 0.01            # _adaptive.py:21-24


class AdaptiveTau:
    """Persistent-threshold selector (``_adaptive.py:79-187``).

    While warming up (and whenever the threshold has collapsed) the mask
    comes from the histogram select in ``warmup_mode``; afterwards one
    ``|g| >= tau`` sweep produces masks and their count, and tau follows the
    measured ratio by the dead-band multiplicative rule.
    """

    def __init__(self, ratio_percent, warmup_syncs, warmup_mode, global_allreduce=True):
        if warmup_mode not in _HIST_MODES:
            raise ValueError(f"unknown adaptive_warmup_mode: {warmup_mode!r} "
                             f"(expected one of {sorted(_HIST_MODES)})")
        if not isinstance(global_allreduce, bool):
            raise ValueError(f"global_allreduce must be a bool, got {global_allreduce!r}")
        self.target_ratio = ratio_percent / 100.0
        self.warmup_syncs = warmup_syncs
        self.warmup_mode = warmup_mode
        self.global_allreduce = global_allreduce
        self.tau = None
        self.warmup_passed = 0

    def warmup_sync_target(self, start_iter, period):
        """Gated warmup selects left for a selection that starts at
        ``start_iter`` (``_adaptive.py:104-122``); a boundary exactly on the
        window edge is post-warmup."""
        if self.warmup_syncs is None:
            return None
        return max(0, (self.warmup_syncs * period - 1 - start_iter) // period)

    def _bootstrap(self, grads, k, comm_group):
        thresh, masks = select_masks_histogram(grads, k, comm_group, mode=self.warmup_mode,
                                               global_allreduce=self.global_allreduce)
        # bin 0's edge is 0.0, which the multiplicative rule can never leave
        self.tau = thresh if thresh > 0.0 else _bin_edge_float(
            1, _HIST_MODES[self.warmup_mode][0])
        return masks

    @staticmethod
    def _measured(masks, grads):
        return sum(count_on(m) for m in masks) / sum(g.numel() for g in grads)

    def select(self, grads, k, comm_group, warmup_target):
        if warmup_target is not None:
            required = max(warmup_target, 1)
        else:
            required = max(self.warmup_syncs if self.warmup_syncs is not None else 1, 1)
        if self.tau is None or self.warmup_passed < required:
            masks = self._bootstrap(grads, k, comm_group)
            hit = abs(self._measured(masks, grads) - self.target_ratio) <= _ADAPT_BAND
            self.warmup_passed = self.warmup_passed + 1 if hit else 0
            return self.tau, masks
        masks, on = threshold_masks(grads, self.tau)
        measured = on / sum(g.numel() for g in grads)
        if measured == 0.0 or self.tau <= 0.0:
            masks = self._bootstrap(grads, k, comm_group)
            return self.tau, masks
        used = self.tau
        self.tau = adapt_threshold(used, measured, self.target_ratio)
        return used, masks


class ExactKthvalue:
    def select(self, grads, k, comm_group, warmup_target=None):
        return select_masks_exact_kthvalue(grads, k, comm_group)


class TopkSelection:
    """``selection/topk.py:59-167``; reads the ``sga_selection_*`` flags from
    the args singleton, like the reference (``:59-60``)."""

    def __init__(self):
        args = get_args()
        self.method = args.sga_selection_method
        self.ratio_percent = float(args.sga_selection_ratio_percent)
        assert 0.0 < self.ratio_percent < 100.0, (
            f"ratio_percent must be in (0, 100), got {self.ratio_percent}")
        if self.method == "histogram":
            self._impl = HistogramSelect(
                getattr(args, "sga_selection_histogram_mode", "exact"),
                block_size=int(getattr(args, "sga_selection_block_size", 1)),
                block_reduce=getattr(args, "sga_selection_block_reduce", "mean"),
                global_allreduce=bool(getattr(
                    args, "sga_selection_topk_histogram_add_global_allreduce", False)))
        elif self.method == "exact":
            self._impl = ExactKthvalue()
        elif self.method == "adaptive":
            ws = getattr(args, "sga_selection_adaptive_warmup_syncs", None)
            self._impl = AdaptiveTau(
                self.ratio_percent, int(ws) if ws is not None else None,
                getattr(args, "sga_selection_adaptive_warmup_mode", "fast"),
                global_allreduce=bool(getattr(
                    args, "sga_selection_topk_histogram_add_global_allreduce", False)))
        else:
            raise ValueError("sga_selection_method must be adaptive|exact|histogram "
                             f"(got {self.method!r})")
        self.last_threshold = None

    @property
    def block_size(self):
        return getattr(self._impl, "block_size", 1)

    @property
    def tau(self):
        return getattr(self._impl, "tau", None)

    @property
    def warmup_passed(self):
        return getattr(self._impl, "warmup_passed", None)

    def k_for(self, n_total):
        return max(1, int(round(n_total * self.ratio_percent / 100.0)))

    def warmup_sync_target(self, start_iter, period):
        hook = getattr(self._impl, "warmup_sync_target", None)
        return hook(start_iter, period) if callable(hook) else None

    def select(self, ctx):
        k = self.k_for(sum(g.numel() for g in ctx.grad_views))
        thresh, masks = self._impl.select(ctx.grad_views, k,
                                          getattr(ctx, "comm_group", None),
                                          getattr(ctx, "warmup_target", None))
        self.last_threshold = thresh
        return masks
