"""Oracle top-k selection (test infrastructure; torch CPU).

Two tie semantics exist in the reference and both are restated here:

* replay / north-star: EXACTLY k coordinates, boundary ties filled in
  ascending flat-index order (``sga/replay.py:518-572``,
  ``sga/replay_fused.py:290-402``);
* online plugin: every coordinate with ``|s| >= thresh`` (count >= k)
  (``sga/plugins/selection/_histogram.py:161-201``, ``_exact.py:12-41``).

The threshold is the exact k-th largest magnitude.  It is found the way the
reference finds it -- a histogram over the top 16 bits of the sign-stripped
fp32 pattern, then a k-th value inside the crossing bin -- because
non-negative floats order like their integer patterns.
"""
import torch

HIST_SHIFT = 16            # _histogram.py:50
HIST_BINS = 32769          # _histogram.py:51
HIST_SHIFT_COARSE = 19     # _histogram.py:53
HIST_BINS_COARSE = 4097    # _histogram.py:54
SAMPLE_STRIDE = 8          # _histogram.py:57
HIST_MODES = {             # _histogram.py:68-72
    "exact": (HIST_SHIFT, HIST_BINS, 1),
    "balanced": (HIST_SHIFT, HIST_BINS, SAMPLE_STRIDE),
    "fast": (HIST_SHIFT_COARSE, HIST_BINS_COARSE, SAMPLE_STRIDE),
}


def k_for(n_total, ratio_percent):
    """Online plugin k (``selection/topk.py:111-112``)."""
    return max(1, int(round(n_total * ratio_percent / 100.0)))


def replay_k(n_total, ratio_percent):
    """Replay k (``replay_fused.py:1336``): note the different op order."""
    return max(1, int(round(ratio_percent / 100.0 * n_total)))


def abs_bit_top(t, shift=HIST_SHIFT):
    """Top bits of the sign-stripped pattern (``_histogram.py:75-77``)."""
    return (t.contiguous().view(torch.int32) & 0x7FFFFFFF) >> shift


def bin_edge_float(b, shift):
    """Lower edge of bin ``b`` as a float (``_histogram.py:85-88``)."""
    bits = (b << shift) & 0x7FFFFFFF
    return torch.tensor([bits], dtype=torch.int32).view(torch.float32).item()


def sampled_count(n, stride, phase=0):
    """How many of ``phase, phase+stride, ...`` fall below n
    (``_histogram.py:91-94``)."""
    if n <= phase:
        return 0
    return (n - phase + stride - 1) // stride


def build_histogram(views, shift, nbins, stride, phases=None):
    """int64 histogram of ``abs_bit_top`` over (a stride subsample of) every
    view (``_histogram.py:97-112``); ``phases`` gives the per-view first
    sampled index (``replay_fused.py:463-470``), default 0."""
    hist = torch.zeros(nbins, dtype=torch.int64)
    for i, g in enumerate(views):
        top = abs_bit_top(g.reshape(-1), shift)
        if stride > 1:
            top = top[(phases[i] if phases else 0)::stride]
        hist += torch.bincount(top, minlength=nbins)
    return hist


def _crossing(hist, k, world=1):
    """(bin, n_above) of the k-th largest (``_histogram.py:138-142``)."""
    cum = torch.cumsum(hist, 0)
    total = int(cum[-1])
    r = total - k * world + 1
    b = int(torch.searchsorted(cum, r))
    n_above = (total - int(cum[b])) // world
    return b, n_above, total


def hist_threshold(t, k):
    """Exact k-th largest of a non-negative flat fp32 vector
    (``replay.py:518-535``)."""
    t = t.reshape(-1)
    top = abs_bit_top(t)
    hist = torch.bincount(top, minlength=HIST_BINS)
    b, n_above, _ = _crossing(hist, k)
    cand = t[top == b].abs()
    kk = cand.numel() - (k - n_above) + 1
    if cand.numel() == 0 or not (1 <= kk <= cand.numel()):
        raise RuntimeError(
            f"hist select math out of range: cand={cand.numel()} kk={kk}")
    return float(torch.kthvalue(cand, kk).values)


def select_topk_flat(t, k):
    """Exactly-k mask with lowest-index tie fill + threshold
    (``replay.py:538-572``)."""
    t = t.reshape(-1)
    n = t.numel()
    if k > n:
        raise ValueError(f"k={k} > N={n}")
    if n and float(t.min()) < 0.0:
        raise ValueError("select_topk_flat requires non-negative scores")
    if not bool(torch.isfinite(t).all()):
        raise ValueError("select_topk_flat requires finite scores (NaN/Inf "
                         "would land in the top bins and silently pollute "
                         "the topk)")
    thresh = hist_threshold(t, k)
    sel = t > thresh
    need = k - int(sel.sum())
    if need > 0:
        ties = torch.nonzero(t == thresh).reshape(-1)
        sel[ties[:need]] = True
    if int(sel.sum()) != k:
        raise RuntimeError("internal tie-break error")
    return sel, thresh


def select_threshold_views(views, k, shift=HIST_SHIFT, world=1):
    """Exact threshold over a list of signed views
    (``_histogram.py:126-158``)."""
    hist = build_histogram(views, shift, HIST_BINS, 1)
    hist = hist * world
    b, n_above, _ = _crossing(hist, k, world)
    cands = [g.reshape(-1)[abs_bit_top(g.reshape(-1), shift) == b].abs()
             for g in views]
    cand = torch.cat(cands)
    assert cand.numel() > 0, "histogram select found no candidates"
    kk = cand.numel() - (k - n_above) + 1
    assert 1 <= kk <= cand.numel()
    return torch.kthvalue(cand, kk).values.item()


def balanced_crossing_bin(hist, n_total, n_sampled, k, replicas=1):
    """Approximate crossing bin (``_histogram.py:115-123``)."""
    r = max(1, round(n_sampled * (n_total - k + 1) / n_total)) * replicas
    return int(torch.searchsorted(torch.cumsum(hist, 0), r))


def select_masks_histogram(views, k, mode="exact"):
    """Per-view uint8 masks, ties ALL selected
    (``_histogram.py:161-216``, world == 1)."""
    try:
        shift, nbins, stride = HIST_MODES[mode]
    except KeyError:
        raise ValueError(f"unknown histogram_mode: {mode!r}") from None
    if mode == "exact":
        thresh = select_threshold_views(views, k, shift)
        return thresh, [(g.reshape(-1).abs() >= thresh).to(torch.uint8)
                        for g in views]
    hist = build_histogram(views, shift, nbins, stride)
    n_total = sum(g.numel() for g in views)
    n_sampled = sum(sampled_count(g.numel(), stride) for g in views)
    b = balanced_crossing_bin(hist, n_total, n_sampled, k)
    masks = [(abs_bit_top(g.reshape(-1), shift) >= b).to(torch.uint8)
             for g in views]
    return bin_edge_float(b, shift), masks


def select_masks_exact_kthvalue(views, k):
    """cat + kthvalue control path (``_exact.py:12-41``)."""
    a = torch.cat([g.reshape(-1) for g in views]).abs()
    thresh = torch.kthvalue(a, a.numel() - k + 1).values.item()
    m = (a >= thresh).to(torch.uint8)
    out, off = [], 0
    for g in views:
        out.append(m[off:off + g.numel()])
        off += g.numel()
    return thresh, out


def shard_select_balanced(score, k, entries):
    """Replay twin of the balanced select on a flat score with per-param
    entries ``{"a", "n", "p_off"}`` (``replay_fused.py:405-489``, world 1)."""
    if not bool(torch.isfinite(score).all()):
        raise ValueError("shard_select_balanced requires finite scores")
    shift, nbins, stride = HIST_MODES["balanced"]
    views, phases = [], []
    n_total = n_sampled = 0
    for e in entries:
        v = score[e["a"]:e["a"] + e["n"]]
        ph = (-int(e.get("p_off", 0))) % stride
        views.append(v)
        phases.append(ph)
        n_total += v.numel()
        n_sampled += sampled_count(v.numel(), stride, ph)
    hist = build_histogram(views, shift, nbins, stride, phases)
    b = balanced_crossing_bin(hist, n_total, n_sampled, k)
    return abs_bit_top(score, shift) >= b, bin_edge_float(b, shift)


def block_reduce_views(views, x, reduce):
    """|g| reduced over x-element blocks, tail over its real length
    (``_histogram.py:219-251``)."""
    out = []
    for g in views:
        c = g.reshape(-1).abs()
        if c.numel() == 0:
            out.append(torch.empty(0))
            continue
        nb, rem = divmod(c.numel(), x)
        parts = []
        if nb:
            b = c[:nb * x].view(nb, x)
            parts.append(b.mean(dim=1) if reduce == "mean" else b.amax(dim=1))
        if rem:
            t = c[nb * x:]
            parts.append((t.mean() if reduce == "mean" else t.amax()).reshape(1))
        out.append(torch.cat(parts))
    return out


def select_masks_blocks(views, k, x, reduce="mean", mode="exact"):
    """Block-granular histogram select (``_histogram.py:291-307``)."""
    k_blocks = max(1, int(round(k / x)))
    bviews = block_reduce_views(views, x, reduce)
    thresh, bmasks = select_masks_histogram(bviews, k_blocks, mode=mode)
    return thresh, [bm.repeat_interleave(x)[:g.numel()] for bm, g in zip(bmasks, views)]


def block_idx_from_mask(mask_u8, spans, x):
    """Block starts with ANY set byte, per span (``support.py:102-142``)."""
    out = []
    m = mask_u8.tolist()
    for start, end in spans:
        for lo in range(start, end, x):
            if any(m[lo:min(lo + x, end)]):
                out.append(lo)
    return torch.tensor(out, dtype=torch.int32)


ADAPT_BAND = 0.01          # _adaptive.py:21
ADAPT_LOG_GAIN = 0.5       # _adaptive.py:22
ADAPT_MAX_UP = 1.15        # _adaptive.py:23
ADAPT_MAX_DOWN = 0.9       # _adaptive.py:24


def adapt_threshold(thresh, measured, target):
    """Dead-band multiplicative tau update (``_adaptive.py:27-41``)."""
    if abs(measured - target) <= ADAPT_BAND:
        return thresh
    f = (measured / target) ** ADAPT_LOG_GAIN
    return thresh * min(max(f, ADAPT_MAX_DOWN), ADAPT_MAX_UP)


class AdaptiveTau:
    """Persistent-threshold selector state machine (``_adaptive.py:79-187``,
    world 1)."""

    def __init__(self, ratio_percent, warmup_syncs, warmup_mode):
        self.target = ratio_percent / 100.0
        self.warmup_syncs = warmup_syncs
        self.mode = warmup_mode
        self.tau = None
        self.warmup_passed = 0

    def warmup_sync_target(self, start_iter, period):
        if self.warmup_syncs is None:
            return None
        return max(0, (self.warmup_syncs * period - 1 - start_iter) // period)

    def _boot(self, views, k):
        thresh, masks = select_masks_histogram(views, k, self.mode)
        self.tau = thresh if thresh > 0.0 else bin_edge_float(1, HIST_MODES[self.mode][0])
        return masks

    def select(self, views, k, warmup_target=None):
        n = sum(g.numel() for g in views)
        required = max(warmup_target if warmup_target is not None else
                       (self.warmup_syncs if self.warmup_syncs is not None else 1), 1)
        if self.tau is None or self.warmup_passed < required:
            masks = self._boot(views, k)
            r = sum(int(m.sum()) for m in masks) / n
            self.warmup_passed = self.warmup_passed + 1 if abs(r - self.target) <= ADAPT_BAND else 0
            return self.tau, masks
        masks = [(g.reshape(-1).abs() >= self.tau).to(torch.uint8) for g in views]
        r = sum(int(m.sum()) for m in masks) / n
        if r == 0.0 or self.tau <= 0.0:
            masks = self._boot(views, k)
            return self.tau, masks
        used = self.tau
        self.tau = adapt_threshold(used, r, self.target)
        return used, masks
