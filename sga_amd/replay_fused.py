"""Replay-side selectors of ``sga/replay_fused.py`` on MI355X at world == 1."""
import torch

from . import _lib as L
from .replay import select_topk_flat
from .selection import _HIST_MODES, _bin_edge_float, _sampled_count


def shard_bounds(N, world):
    """``replay_fused.py:274-283``"""
    base, rem = divmod(N, world)
    out, lo = [], 0
    for r in range(world):
        hi = lo + base + (1 if r < rem else 0)
        out.append((lo, hi))
        lo = hi
    return out


def shard_select(score, k, comms=None, prof=None):
    """Exact global top-k with the tie layer filled in flat-index order
    (``replay_fused.py:290-402``); one shard, no collectives.  Raises on
    non-finite scores like the reference."""
    if comms is not None and getattr(comms, "distributed", False):
        raise NotImplementedError("this build runs one shard on one GPU")
    L.require_dev(score)
    flat = score.reshape(-1)
    if k > flat.numel():
        raise ValueError(f"k={k} > N={flat.numel()}")
    try:
        return select_topk_flat(flat, k)
    except ValueError as e:
        if "finite" in str(e):
            raise ValueError(
                "shard_select requires finite scores (NaN/Inf would land in the top "
                "bins and silently pollute the topk)") from None
        raise


def shard_select_balanced(score, k, comms, entries):
    """Balanced-histogram replay select (``replay_fused.py:405-489``): stride-8
    subsample per param view with the param-relative phase, crossing bin from
    the integer closed form, mask = top16 >= bin."""
    L.require_dev(score)
    flat = score.reshape(-1)
    if not bool(torch.isfinite(flat).all().item()):
        raise ValueError("shard_select_balanced requires finite scores (NaN/Inf land in "
                         "the top bit-pattern bins and would be selected; parity is "
                         "undefined there)")
    shift, nbins, stride = _HIST_MODES["balanced"]
    hist = torch.zeros(nbins, dtype=torch.int64, device=flat.device)
    n_total = n_sampled = 0
    st = L.stream()
    for e in entries:
        v = flat[e["a"]:e["a"] + e["n"]]
        phase = (-int(e.get("p_off", 0))) % stride
        n_total += v.numel()
        n_sampled += _sampled_count(v.numel(), stride, phase)
        L.call("sga_hist_topbits", L.ptr(v), v.numel(), shift, stride, phase, L.ptr(hist),
               nbins, None, st)
    r = max(1, round(n_sampled * (n_total - k + 1) / n_total))
    b = int(torch.searchsorted(torch.cumsum(hist, 0), r).item())
    mask = torch.empty(flat.numel(), dtype=torch.bool, device=flat.device)
    L.call("sga_mask_topbits_ge", L.ptr(flat), flat.numel(), shift, b,
           L.ptr(mask.view(torch.uint8)), st)
    return mask, _bin_edge_float(b, shift)
