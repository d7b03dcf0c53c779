"""Replay primitives of ``sga/replay.py`` on MI355X: exact-k selection with
lowest-index tie fill, the in-place commit dispatcher, clip coefficient."""
import math

import torch

from . import _lib as L
from . import replay_kernels as K
from .selection import read_result, select_exact_device

OPTIMIZERS = ("adamw", "adams")
ADAMS_BIAS_CORRECTION = 1.0


# Declared dtypes of a replay run (``sga/replay.py:96-119``): the scans of this build hold their
# state in fp32; fp64 names the reference's host-side self-check, which is not a scan.
REPLAY_DTYPES = {"fp32": torch.float32, "fp64": torch.float64}


def resolve_replay_dtype(value):
    try:
        return REPLAY_DTYPES[value]
    except (KeyError, TypeError):
        raise ValueError(f"--replay-dtype must be one of {sorted(REPLAY_DTYPES)}, "
                         f"got {value!r}") from None


def require_scan_dtypes(replay_dtype, norm_dtype):
    """Scans are fp32-only, as in the reference (``sga/replay.py:109-119``)."""
    resolve_replay_dtype(replay_dtype)
    if norm_dtype not in REPLAY_DTYPES:
        raise ValueError(f"--norm-dtype must be one of {sorted(REPLAY_DTYPES)}, "
                         f"got {norm_dtype!r}")
    if replay_dtype != "fp32" or norm_dtype != "fp32":
        raise ValueError("offline scans require --replay-dtype fp32 and --norm-dtype fp32; "
                         "fp64 is reserved for --self-check")


def _bc_pair(optimizer, count, b1, b2):
    """``sga/replay.py:132-137``"""
    if optimizer == "adamw":
        return 1.0 - b1 ** count, 1.0 - b2 ** count
    return ADAMS_BIAS_CORRECTION, ADAMS_BIAS_CORRECTION


def coef_dense_for(meta):
    """``sga/replay.py:628-645``"""
    clip = float(meta.get("clip_grad", 0.0))
    norm = float(meta.get("grad_norm", float("nan")))
    if clip <= 0.0:
        return 1.0, "clipping_disabled"
    if not math.isfinite(norm) or norm <= 0.0:
        return 1.0, "grad_norm_unavailable"
    return min(clip / (norm + 1.0e-6), 1.0), None


def select_topk_flat(t, k, check=True):
    """Exact top-k of a non-negative finite fp32 device vector; boundary ties
    go to the lowest flat indices (``sga/replay.py:538-572``).  Returns
    (bool mask, threshold).  The whole select runs on the device; the single
    host read fetches the threshold and the rejection counters."""
    L.require_dev(t)
    flat = t.reshape(-1)
    n = flat.numel()
    if k > n:
        raise ValueError(f"k={k} > N={n}")
    mask = torch.empty(n, dtype=torch.bool, device=flat.device)
    res, _ = select_exact_device([flat], k, L.TIE_LOWEST_INDEX,
                                 masks=[mask.view(torch.uint8)])
    r = read_result(res)
    if check:
        if r.nonfinite:
            raise ValueError("select_topk_flat requires finite scores (NaN/Inf would "
                             "land in the top bins and silently pollute the topk)")
        if r.negative:        # seen by the select's own sweep: no pass of its own, no second sync
            raise ValueError("select_topk_flat requires non-negative scores")
    if r.n_selected != k:
        raise RuntimeError(f"internal tie-break error: selected {r.n_selected} != {k}")
    return mask, r.thresh


def hist_threshold(t, k):
    """Exact k-th largest value (``sga/replay.py:518-535``)."""
    return select_topk_flat(t, k, check=False)[1]


def _opt_step_inplace(q, m, v, w, lab, lr, wd, b1, b2, bc1c, bc2c, eps,
                      optimizer="adamw", inactive=None, lr_inactive=None):
    """``sga/replay.py:732-744``"""
    if (inactive is None) != (lr_inactive is None):
        raise ValueError(
            "inactive and lr_inactive come as a pair (the boundary dual-lr split "
            f"needs both; got inactive={inactive is not None}, "
            f"lr_inactive={lr_inactive!r})")
    K.opt_step_inplace(q, m, v, w, lab, lr, wd, b1, b2, bc1c, bc2c, eps,
                       optimizer=optimizer, inactive=inactive, lr_inactive=lr_inactive)


def score_formula(name, w, m, v, g, b1, b2, eps, wd, bc1, bc2, optimizer,
                  update_includes_wd=False):
    """``sga/replay.py:486-505``"""
    from .scores import SCORE_MAP, device_formula
    if name not in SCORE_MAP:
        raise ValueError(f"Unknown SGA score '{name}'. Registered: {sorted(SCORE_MAP)}")
    return device_formula(SCORE_MAP[name], w, m, v, g, b1, b2, eps, wd, bc1, bc2,
                          optimizer=optimizer, update_includes_wd=update_includes_wd)
