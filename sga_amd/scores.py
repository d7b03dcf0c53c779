"""Score registry of ``sga/plugins/scores.py`` on MI355X: same names, same
``get_score_spec(name).formula(...)`` call shape, one fused HIP pass per
formula instead of a chain of torch elementwise ops."""
from dataclasses import dataclass
from typing import Callable

import torch

from . import _lib as L

SCORE_MAP = {"update": 0, "abs_g": 1, "abs_m": 2, "coi": 3}   # adamw.py:75-80
# Two benchmark scores OUTSIDE the reference's registry (not returned by
# score_names / get_score_spec): the fused step and the replay group accept
# them by these names.  abs_g_blind ranks by the recorded gradient alone while
# the residual keeps accumulating; abs_gr_over_sqrt_v is |g + r| / sqrt(v + eps).
EXTRA_SCORE_MAP = {"abs_g_blind": 4, "abs_gr_over_sqrt_v": 5}
STEP_SCORE_MAP = dict(SCORE_MAP, **EXTRA_SCORE_MAP)


@dataclass(frozen=True)
class ScoreSpec:
    formula: Callable[..., torch.Tensor]
    doc: str
    scratch: bool = False


_DOCS = {
    "update": "the SIGNED weight update wd*w + U(g); consumers rank by absolute value",
    "abs_g": "|g| of the committed, fully-synced gradient",
    "abs_m": "|m| of the pre-commit first moment",
    "coi": "counterfactual optimizer impact |U(g) - U(0)|",
}


def device_formula(score_id, w, m, v, g, b1, b2, eps, wd, bc1, bc2, absolute=False,
                   optimizer="adamw", out=None, update_includes_wd=True):
    """One-pass registry formula on flat fp32 device tensors."""
    if optimizer not in ("adamw", "adams"):
        raise ValueError(f"Unknown SGA optimizer '{optimizer}' for the score "
                         "formulas (registered: adamw, adams)")
    ref = g if score_id != 2 else m
    L.require_dev(w, m, v, g)
    n = ref.numel()
    shape = ref.shape
    flat = [None if t is None else t.reshape(-1) for t in (w, m, v, g)]
    for t in flat:
        if t is not None:
            if t.dtype != torch.float32:
                raise TypeError("score formulas take fp32 tensors")
            L.require_contig(t=t)
    if out is None:
        out = torch.empty(n, dtype=torch.float32, device=ref.device)
    flags = (1 if optimizer == "adams" else 0) | (0 if update_includes_wd else 2)   # SGA_SF_*
    L.call("sga_score_formula", score_id, L.ptr(flat[0]), L.ptr(flat[1]), L.ptr(flat[2]),
           L.ptr(flat[3]), L.ptr(out), n, L.f32(b1), L.f32(1.0 - b1), L.f32(b2),
           L.f32(1.0 - b2), L.f32(wd), L.f32(bc1), L.f32(bc2), L.f32(eps),
           1 if absolute else 0, flags, L.stream())
    return out.view(shape)


def _mk(name):
    sid = SCORE_MAP[name]

    def formula(w, m, v, g, beta1, beta2, eps, weight_decay, bias_correction1,
                bias_correction2, update_includes_wd=True, optimizer="adamw",
                scratch=None):
        return device_formula(sid, w, m, v, g, beta1, beta2, eps, weight_decay,
                              bias_correction1, bias_correction2, optimizer=optimizer,
                              update_includes_wd=update_includes_wd)
    return formula


_SCORES = {name: ScoreSpec(formula=_mk(name), doc=_DOCS[name],
                           scratch=name in ("update", "coi")) for name in SCORE_MAP}


def get_score_spec(name):
    """``sga/plugins/scores.py:119-126``"""
    try:
        return _SCORES[name]
    except KeyError:
        raise ValueError(
            f"Unknown SGA score '{name}'. Registered: {score_names()}") from None


def score_names():
    return sorted(_SCORES)
