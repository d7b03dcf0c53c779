"""Oracle for the replay commit and the fused group step (test
infrastructure; torch CPU).

Follows ``sga/replay.py:628-744`` (clip coefficient, AdamW/AdamS in-place
commits, dual-lr split) and the per-step state machine of
``sga/replay_fused.py:1607-1914`` at world == 1 (fold -> pass 1 norms ->
coefficients -> pass 2 boundary reselect -> pass 3 commit + residual).
"""
import math

import torch

from . import ieee
from . import scores as S
from . import select as SEL


def bc_pair(optimizer, count, b1, b2):
    """(replay.py:132-137)"""
    if optimizer == "adamw":
        return 1.0 - b1 ** count, 1.0 - b2 ** count
    return 1.0, 1.0


def coef_dense_for(clip_grad, grad_norm):
    """Dense-run clip coefficient from the trace meta (replay.py:628-645)."""
    if clip_grad <= 0.0:
        return 1.0
    if not math.isfinite(grad_norm) or grad_norm <= 0.0:
        return 1.0
    return min(clip_grad / (grad_norm + 1.0e-6), 1.0)


def apply_lr_split(w, upd, lr, lr_inactive, inactive, wd):
    """``w -= where(inactive, lr_i, lr) * (wd*w + upd)`` (replay.py:674-684)."""
    step = torch.full_like(w, lr)
    step.masked_fill_(inactive, lr_inactive)
    full = w * wd
    full.add_(upd)
    w.addcmul_(full, step, value=-1.0)


def opt_step_inplace(q, m, v, w, lab, lr, wd, b1, b2, bc1c, bc2c, eps,
                     optimizer="adamw", inactive=None, lr_inactive=None):
    """In-place AdamW / AdamS commit (replay.py:687-744)."""
    if (inactive is None) != (lr_inactive is None):
        raise ValueError("inactive and lr_inactive come as a pair")
    if optimizer == "adams":
        v.copy_(m)
        v.mul_(m)
        v.mul_(b2)
        v.addcmul_(q, q, value=1.0 - b2)
        m.mul_(b1).add_(q, alpha=1.0 - b1)
    else:
        m.mul_(b1).add_(q, alpha=1.0 - b1)
        v.mul_(b2).addcmul_(q, q, value=1.0 - b2)
    mh = m / bc1c
    vh = ieee.sqrt(v / bc2c)
    upd = mh / (vh + eps)
    if inactive is None:
        w.mul_(1.0 - lr * wd).add_(upd, alpha=-lr)
    else:
        apply_lr_split(w, upd, lr, lr_inactive, inactive, wd)
    if lab is not None:
        lab.addcmul_(upd, upd, value=lr * lr)


class Config:
    """One replay arm: (score, ratio %, cycle length T, optimizer, fold,
    dual-lr scale) -- ``replay_fused.py:1501-1505``."""

    def __init__(self, score, ratio, T, optimizer="adamw", fold=False,
                 dual_lr=1.0):
        self.score, self.ratio, self.T = score, ratio, T
        self.optimizer, self.fold, self.dual_lr = optimizer, fold, dual_lr


def group_replay(entries, w0, m0, v0, sel0, configs, g_steps, metas, t0,
                 horizons=(), snapshots=None, norm_chunk=None, coef_hook=None,
                 trace=None, selection_semantics="topk"):
    """Fused-replay group loop on one shard (replay_fused.py:1536-1914).

    entries : list of dicts {"a": flat offset, "n": numel, "b1","b2","eps",
              "wd", "lr_group"} (ShardParams, replay_fused.py:251-271)
    w0/m0/v0: flat fp32 branch-point state
    sel0    : list (per config) of flat bool masks (branch selection)
    g_steps : list of flat fp32 recorded gradients (post-clip, as logged)
    metas   : per step {"clip_grad", "grad_norm", "lr"}
    coef_hook(si, ci, coef) -> coef lets a test substitute the clip
    coefficient (e.g. the device's bits) so everything downstream is compared
    on identical inputs; trace (a list) receives (si, ci, qn2, coef).
    selection_semantics: what a boundary re-selects with ("topk" |
    "balanced-histogram", replay_fused.py:1340-1344, 1805-1812).
    Returns per-config dict with final w, m, v, res, sel and the per-horizon
    distances ``||w - snapshot||``.
    """
    N = w0.numel()
    W = len(g_steps)
    st = [{"w": w0.clone(), "m": m0.clone(), "v": v0.clone(),
           "res": torch.zeros(N), "sel": sel0[ci].clone()}
          for ci in range(len(configs))]
    dist_at = [dict() for _ in configs]
    ks = {c.ratio: SEL.replay_k(N, c.ratio) for c in configs}
    chunk = norm_chunk or N
    for si in range(W):
        meta = metas[si]
        clip = float(meta.get("clip_grad", 0.0))
        coef_dense = coef_dense_for(clip, float(meta.get("grad_norm",
                                                         float("nan"))))
        count = t0 + si + 1
        bnd = [si % c.T == 0 for c in configs]
        if si > 0:                                   # fold (:1632-1636)
            for ci, c in enumerate(configs):
                if bnd[ci] and c.fold:
                    st[ci]["res"].div_(float(c.T))
        gd = g_steps[si].float() / coef_dense        # (:1664)
        out_sel = {}
        # pass 1: fp32 chunk sums accumulated in a Python double (:1682-1720)
        coefs = []
        for ci, c in enumerate(configs):
            s = st[ci]
            qn2 = 0.0
            for e in entries:
                for a in range(e["a"], e["a"] + e["n"], chunk):
                    b = min(e["a"] + e["n"], a + chunk)
                    qp = (gd[a:b] + s["res"][a:b]) if bnd[ci] \
                        else gd[a:b] * s["sel"][a:b]
                    qn2 += float((qp * qp).sum())
            coef = 1.0
            if clip > 0.0:
                coef = min(1.0, clip / (math.sqrt(qn2) + 1.0e-6))
            if trace is not None:
                trace.append((si, ci, qn2, coef))
            if coef_hook is not None:
                coef = coef_hook(si, ci, coef)
            coefs.append(coef)
        # pass 2: boundary reselect (:1752-1825)
        for ci, c in enumerate(configs):
            if not (bnd[ci] and si > 0 and si + 1 < W):
                continue
            s = st[ci]
            score = torch.empty(N)
            for e in entries:
                a, b = e["a"], e["a"] + e["n"]
                bc1c, bc2c = bc_pair(c.optimizer, count, e["b1"], e["b2"])
                q = (gd[a:b] + s["res"][a:b]) * coefs[ci]
                # the residual-blind variant (build-side) ranks q without its residual term
                blind = gd[a:b] * coefs[ci]
                score[a:b] = S.step_score(c.score, s["w"][a:b], s["m"][a:b],
                                          s["v"][a:b], q, blind, e["b1"],
                                          e["b2"], e["eps"], e["wd"], bc1c,
                                          bc2c, c.optimizer).float()
            if selection_semantics == "balanced-histogram":
                newsel, _ = SEL.shard_select_balanced(score, ks[c.ratio],
                                                      entries)
            elif selection_semantics == "topk":
                newsel, _ = SEL.select_topk_flat(score, ks[c.ratio])
            else:
                raise ValueError(f"unknown selection semantics "
                                 f"{selection_semantics!r}")
            if c.dual_lr != 1.0:
                out_sel[ci] = s["sel"]
            s["sel"] = newsel
        # pass 3: commit + residual (:1836-1889)
        hz = (si + 1) if (si + 1) in horizons else None
        for ci, c in enumerate(configs):
            s = st[ci]
            for e in entries:
                a, b = e["a"], e["a"] + e["n"]
                lr = float(meta["lr"][e.get("lr_group", 0)]
                           if isinstance(meta["lr"], (list, tuple))
                           else meta["lr"])
                bc1c, bc2c = bc_pair(c.optimizer, count, e["b1"], e["b2"])
                if bnd[ci]:
                    q = (gd[a:b] + s["res"][a:b]) * coefs[ci]
                    s["res"][a:b] = 0.0
                else:
                    sl = s["sel"][a:b]
                    q = gd[a:b] * sl * coefs[ci]
                    s["res"][a:b] += gd[a:b] * (~sl)
                if bnd[ci] and c.dual_lr != 1.0:
                    so = out_sel.get(ci, s["sel"])
                    inactive, lr_i = ~so[a:b], lr * c.dual_lr
                else:
                    inactive = lr_i = None
                opt_step_inplace(q, s["m"][a:b], s["v"][a:b], s["w"][a:b],
                                 None, lr, e["wd"], e["b1"], e["b2"], bc1c,
                                 bc2c, e["eps"], optimizer=c.optimizer,
                                 inactive=inactive, lr_inactive=lr_i)
            if hz is not None:
                d = (s["w"] - snapshots[hz]).double()
                dist_at[ci][hz] = math.sqrt(float((d * d).sum()))
    for ci in range(len(configs)):
        st[ci]["dist"] = dist_at[ci]
    return st
