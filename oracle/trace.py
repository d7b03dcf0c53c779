"""Oracle for the recorded-trace path (test infrastructure; torch CPU).

Loads trace files with ``torch.load(weights_only=True)`` (full tensors on the
heap -- only for the small traces the tests write), restates the dense
reference pass ``dense_replay_dev`` (``sga/replay.py:848-926``) per param
with the in-place commit of ``oracle.replay.opt_step_inplace`` and the
branch-point scores in fp64 (``sga/replay_fused.py:1236-1265``).

Pinned by: byte equality of loaded slices against ``torch.load``; the dense
pass is the repeated single commit already pinned in ``oracle.replay``
(labels are ``sum (lr*upd)^2``, checked against an fp64 recomputation in the
tests); horizon norms and reconstruction norms are closed-form fp64 sums.
"""
import glob
import math
import os
import re

import torch

from . import replay as R
from . import scores as S


def load_file(path):
    return torch.load(path, map_location="cpu", weights_only=True)


def discover(trace_dir):
    cat = load_file(os.path.join(trace_dir, "catalog.pt"))["catalog"]
    names = list(cat)
    numel = {n: int(torch.Size(cat[n]["shape"]).numel()) for n in names}
    g_files, s_files = {}, {}
    for f in sorted(glob.glob(os.path.join(trace_dir, "*.pt"))):
        b = os.path.basename(f)
        m = re.match(r"step_(\d+)_g\.pt$", b)
        if m:
            g_files[int(m.group(1))] = f
        m = re.match(r"step_(\d+)_state\.pt$", b)
        if m:
            s_files[int(m.group(1))] = f
    return cat, names, numel, s_files, g_files


def param_hp(meta, cat_entry):
    groups, gi = meta.get("param_groups"), cat_entry.get("param_group")
    if groups is not None and gi is not None:
        g = groups[int(gi)]
        return (float(g["adam_beta1"]), float(g["adam_beta2"]), float(g["adam_eps"]),
                float(g["weight_decay"]), int(gi))
    return (float(meta["adam_beta1"]), float(meta["adam_beta2"]), float(meta["adam_eps"]),
            float(meta["weight_decay"]), None)


def lr_for(meta, group):
    lrs = [float(x) for x in meta.get("lr", [0.0])]
    if group is not None and group < len(lrs):
        return lrs[group]
    return sum(lrs) / len(lrs)


def entries_for(cat, names, numel, meta, lo=None, hi=None):
    total = sum(numel.values())
    lo, hi = (0 if lo is None else lo), (total if hi is None else hi)
    out, off = [], 0
    for n in names:
        a, b = max(off, lo), min(off + numel[n], hi)
        if b > a:
            b1, b2, eps, wd, gi = param_hp(meta, cat[n])
            out.append({"name": n, "p_off": a - off, "a": a - lo, "n": b - a, "b1": b1,
                        "b2": b2, "eps": eps, "wd": wd, "group": gi,
                        "lr_group": gi if gi is not None else 0})
        off += numel[n]
    return out


def flat_slice(payload, entries, n, upcast=True):
    """Flat vector of the shard from a name->tensor payload; absent params
    are zeros.  bf16 is upcast to fp32 (replay_fused.py:1071-1082)."""
    out = torch.zeros(n, dtype=torch.float32)
    for e in entries:
        t = payload.get(e["name"])
        if t is not None:
            out[e["a"]:e["a"] + e["n"]] = \
                t.reshape(-1)[e["p_off"]:e["p_off"] + e["n"]].float()
    return out


def dense_replay(entries, w0, m0, v0, g_steps, metas, t0, horizons, optimizer="adamw"):
    """(label, label_total, den_at, recon_steps, snapshots) of the dense
    trajectory (replay.py:848-926)."""
    w, m, v = w0.clone(), m0.clone(), v0.clone()
    lab = torch.zeros_like(w0)
    den_at, snaps, recon = {}, {}, []
    for si, (g, meta) in enumerate(zip(g_steps, metas)):
        clip = float(meta.get("clip_grad", 0.0))
        norm = float(meta.get("grad_norm", float("nan")))
        coef = R.coef_dense_for(clip, norm)
        count = t0 + si + 1
        r2 = 0.0
        for e in entries:
            a, b = e["a"], e["a"] + e["n"]
            bc1, bc2 = R.bc_pair(optimizer, count, e["b1"], e["b2"])
            q = g[a:b].float()
            R.opt_step_inplace(q, m[a:b], v[a:b], w[a:b], lab[a:b], lr_for(meta, e["group"]),
                               e["wd"], e["b1"], e["b2"], bc1, bc2, e["eps"],
                               optimizer=optimizer)
            r2 += float(((q.double() / coef) ** 2.0).sum())
        recon.append({"coef_dense": coef, "recon_grad_norm": math.sqrt(r2)})
        if si + 1 in horizons:
            d = (w - w0).double()
            den_at[si + 1] = math.sqrt(float((d * d).sum()))
            snaps[si + 1] = w.clone()
    return lab, float(lab.double().sum()), den_at, recon, snaps


def branch_scores(score, optimizer, entries, w0, m0, v0, g0, count, include_wd=True):
    """fp64 registry score -> |.| -> fp32 (replay_fused.py:1248-1265)."""
    out = torch.empty(w0.numel(), dtype=torch.float32)
    for e in entries:
        a, b = e["a"], e["a"] + e["n"]
        bc1, bc2 = R.bc_pair(optimizer, count, e["b1"], e["b2"])
        sc = S.score_formula(score, w0[a:b].double(), m0[a:b].double(), v0[a:b].double(),
                             g0[a:b].double(), e["b1"], e["b2"], e["eps"], e["wd"], bc1, bc2,
                             optimizer, update_includes_wd=include_wd)
        out[a:b] = sc.abs()
    return out
