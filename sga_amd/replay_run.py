"""Offline replay of one recorded window, end to end on one device: trace
directory -> branch state -> dense reference pass -> branch selection ->
fused group streaming pass (``sga/replay_fused.py:1120-1914`` at world 1,
without the report/ranking diagnostics).
"""
import torch

from . import _lib as L
from .replay import _bc_pair, require_scan_dtypes, select_topk_flat
from .replay_dense import dense_replay_dev
from .replay_fused import shard_select_balanced
from .replay_group import SELECTION_SEMANTICS, Config, ReplayGroup
from .scores import SCORE_MAP
from .trace_io import (ResidentWindow, ShardParams, TraceFile, WindowReader, discover_trace,
                       load_branch_state, lr_for_step, window_steps_for)


# The reference's run-level switches of the fused replay (replay_fused.py:1137-1198): same names,
# same allowed values, and the same contract that an unknown value raises instead of silently
# leaving the switch a no-op.  Every "kill" arm routes the reference to a CPU / eager / mmap path
# that does not exist here (no second code path by design), so asking for one is refused loudly.
_REPLAY_SWITCHES = {
    "REPLAY_FUSED_FRONT_SORT": (("auto", "cpu"), "auto"),
    "REPLAY_FUSED_SELECT": (("auto", "cpu"), "auto"),
    "REPLAY_FUSED_FRONT_RANK_BG": (("auto", "off"), "auto"),
    "REPLAY_FUSED_KERNEL": (("auto", "off"), "auto"),
    "REPLAY_FUSED_P1_READ": (("pread", "mmap"), "pread"),
}


def replay_switches(environ=None):
    """Reads and validates the replay switches; returns {name: value}."""
    import os
    env = os.environ if environ is None else environ
    out = {}
    for name, (allowed, default) in _REPLAY_SWITCHES.items():
        val = env.get(name, default)
        if val not in allowed:
            raise ValueError(f"{name}={val!r} is not one of the allowed values "
                             f"({', '.join(repr(a) for a in allowed)})")
        # the front ranking diagnostics are not built, so its background switch has nothing to do
        if val != default and name != "REPLAY_FUSED_FRONT_RANK_BG":
            raise RuntimeError(f"{name}={val} asks for the reference's {val} path; this build runs "
                               "the HIP kernels only (no CPU / eager / mmap fallback)")
        out[name] = val
    return out


def branch_scores(score, optimizer, sp, w0, m0, v0, g0, count, include_wd=True):
    """|registry score| at the branch point, evaluated in double and rounded
    once to fp32, flat over the shard (``replay_fused.py:1236-1265``)."""
    L.require_dev(w0, m0, v0, g0)
    out = torch.empty(sp.n, dtype=torch.float32, device=w0.device)
    st = L.stream()
    for e in sp.entries:
        a, n = e["a"], e["n"]
        bc1, bc2 = _bc_pair(optimizer, count, e["b1"], e["b2"])
        L.call("sga_branch_score_f64", SCORE_MAP[score], L.ptr(w0[a:a + n]), L.ptr(m0[a:a + n]),
               L.ptr(v0[a:a + n]), L.ptr(g0[a:a + n]), L.ptr(out[a:a + n]), n,
               float(e["b1"]), float(e["b2"]), float(e["eps"]), float(e["wd"]), float(bc1),
               float(bc2), int(optimizer == "adams"), int(include_wd), st)
    return out


def _branch_grad(state_path, sp, device):
    """The branch step's own gradient from the state file (zeros when a param
    has none), flat fp32 on the device (``replay_fused.py:1230-1233``)."""
    tf = TraceFile(state_path)
    host = torch.zeros(sp.n, dtype=torch.float32)
    for e in sp.entries:
        card = tf.payload.get("g", {}).get(e["name"])
        if card is not None:
            host[e["a"]:e["a"] + e["n"]] = tf.read_tensor(card, e["p_off"], e["n"]).float()
    return host.to(device)


def replay_window(trace_dir, t0, window, configs, horizons, device,
                  selection_semantics="topk", depth=2, replay_dtype="fp32", norm_dtype="fp32"):
    """Replays ``configs`` (``replay_group.Config``) over the recorded window
    that starts at branch point ``t0``.  ``selection_semantics`` applies to
    BOTH select sites, the branch-point select and every boundary
    re-selection of the streaming pass (``replay_fused.py:1340-1344``).

    Returns a dict with the dense reference (``den_at``, ``label_total``,
    ``recon_steps``), and per config the distances ``||w_s(H) - w_d(H)||`` and
    distortions ``dist / den`` at every effective horizon, plus the resident
    ``ReplayGroup`` for inspection.
    """
    replay_switches()
    require_scan_dtypes(replay_dtype, norm_dtype)
    if selection_semantics not in SELECTION_SEMANTICS:
        raise ValueError(f"unknown selection semantics {selection_semantics!r} "
                         f"(expected one of {SELECTION_SEMANTICS})")
    catalog, names, _offs, N, state_files, g_files = discover_trace(trace_dir)
    if t0 not in state_files:
        raise ValueError(f"branch point {t0} has no step_{t0:06d}_state.pt in {trace_dir}")
    steps = window_steps_for(g_files, t0, window)
    if not steps:
        raise ValueError(f"no recorded gradient for step {t0} in {trace_dir}")
    W = len(steps)
    eff_h = sorted(h for h in horizons if 1 <= h <= W)
    base_meta = TraceFile(state_files[t0]).meta
    sp = ShardParams(names, catalog, base_meta, 0, N)
    w0, m0, v0, _ = load_branch_state(state_files[t0], sp, device)
    g0 = _branch_grad(state_files[t0], sp, device)
    cache = {}
    out = {"N": N, "window_steps": steps, "horizons": eff_h, "dense": {}, "configs": []}
    snaps = {}
    # the trace is read once; every later pass iterates the device-resident copy
    window = ResidentWindow(
        lambda: WindowReader(g_files, steps, sp, device, depth=depth, index_cache=cache), W, N)
    for opt in sorted({c.optimizer for c in configs}):
        total, den_at, recon, snap, dense = dense_replay_dev(
            sp.entries, w0, m0, v0, window, t0, eff_h, optimizer=opt)
        out["dense"][opt] = {"label_total": total, "den_at": den_at, "recon_steps": recon,
                             "label": dense.label}
        snaps[opt] = snap
    count0 = int(base_meta["step"]) + 1
    sel_cache, sel0 = {}, []
    for c in configs:
        key = (c.score, c.ratio, c.optimizer)
        if key not in sel_cache:
            sc = branch_scores(c.score, c.optimizer, sp, w0, m0, v0, g0, count0)
            k = max(1, int(round(c.ratio / 100.0 * N)))
            if selection_semantics == "balanced-histogram":
                sel_cache[key] = shard_select_balanced(sc, k, None, sp.entries)[0]
            else:
                sel_cache[key] = select_topk_flat(sc, k)[0]
        sel0.append(sel_cache[key])
    by_opt = {}
    for ci, c in enumerate(configs):
        by_opt.setdefault(c.optimizer, []).append(ci)
    results = [None] * len(configs)
    for opt, idxs in by_opt.items():
        group = ReplayGroup(sp.entries, w0, m0, v0, [sel0[i] for i in idxs],
                            [configs[i] for i in idxs], t0, W,
                            selection_semantics=selection_semantics)
        for _gstep, gmeta, g in window:
            meta = {"clip_grad": gmeta.get("clip_grad", 0.0),
                    "grad_norm": gmeta.get("grad_norm", float("nan")),
                    "lr": (lambda e, gm=gmeta: lr_for_step(gm, e.get("group")))}
            group.step(g, meta, snapshots=snaps[opt], horizons=eff_h)
        den = out["dense"][opt]["den_at"]
        for j, i in enumerate(idxs):
            dist = group.dist_at[j]
            results[i] = {"config": configs[i], "dist_at": dist, "group": group, "slot": j,
                          "distortion": {h: (dist[h] / den[h] if den[h] > 0.0 else None)
                                         for h in dist}}
    out["configs"] = results
    return out


__all__ = ["Config", "branch_scores", "replay_switches", "replay_window"]
