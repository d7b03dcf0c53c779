"""Fused offline-replay group step on MI355X: the per-recorded-step loop of
``sga/replay_fused.py:1607-1914`` at world == 1.  G configurations
(score x ratio x cycle length x optimizer x fold x dual-lr) share one read of
the recorded gradient per pass.  State stays resident on the device: per
config one packed buffer (res / w / m / v interleaved in 64 KiB records) and
the selection mask as bit planes; the residual's traffic is skipped while it
is known to be all zeros."""
import ctypes as C
import math

import torch

from . import _lib as L
from .scores import STEP_SCORE_MAP as SCORE_MAP
from .selection import read_result

MAX_CONFIGS = 16
# what a boundary re-selects with (replay_fused.py:1340-1344): the exact top-k with the tie
# layer filled in index order, or the online engine's balanced-histogram tier
SELECTION_SEMANTICS = ("topk", "balanced-histogram")
_BAL_STRIDE = 8


class ReplayCfg(C.Structure):
    """struct sga_replay_cfg"""
    _fields_ = [("w", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p), ("res", C.c_void_p),
                ("sel", C.c_void_p), ("out_sel", C.c_void_p), ("lr_scale", C.c_double),
                ("boundary", C.c_int), ("adams", C.c_int), ("split", C.c_int), ("packed", C.c_int),
                ("res_zero", C.c_int), ("pad_", C.c_int)]


class ReplaySegment(C.Structure):
    """struct sga_replay_segment"""
    _fields_ = [("start", C.c_int64), ("n", C.c_int64), ("lr", C.c_double), ("wd", C.c_double),
                ("beta1", C.c_float), ("om1", C.c_float), ("beta2", C.c_float),
                ("om2", C.c_float), ("eps", C.c_float), ("bc1", C.c_float), ("bc2", C.c_float),
                ("wdf", C.c_float)]


class Config:
    """One replay arm (``replay_fused.py:1501-1505``)."""

    def __init__(self, score, ratio, T, optimizer="adamw", fold=False, dual_lr=1.0):
        if score not in SCORE_MAP:
            raise ValueError(f"Unknown SGA score '{score}'. Registered: {sorted(SCORE_MAP)}")
        if optimizer not in ("adamw", "adams"):
            raise ValueError(f"unknown optimizer {optimizer!r}")
        self.score, self.ratio, self.T = score, float(ratio), int(T)
        self.optimizer, self.fold, self.dual_lr = optimizer, bool(fold), float(dual_lr)


def coef_dense_for(clip_grad, grad_norm):
    """``sga/replay.py:628-645``"""
    if clip_grad <= 0.0 or not math.isfinite(grad_norm) or grad_norm <= 0.0:
        return 1.0
    return min(clip_grad / (grad_norm + 1.0e-6), 1.0)


_RUN = 4096                       # floats per array per packed record
_ARRAY_SLOT = {"res": 0, "w": 1, "m": 2, "v": 3}


class ConfigState:
    """One config's resident state: res / w / m / v interleaved in one packed
    buffer (64 KiB records, array order res, w, m, v) plus the byte masks.
    ``state["w"]`` etc. return flat unpacked copies for inspection,
    ``state["sel"]`` the mask expanded to bytes."""

    def __init__(self, n, w0, m0, v0, sel):
        dev = w0.device
        self.n = n
        self.data = torch.zeros(int(L.raw("sga_packed_state_elems", n)), dtype=torch.float32,
                                device=dev)
        L.call("sga_state_repack", None, L.ptr(w0), L.ptr(m0), L.ptr(v0), L.ptr(self.data), n, 0,
               L.stream())
        # masks live as bit planes (four wave ballots per 256 elements): the
        # re-selection writes them directly and the sweeps read 1 bit per element
        words = int(L.raw("sga_plane_words", n))
        self.sel = torch.zeros(words, dtype=torch.int32, device=dev)
        self.spare = torch.zeros(words, dtype=torch.int32, device=dev)
        m8 = sel.reshape(-1).to(torch.uint8).contiguous()
        L.call("sga_mask_to_planes", L.ptr(m8), n, L.ptr(self.sel), L.stream())

    def base(self, name):
        """Device address of an array's first run inside the packed buffer."""
        return self.data.data_ptr() + 4 * _RUN * _ARRAY_SLOT[name]

    def __getitem__(self, name):
        if name == "sel":
            out = torch.empty(self.n, dtype=torch.uint8, device=self.data.device)
            L.call("sga_planes_to_mask", L.ptr(self.sel), self.n, L.ptr(out), L.stream())
            return out
        out = torch.empty(self.n, dtype=torch.float32, device=self.data.device)
        args = [None] * 4
        args[_ARRAY_SLOT[name]] = L.ptr(out)
        L.call("sga_state_repack", *args, L.ptr(self.data), self.n, 1, L.stream())
        return out


class ReplayGroup:
    """Resident state of one config group over a flat shard of N elements.

    entries : list of dicts {"a", "n", "b1", "b2", "eps", "wd"} tiling [0, N)
              (ShardParams entries, ``replay_fused.py:251-271``)
    w0/m0/v0: flat fp32 device tensors, the branch-point state (copied per config)
    sel0    : per-config flat bool/uint8 device masks (branch selection)

    ``state[ci]["w" | "m" | "v" | "res" | "sel"]`` returns flat copies for
    inspection; ``dist_at[ci][H]`` holds ``||w - snapshot_H||`` after ``step``
    was given the snapshots.
    """

    def __init__(self, entries, w0, m0, v0, sel0, configs, t0, window,
                 selection_semantics="topk"):
        if not (1 <= len(configs) <= MAX_CONFIGS):
            raise ValueError(f"1..{MAX_CONFIGS} configs per group")
        if selection_semantics not in SELECTION_SEMANTICS:
            raise ValueError(f"unknown selection semantics {selection_semantics!r} "
                             f"(expected one of {SELECTION_SEMANTICS})")
        self.semantics = selection_semantics
        L.require_dev(w0, m0, v0, *sel0)
        self.N = w0.numel()
        off = 0
        for e in entries:
            if e["a"] != off:
                raise ValueError("entries must tile [0, N) in order")
            off += e["n"]
        if off != self.N:
            raise ValueError("entries do not cover the shard")
        self.entries, self.configs, self.t0, self.W = entries, configs, t0, window
        dev = w0.device
        self.dev = dev
        self.state = [ConfigState(self.N, w0, m0, v0, sel0[ci]) for ci in range(len(configs))]
        G = len(configs)
        self.ks = {c.ratio: max(1, int(round(c.ratio / 100.0 * self.N))) for c in configs}
        self.partials = torch.empty(int(L.raw("sga_replay_partials")), dtype=torch.float64,
                                    device=dev)
        self.qn2 = torch.zeros(G, dtype=torch.float64, device=dev)
        self.coef_d = torch.ones(G, dtype=torch.float64, device=dev)
        self.coef_f = torch.ones(G, dtype=torch.float32, device=dev)
        # one select workspace and result block per configuration that can re-select in the
        # same step (allocated on first use)
        self.ws_bytes = int(L.raw("sga_select_workspace_bytes", self.N))
        self._ws = []
        self.sel_results = torch.zeros(G, 8, dtype=torch.int32, device=dev)
        self._last_result = self.sel_results[0]
        if selection_semantics == "balanced-histogram":
            # every tensor is subsampled on its own param-relative stride-8 grid
            phases = [(-int(e.get("p_off", 0))) % _BAL_STRIDE for e in entries]
            self._n_sampled = sum(len(range(ph, e["n"], _BAL_STRIDE))
                                  for ph, e in zip(phases, entries))
            self._seg_phase = torch.tensor(phases, dtype=torch.int32, device=dev)
            self._bal_hist = torch.zeros(int(L.raw("sga_balanced_hist_words")),
                                         dtype=torch.int32, device=dev)
        self._cfg_host = (ReplayCfg * G)()
        self._rseg_host = (ReplaySegment * len(entries))()
        self._rseg_up = L.TableUploader(C.sizeof(self._rseg_host), dev)
        self._rseg_dev = self._rseg_up.dev
        self._seg_host = (L.Segment * len(entries))()
        self._seg_up = L.TableUploader(C.sizeof(self._seg_host), dev)
        self._seg_dev = self._seg_up.dev
        self.dist_at = [dict() for _ in configs]
        # res is all zeros at the start and again after every boundary commit;
        # the kernels then skip its traffic (same values either way)
        self.res_zero = [True] * len(configs)
        self.si = 0

    def _select_ws(self, j):
        while len(self._ws) <= j:
            self._ws.append(torch.empty(self.ws_bytes, dtype=torch.uint8, device=self.dev))
        return self._ws[j]

    # -- per-step tables ----------------------------------------------------
    def _fill_segments(self, count, lr_of):
        for i, e in enumerate(self.entries):
            r = self._rseg_host[i]
            r.start, r.n = e["a"], e["n"]
            r.lr, r.wd = float(lr_of(e)), float(e["wd"])
            r.beta1, r.om1 = L.f32(e["b1"]), L.f32(1.0 - e["b1"])
            r.beta2, r.om2 = L.f32(e["b2"]), L.f32(1.0 - e["b2"])
            r.eps, r.wdf = L.f32(e["eps"]), L.f32(e["wd"])
            r.bc1 = L.f32(1.0 - e["b1"] ** count)
            r.bc2 = L.f32(1.0 - e["b2"] ** count)
            s = self._seg_host[i]
            s.start, s.n, s.lr = e["a"], e["n"], L.f32(lr_of(e))
            s.beta1, s.om1, s.beta2, s.om2 = r.beta1, r.om1, r.beta2, r.om2
            s.eps, s.wd, s.bc1, s.bc2 = r.eps, r.wdf, r.bc1, r.bc2
        self._rseg_up.upload(self._rseg_host)
        self._seg_up.upload(self._seg_host)

    def _fill_cfgs(self, bnd, out_sel):
        for ci, c in enumerate(self.configs):
            s, h = self.state[ci], self._cfg_host[ci]
            h.w, h.m, h.v, h.res = (s.base(k) for k in ("w", "m", "v", "res"))
            h.sel = s.sel.data_ptr()
            split = bool(bnd[ci] and c.dual_lr != 1.0)
            h.out_sel = (out_sel.get(ci, s.sel)).data_ptr() if split else None
            h.lr_scale, h.packed, h.res_zero = c.dual_lr, 1, int(self.res_zero[ci])
            h.boundary, h.adams, h.split = int(bnd[ci]), int(c.optimizer == "adams"), int(split)

    # -- one recorded step ----------------------------------------------------
    def step(self, g, meta, snapshots=None, horizons=()):
        """Advance every config over the recorded (post-clip) gradient ``g``
        (flat bf16/fp32 device tensor).  ``meta``: {"clip_grad", "grad_norm",
        "lr"} (``lr`` a float, or a callable entry -> float)."""
        si, N, G = self.si, self.N, len(self.configs)
        L.require_dev(g)
        L.require_contig(g=g)
        assert g.numel() == N
        clip = float(meta.get("clip_grad", 0.0))
        coef_dense = coef_dense_for(clip, float(meta.get("grad_norm", float("nan"))))
        lr = meta["lr"]
        lr_of = lr if callable(lr) else (lambda e: lr)
        count = self.t0 + si + 1
        bnd = [si % c.T == 0 for c in self.configs]
        st = L.stream()
        if si > 0:                                   # residual fold
            for ci, c in enumerate(self.configs):
                if bnd[ci] and c.fold and not self.res_zero[ci]:
                    L.call("sga_div_inplace", C.c_void_p(self.state[ci].base("res")), N,
                           L.f32(float(c.T)), 1, st)
        self._fill_segments(count, lr_of)
        self._fill_cfgs(bnd, {})
        gd = L.dtype_code(g)
        L.call("sga_replay_pass1", L.ptr(g), gd, N, L.f32(coef_dense), clip, self._cfg_host, G,
               L.ptr(self.partials), L.ptr(self.qn2), L.ptr(self.coef_d), L.ptr(self.coef_f), st)
        out_sel = {}
        # boundary re-selections of this step: under the exact-k semantics they go out as ONE
        # call (configs that rank by the same score share the short kernels of the select)
        resel = [ci for ci, c in enumerate(self.configs)
                 if bnd[ci] and si > 0 and si + 1 < self.W]
        if resel and self.semantics == "topk":
            jobs = (L.ReselectJob * len(resel))()
            for j, ci in enumerate(resel):
                c, s, e = self.configs[ci], self.state[ci], jobs[j]
                e.res, e.w, e.m, e.v = (s.base(x) for x in ("res", "w", "m", "v"))
                e.k, e.score_id = self.ks[c.ratio], SCORE_MAP[c.score]
                e.adams, e.res_zero = int(c.optimizer == "adams"), int(self.res_zero[ci])
                e.coef_f = self.coef_f.data_ptr() + 4 * ci
                e.sel_out = s.spare.data_ptr()
                e.result = self.sel_results[j].data_ptr()
                ws = self._select_ws(j)
                e.ws, e.ws_bytes = ws.data_ptr(), self.ws_bytes
            L.call("sga_replay_reselect_multi", L.ptr(g), gd, N, L.ptr(self._seg_dev),
                   len(self.entries), L.f32(coef_dense), 1, jobs, len(resel), st)
            self._last_result = self.sel_results[len(resel) - 1]
        for ci in resel:
            c, s = self.configs[ci], self.state[ci]
            if self.semantics == "balanced-histogram":
                k = self.ks[c.ratio]
                rank = max(1, round(self._n_sampled * (N - k + 1) / N))   # _histogram.py:122
                L.call("sga_replay_reselect_balanced", L.ptr(g), gd,
                       *[C.c_void_p(s.base(x)) for x in ("res", "w", "m", "v")], N, rank,
                       L.ptr(self._seg_dev), len(self.entries), L.ptr(self._seg_phase),
                       SCORE_MAP[c.score], C.c_void_p(self.coef_f.data_ptr() + 4 * ci),
                       L.f32(coef_dense), int(c.optimizer == "adams"), 1, int(self.res_zero[ci]),
                       L.ptr(s.spare), L.ptr(self.sel_results[0]), L.ptr(self._bal_hist),
                       L.ptr(self._select_ws(0)), self.ws_bytes, st)
                self._last_result = self.sel_results[0]
            if c.dual_lr != 1.0:
                out_sel[ci] = s.sel
            s.sel, s.spare = s.spare, s.sel
        self._fill_cfgs(bnd, out_sel)
        L.call("sga_replay_pass3", L.ptr(g), gd, N, L.f32(coef_dense), self._cfg_host, G,
               L.ptr(self.coef_f), L.ptr(self._rseg_dev), len(self.entries), st)
        self.res_zero = list(bnd)
        hz = si + 1
        if hz in horizons and snapshots is not None:
            out = torch.zeros(1, dtype=torch.float64, device=self.dev)
            part = torch.empty(1024, dtype=torch.float64, device=self.dev)
            for ci in range(G):
                L.call("sga_sq_dist", C.c_void_p(self.state[ci].base("w")), 1, L.ptr(snapshots[hz]), N,
                       L.ptr(part), L.ptr(out), st)
                self.dist_at[ci][hz] = math.sqrt(float(out.item()))
        self.si += 1

    def last_select(self):
        """Result block of the last re-selection launched."""
        return read_result(self._last_result)
