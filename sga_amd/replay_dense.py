"""Dense reference pass of the offline replay on the device
(``dense_replay_dev``, ``sga/replay.py:848-926``): the full-gradient AdamW /
AdamS trajectory from a branch point, the per-coordinate label
``sum_t (lr_t * upd_t)^2``, per-horizon ``||w_d(H) - w0||`` and snapshots of
``w_d``, and the pre-clip reconstruction diagnostics of every step.

State is flat over the shard (one launch per recorded step, per-tensor
hyper-parameters through a segment table) and the snapshots stay resident on
the device, where the sparse arms compare against them.
"""
import ctypes as C
import math

import torch

from . import _lib as L
from .replay import _bc_pair, coef_dense_for
from .replay_group import ReplaySegment
from .trace_io import lr_for_step


def lr_max_abs_diff(gmeta):
    """Largest |lr_g - mean lr| over the recorded groups (``replay.py:260-265``)."""
    lrs = [float(x) for x in gmeta.get("lr", [])]
    if not lrs:
        return 0.0
    mean = sum(lrs) / len(lrs)
    return max(abs(x - mean) for x in lrs)


class DenseReplay:
    """Resident dense trajectory over a flat shard; ``entries`` as in
    ``ShardParams`` ({"a", "n", "b1", "b2", "eps", "wd", "group"})."""

    def __init__(self, entries, w0, m0, v0, t0, optimizer="adamw"):
        if optimizer not in ("adamw", "adams"):
            raise ValueError(f"unknown optimizer {optimizer!r}")
        L.require_dev(w0, m0, v0)
        self.entries, self.t0, self.optimizer = entries, t0, optimizer
        self.N = w0.numel()
        self.w0 = w0
        self.w, self.m, self.v = w0.clone(), m0.clone(), v0.clone()
        dev = w0.device
        self.label = torch.zeros(self.N, dtype=torch.float32, device=dev)
        self._partials = torch.empty(int(L.raw("sga_replay_partials")), dtype=torch.float64,
                                     device=dev)
        self._recon2 = torch.zeros(1, dtype=torch.float64, device=dev)
        self._dist = torch.zeros(1, dtype=torch.float64, device=dev)
        self._seg_host = (ReplaySegment * len(entries))()
        self._seg_up = L.TableUploader(C.sizeof(self._seg_host), dev)
        self._seg_dev = self._seg_up.dev
        self.si = 0
        self.den_at, self.snapshots, self.recon_steps = {}, {}, []

    def step(self, gstep, g, gmeta, horizons=()):
        """Commit one recorded step; ``g`` is the flat post-clip gradient
        (bf16 or fp32) on the device."""
        L.require_dev(g)
        L.require_contig(g=g)
        if g.numel() != self.N:
            raise ValueError("gradient length does not match the shard")
        coef_dense, flag = coef_dense_for(gmeta)
        count = self.t0 + self.si + 1
        for i, e in enumerate(self.entries):
            r = self._seg_host[i]
            bc1, bc2 = _bc_pair(self.optimizer, count, e["b1"], e["b2"])
            r.start, r.n = e["a"], e["n"]
            r.lr, r.wd = float(lr_for_step(gmeta, e.get("group"))), float(e["wd"])
            r.beta1, r.om1 = L.f32(e["b1"]), L.f32(1.0 - e["b1"])
            r.beta2, r.om2 = L.f32(e["b2"]), L.f32(1.0 - e["b2"])
            r.eps, r.wdf, r.bc1, r.bc2 = L.f32(e["eps"]), L.f32(e["wd"]), L.f32(bc1), L.f32(bc2)
        self._seg_up.upload(self._seg_host)
        st = L.stream()
        L.call("sga_dense_replay_step", L.ptr(g), L.dtype_code(g), L.ptr(self.w), L.ptr(self.m),
               L.ptr(self.v), L.ptr(self.label), self.N, L.ptr(self._seg_dev),
               len(self.entries), int(self.optimizer == "adams"), float(coef_dense),
               L.ptr(self._partials), L.ptr(self._recon2), st)
        recon = math.sqrt(float(self._recon2.item()))
        norm = float(gmeta.get("grad_norm", float("nan")))
        self.recon_steps.append({
            "step": gstep, "lr": lr_for_step(gmeta), "lr_max_abs_diff": lr_max_abs_diff(gmeta),
            "grad_norm": norm, "clip_grad": float(gmeta.get("clip_grad", 0.0)),
            "coef_dense": coef_dense, "reconstruct_flag": flag, "recon_grad_norm": recon,
            "recon_rel_err": ((recon - norm) / norm
                              if math.isfinite(norm) and norm > 0.0 else None)})
        self.si += 1
        if self.si in horizons:
            L.call("sga_sq_dist", L.ptr(self.w), 0, L.ptr(self.w0), self.N, L.ptr(self._partials),
                   L.ptr(self._dist), st)
            self.den_at[self.si] = math.sqrt(float(self._dist.item()))
            self.snapshots[self.si] = self.w.clone()

    def label_total(self):
        return float(self.label.sum(dtype=torch.float64).item())


def dense_replay_dev(entries, w0, m0, v0, reader, t0, eff_horizons, optimizer="adamw"):
    """Run the dense pass over a window; ``reader`` yields
    ``(gstep, meta, g_flat)``.  Returns ``(label_total, den_at, recon_steps,
    snapshots, dense)`` with the label left on the device in ``dense.label``."""
    dense = DenseReplay(entries, w0, m0, v0, t0, optimizer)
    for gstep, gmeta, g in reader:
        dense.step(gstep, g, gmeta, eff_horizons)
    return dense.label_total(), dense.den_at, dense.recon_steps, dense.snapshots, dense
