"""Fused per-rank sparse step over a flat bucket (engine order of
``sga/engine.py:416-604``): score -> exact top-k -> index pack -> residual
update -> residual-aware AdamW, as two kinds of sweeps over HBM."""
import ctypes as C

import torch

from . import _lib as L
from .scores import STEP_SCORE_MAP as SCORE_MAP
from .selection import read_result


class SingleSweepLost(RuntimeError):
    """The single-sweep step committed on a sampled bracket that turned out not
    to hold the k-th key (``result.status == 3``): resid / p / m / v of this
    step are not the exact top-k step's and the pack was not written.  The
    two-sweep step (``single_sweep=False``) has no such outcome."""


def k_for(n_total, ratio_percent):
    """``sga/plugins/selection/topk.py:111-112``"""
    return max(1, int(round(n_total * ratio_percent / 100.0)))


class FusedSparseStep:
    """Owns the workspace, the device segment table and the pack buffers for
    one flat bucket of ``n`` elements.

    segments: list of dicts {"start", "n", "lr", "b1", "b2", "eps", "wd"}
    tiling [0, n) in ascending order (one per parameter tensor).
    """

    def __init__(self, n, segments, device, values_dtype=torch.bfloat16,
                 max_k=None, want_mask=False):
        assert 0 < n < 2 ** 31
        off = 0
        for s in segments:
            if s["start"] != off or s["n"] <= 0:
                raise ValueError("segments must tile [0, n) contiguously in order")
            off += s["n"]
        if off != n:
            raise ValueError(f"segments cover {off} elements, bucket has {n}")
        self.n, self.segments, self.device = n, segments, device
        self.values_dtype = values_dtype
        self.ws_bytes = int(L.raw("sga_fused_workspace_bytes", n))
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=device)
        self.result = torch.zeros(8, dtype=torch.int32, device=device)
        self.max_k = max_k or n
        self.idx = torch.empty(self.max_k, dtype=torch.int32, device=device)
        self.values = torch.empty(self.max_k, dtype=values_dtype, device=device)
        self.mask = (torch.empty(n, dtype=torch.uint8, device=device)
                     if want_mask else None)
        self._seg_host = (L.Segment * len(segments))()
        for e, s in zip(self._seg_host, segments):
            e.start, e.n = s["start"], s["n"]
            e.lr = L.f32(s["lr"])
            e.beta1, e.om1 = L.f32(s["b1"]), L.f32(1.0 - s["b1"])
            e.beta2, e.om2 = L.f32(s["b2"]), L.f32(1.0 - s["b2"])
            e.eps, e.wd = L.f32(s["eps"]), L.f32(s["wd"])
        self._seg_up = L.TableUploader(C.sizeof(self._seg_host), device)
        self._seg_dev = self._seg_up.dev
        self._seg_step = None
        self._ws2 = None          # second workspace of the single-sweep step, on first use
        self._calls = 0

    def _single_sweep_ws(self):
        if self._ws2 is None:
            nbytes = int(L.raw("sga_fused_single_sweep_workspace_bytes", self.n,
                               L.dtype_code(self.values)))
            self._ws2 = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        return self._ws2

    def _upload_segments(self, step):
        if self._seg_step == step:
            return
        bc = {}
        for e, s in zip(self._seg_host, self.segments):
            key = (s["b1"], s["b2"])
            if key not in bc:
                bc[key] = (L.f32(1.0 - s["b1"] ** step), L.f32(1.0 - s["b2"] ** step))
            e.lr = L.f32(s["lr"])                      # callers may retune lr between steps
            e.bc1, e.bc2 = bc[key]
        self._seg_up.upload(self._seg_host)
        self._seg_step = step

    @staticmethod
    def _flags(optimizer, fold, interval, inactive_lr_scale):
        if optimizer not in ("adamw", "adams"):
            raise ValueError(f"unknown optimizer {optimizer!r} (adamw, adams)")
        if inactive_lr_scale != 1.0:
            raise ValueError("grad-correct boundary dual-lr (inactive_lr_scale="
                             f"{inactive_lr_scale!r}) requires a full step (emit_score set) "
                             "with a mask; the fused step is a sparse step")
        if fold and not interval > 0.0:
            raise ValueError(f"fold needs interval > 0 (got {interval!r})")
        return (L.GC_ADAMS if optimizer == "adams" else 0) | (L.GC_FOLD if fold else 0)

    def _run(self, name, g, state_args, step, k, ratio_percent, score, factor, coeff, fast,
             optimizer, fold, interval, inactive_lr_scale, single_sweep, seed, check, result):
        """Checks shared by the two state layouts, then one call of entry point
        ``name`` (``state_args``: what that entry point takes between the
        gradient and ``n``)."""
        flags = self._flags(optimizer, fold, interval, inactive_lr_scale)
        n = self.n
        if k is None:
            k = k_for(n, ratio_percent)
        if not (1 <= k <= min(n, self.max_k)):
            raise ValueError(f"k={k} out of range (n={n}, max_k={self.max_k})")
        if score not in SCORE_MAP:
            raise ValueError(f"Unknown SGA score '{score}'. Registered: {sorted(SCORE_MAP)}")
        self._upload_segments(step)
        if g is None and score == "abs_g_blind":
            raise ValueError("score 'abs_g_blind' ranks the step's own gradient: pass g")
        head = [L.ptr(g), L.SGA_F32 if g is None else L.dtype_code(g), *state_args, n, k,
                L.ptr(self._seg_dev),
                len(self.segments), SCORE_MAP[score], L.ptr(self.idx), L.ptr(self.values),
                L.dtype_code(self.values), L.ptr(self.mask), L.f32(factor), L.f32(coeff)]
        if result is None:
            result = self.result
        elif (result.dtype != torch.int32 or result.numel() != 8 or not result.is_cuda
              or not result.is_contiguous()):
            raise ValueError("result: a contiguous int32[8] device tensor")
        if single_sweep:
            ws2 = self._single_sweep_ws()
            self._calls += 1
            L.call(name, *head, flags, L.f32(interval),
                   (self._calls if seed is None else seed) & 0xFFFFFFFF, L.ptr(result),
                   L.ptr(self.ws), self.ws_bytes, L.ptr(ws2), ws2.numel(), L.stream())
            if check:
                res = read_result(result)              # synchronises with the step
                if res.status == 3:
                    raise SingleSweepLost(
                        f"single-sweep step {step}: the sampled bracket missed the k-th key "
                        f"after the commit (k={k}, n={n}, seed={self._calls if seed is None else seed}); "
                        "the state of this step is not the exact top-k step's -- restore it "
                        "from the caller's copy, or use the two-sweep step")
        else:
            L.call(name, *head, 1 if fast else 0, flags, L.f32(interval), L.ptr(result),
                   L.ptr(self.ws), self.ws_bytes, L.stream())
        return self.idx[:k], self.values[:k]

    def step(self, g, resid, p, m, v, step, k=None, ratio_percent=None,
             score="abs_g", factor=1.0, coeff=1.0, fast=True, optimizer="adamw", fold=False,
             interval=1.0, inactive_lr_scale=1.0, single_sweep=False, seed=None, check=True,
             result=None, out=None):
        """Run one fused step in place; returns (idx[:k], values[:k]) views.
        ``self.result`` holds the device-side select result (threshold bits,
        counts); nothing is synchronised here.  ``g=None``: ``resid`` already
        holds g + r (the reference's own contract, where backward accumulates
        into the buffer that keeps the residual); the step then reads 4 B per
        coordinate less.  ``optimizer="adams"`` commits
        (and scores) with the AdamS tail; ``fold`` divides the new residual by
        ``interval`` (the residual mean taken before a boundary).

        ``single_sweep``: read g / resid / p / m / v once instead of twice --
        coordinates outside the sampled bracket are committed in the sweep
        itself, the few inside it afterwards from their records.  Same outputs
        bit for bit; ``result.status == 3`` reports the one thing that cannot
        be repaired, a sampled bracket that missed the k-th key after the
        commit (12 sigma margins; ``seed`` moves the sample offsets, default a
        per-call counter).  The reference has no such outcome, so this mode is
        for callers that hold a restorable copy of the state (or accept
        restarting from a checkpoint): with ``check`` (the default) the call
        waits for the step and raises ``SingleSweepLost`` on status 3 instead
        of handing back a pack that was not written; ``check=False`` leaves
        the status to the caller (``result``: an int32[8] device tensor of the
        caller's for this step's result block, default ``self.result``).

        ``out`` (single sweep only): ``(resid, p, m, v)`` fp32 tensors that
        receive the new state while the inputs are only read (ping-pong
        state).  A missed bracket then loses nothing: the device redoes the
        step from the untouched inputs, the status stays 0 and
        ``read_result().redone`` is set."""
        for t in (g, resid, p, m, v):
            if t is None and t is g:
                continue
            L.require_dev(t)
            L.require_contig(t=t)
            assert t.numel() == self.n
        state = [L.ptr(resid), L.ptr(p), L.ptr(m), L.ptr(v)]
        name = "sga_fused_sparse_step" + ("_single_sweep" if single_sweep else "")
        if out is not None:
            if not single_sweep:
                raise ValueError("out=: the out-of-place step is the single-sweep step")
            if len(out) != 4:
                raise ValueError("out=: (resid, p, m, v) tensors for the new state")
            for t in out:
                L.require_dev(t)
                L.require_contig(t=t)
                if t.numel() != self.n or t.dtype != torch.float32:
                    raise ValueError("out=: flat fp32 tensors of the bucket's length")
            state += [L.ptr(t) for t in out]
            name += "_out"
        return self._run(name, g, state, step, k, ratio_percent, score, factor, coeff, fast,
                         optimizer, fold, interval, inactive_lr_scale, single_sweep, seed, check,
                         result)

    def step_packed(self, g, state, step, k=None, ratio_percent=None, score="abs_g",
                    factor=1.0, coeff=1.0, fast=True, optimizer="adamw", fold=False,
                    interval=1.0, inactive_lr_scale=1.0, single_sweep=False, seed=None,
                    check=True, result=None, out=None):
        """Same step on a ``PackedState`` (resid/p/m/v interleaved in 64 KiB
        records): same arithmetic and outputs.  ``out`` (single sweep only):
        another ``PackedState`` that receives the new state, as in ``step``."""
        L.require_dev(g, state.data)
        L.require_contig(g=g)
        if (g is not None and g.numel() != self.n) or state.n != self.n:
            raise ValueError("gradient / packed state length does not match the bucket")
        name = ("sga_fused_sparse_step_single_sweep_packed" if single_sweep else
                "sga_fused_sparse_step_packed")
        args = [L.ptr(state.data)]
        if out is not None:
            if not single_sweep:
                raise ValueError("out=: the out-of-place step is the single-sweep step")
            if out.n != self.n:
                raise ValueError("out=: a PackedState of the bucket's length")
            L.require_dev(out.data)
            args.append(L.ptr(out.data))
            name += "_out"
        return self._run(name, g, args, step, k, ratio_percent, score, factor,
                         coeff, fast, optimizer, fold, interval, inactive_lr_scale, single_sweep,
                         seed, check, result)

    def read_result(self):
        return read_result(self.result)


def fused_step_multi(steppers, grads, resids, ps, ms, vs, step, ks=None, ratio_percent=None,
                     score="abs_g", factor=1.0, coeff=1.0, fast=True, optimizer="adamw",
                     fold=False, interval=1.0):
    """One two-sweep fused step for several buckets in ONE call
    (``sga_fused_sparse_step_multi``): the per-bucket online path, where every
    bucket selects its own top-k (``sga/engine.py:822-890``).  ``steppers``:
    one ``FusedSparseStep`` per bucket (its segment table, workspace, pack
    buffers, mask and result block are that bucket's); ``grads`` ... ``vs``:
    the buckets' tensors, same order.  Outputs land where the single-bucket
    ``step`` puts them; returns [(idx[:k], values[:k])] per bucket.  The
    buckets share dtypes, score and knobs; the short dependent kernels around
    their selects run once for up to eight buckets."""
    nb = len(steppers)
    if not (nb == len(grads) == len(resids) == len(ps) == len(ms) == len(vs)) or nb == 0:
        raise ValueError("one gradient / residual / p / m / v per bucket")
    flags = FusedSparseStep._flags(optimizer, fold, interval, 1.0)
    if score not in SCORE_MAP:
        raise ValueError(f"Unknown SGA score '{score}'. Registered: {sorted(SCORE_MAP)}")
    if ks is None:
        ks = [k_for(fs.n, ratio_percent) for fs in steppers]
    table = (L.FusedBucket * nb)()
    some_g = next((g for g in grads if g is not None), None)
    gd = L.SGA_F32 if some_g is None else L.dtype_code(some_g)
    vd = L.dtype_code(steppers[0].values)
    for b, fs in enumerate(steppers):
        g, r, p, m, v = grads[b], resids[b], ps[b], ms[b], vs[b]
        for t in (r, p, m, v) if g is None else (g, r, p, m, v):
            L.require_dev(t)
            L.require_contig(t=t)
            if t.numel() != fs.n:
                raise ValueError(f"bucket {b}: tensor length does not match the bucket")
        if g is None and (gd != L.SGA_F32 or score == "abs_g_blind"):
            raise ValueError(f"bucket {b}: no gradient (resid holds g + r) goes with fp32 "
                             "gradients in the other buckets, and not with score 'abs_g_blind'")
        if (g is not None and L.dtype_code(g) != gd) or L.dtype_code(fs.values) != vd:
            raise ValueError("the buckets of one call share the gradient and value dtypes")
        if not (1 <= ks[b] <= min(fs.n, fs.max_k)):
            raise ValueError(f"bucket {b}: k={ks[b]} out of range (n={fs.n}, max_k={fs.max_k})")
        fs._upload_segments(step)
        e = table[b]
        e.g = None if g is None else g.data_ptr()
        e.resid, e.p, e.m, e.v = (t.data_ptr() for t in (r, p, m, v))
        e.n, e.k = fs.n, ks[b]
        e.segs, e.n_segs = fs._seg_dev.data_ptr(), len(fs.segments)
        e.idx_out, e.values_out = fs.idx.data_ptr(), fs.values.data_ptr()
        e.mask_out = fs.mask.data_ptr() if fs.mask is not None else None
        e.result = fs.result.data_ptr()
        e.ws, e.ws_bytes = fs.ws.data_ptr(), fs.ws_bytes
    L.call("sga_fused_sparse_step_multi", table, nb, gd, SCORE_MAP[score], vd, L.f32(factor),
           L.f32(coeff), 1 if fast else 0, flags, L.f32(interval), L.stream())
    return [(fs.idx[:k], fs.values[:k]) for fs, k in zip(steppers, ks)]


class PackedState:
    """resid, p, m, v of one bucket interleaved in 64 KiB records
    ``[resid[4096] | p[4096] | m[4096] | v[4096]]`` (the layout of
    ``sga_fused_sparse_step_packed``).  ``pack`` / ``unpack`` convert from and
    to flat fp32 tensors; ``None`` leaves that array untouched."""

    def __init__(self, n, device):
        self.n = int(n)
        self.data = torch.zeros(int(L.raw("sga_packed_state_elems", self.n)), dtype=torch.float32,
                                device=device)

    def _repack(self, resid, p, m, v, unpack):
        for t in (resid, p, m, v):
            if t is not None:
                L.require_dev(t)
                L.require_contig(t=t)
                if t.numel() != self.n or t.dtype != torch.float32:
                    raise ValueError("PackedState: flat fp32 tensors of the bucket's length")
        L.call("sga_state_repack", *(L.ptr(t) if t is not None else None for t in (resid, p, m, v)),
               L.ptr(self.data), self.n, int(unpack), L.stream())

    def pack(self, resid=None, p=None, m=None, v=None):
        self._repack(resid, p, m, v, False)
        return self

    def unpack(self, resid=None, p=None, m=None, v=None):
        self._repack(resid, p, m, v, True)
