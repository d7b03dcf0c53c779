"""The SGA AdamW optimizer template on MI355X
(``sga/plugins/optimizer/adamw.py``): ``adamw_grad_correct``,
``adamw_grad_correct_compact``, ``build_dir_table`` and ``SgaAdamW`` with the
reference's signatures, refusals and step order."""
import ctypes as C
import math
from dataclasses import dataclass, field
from typing import Optional

import torch

from . import _lib as L
from .config import get_args
from .scores import SCORE_MAP

_BLOCK_SIZE = 1024


def _flat32(**named):
    for name, t in named.items():
        if t is None:
            continue
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be fp32")
    L.require_contig(**named)


def _gc_prepare(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, mask,
                emit_score, coeff, clear, fold, inactive_lr_scale, adams):
    """The refusals of ``adamw.py:554-592`` and the launch flags; returns
    ``(flags, mask_u8)``."""
    if emit_score is not None and emit_score not in SCORE_MAP:
        raise ValueError(
            f"emit_score '{emit_score}' has no _grad_correct_kernel branch "
            f"(implemented: {sorted(SCORE_MAP)})")
    sparse_fusion = (coeff != 1.0) or clear or fold
    if sparse_fusion and (emit_score is not None or mask is None):
        raise ValueError(
            f"grad-correct sparse fusion (coeff={coeff!r}, clear={clear!r}, "
            f"fold={fold!r}) requires a sparse step (emit_score=None) with a "
            "mask — full steps scale in place engine-side and never clear")
    if inactive_lr_scale != 1.0:
        if not (math.isfinite(inactive_lr_scale) and inactive_lr_scale >= 0.0):
            raise ValueError("grad-correct inactive_lr_scale must be a finite float "
                             f">= 0.0 (got {inactive_lr_scale!r})")
        if emit_score is None or mask is None:
            raise ValueError(
                f"grad-correct boundary dual-lr (inactive_lr_scale="
                f"{inactive_lr_scale!r}) requires a full step (emit_score set) "
                "with a mask")
    if mask is not None and emit_score is not None and inactive_lr_scale == 1.0:
        raise ValueError(
            "grad-correct masked-commit full step (mask + emit_score with "
            "inactive_lr_scale=1.0) is refused: pass inactive_lr_scale != 1.0 for "
            "the boundary split, or drop the mask for the mask-blind full step")
    n = param_buffer.numel()
    if n == 0:
        return 0, None
    L.require_dev(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, mask)
    _flat32(param_buffer=param_buffer, grad_buffer=grad_buffer,
            exp_avg_buffer=exp_avg_buffer, exp_avg_sq_buffer=exp_avg_sq_buffer)
    flags = 0
    mk = None
    if mask is not None:
        mk = mask if mask.dtype == torch.uint8 else mask.to(torch.uint8)
        L.require_contig(mask=mk)
        assert mk.numel() == n
        flags |= L.GC_HAS_MASK
    if coeff != 1.0:
        flags |= L.GC_APPLY_COEFF
    if clear:
        flags |= L.GC_CLEAR
    if fold:
        flags |= L.GC_FOLD
    if inactive_lr_scale != 1.0:
        flags |= L.GC_LR_SPLIT
    if adams:
        flags |= L.GC_ADAMS
    return flags, mk


def adamw_grad_correct(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer,
                       lr, beta1, beta2, eps, weight_decay, step, mask=None,
                       emit_score: Optional[str] = None, coeff=1.0, clear=False,
                       fold=False, interval=1.0, inactive_lr_scale=1.0, _adams=False):
    """One fused commit on contiguous same-size 1-D fp32 buffers
    (``adamw.py:502-634``).  ``emit_score=None`` is the sparse step; a score
    name is the full step that also writes that score into ``grad_buffer``."""
    bias_correction1 = 1.0 - beta1 ** step
    bias_correction2 = 1.0 - beta2 ** step
    flags, mk = _gc_prepare(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, mask,
                            emit_score, coeff, clear, fold, inactive_lr_scale, _adams)
    n = param_buffer.numel()
    if n == 0:
        return
    L.call("sga_adamw_grad_correct", L.ptr(param_buffer), L.ptr(grad_buffer),
           L.ptr(exp_avg_buffer), L.ptr(exp_avg_sq_buffer), L.ptr(mk), n, L.f32(lr),
           L.f32(beta1), L.f32(1.0 - beta1), L.f32(beta2), L.f32(1.0 - beta2),
           L.f32(eps), L.f32(weight_decay), L.f32(bias_correction1),
           L.f32(bias_correction2), L.f32(coeff), L.f32(interval),
           L.f32(lr * inactive_lr_scale),
           SCORE_MAP[emit_score] if emit_score is not None else -1, flags, L.stream())


class GcRecord(C.Structure):
    """struct sga_gc_record"""
    _fields_ = [("p", C.c_void_p), ("g", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p),
                ("mask", C.c_void_p), ("n", C.c_int64), ("first_span", C.c_int64)] + \
               [(k, C.c_float) for k in ("lr", "beta1", "om1", "beta2", "om2", "eps", "wd",
                                         "bc1", "bc2", "lr_inactive")] + \
               [("flags", C.c_int), ("pad_", C.c_int)]


_SPAN = 4096
_uploaders = {}


def adamw_grad_correct_multi(records, emit_score=None, coeff=1.0, interval=1.0, _adams=False):
    """The commit of ``adamw_grad_correct`` over many records in one launch.

    ``records``: dicts with the tensors ``p, g, m, v`` (flat fp32), ``mask``
    (or None) and the scalars ``lr, beta1, beta2, eps, weight_decay, step``
    plus the per-record knobs ``coeff_on, clear, fold, inactive_lr_scale``
    (a record without a mask takes none of them).  Same refusals as the
    single-record call, raised before anything is launched.
    """
    table, keep, spans = [], [], 0
    for r in records:
        c = coeff if r.get("coeff_on", True) else 1.0
        flags, mk = _gc_prepare(r["p"], r["g"], r["m"], r["v"], r.get("mask"), emit_score, c,
                                bool(r.get("clear", False)), bool(r.get("fold", False)),
                                float(r.get("inactive_lr_scale", 1.0)), _adams)
        n = r["p"].numel()
        if n == 0:
            continue
        if c == 1.0:
            flags &= ~L.GC_APPLY_COEFF
        step = r["step"]
        e = GcRecord()
        e.p, e.g, e.m, e.v = (t.data_ptr() for t in (r["p"], r["g"], r["m"], r["v"]))
        e.mask = mk.data_ptr() if mk is not None else None
        e.n, e.first_span = n, spans
        # a Python float stored into a c_float field is rounded to nearest fp32
        e.lr, e.beta1, e.om1 = r["lr"], r["beta1"], 1.0 - r["beta1"]
        e.beta2, e.om2 = r["beta2"], 1.0 - r["beta2"]
        e.eps, e.wd = r["eps"], r["weight_decay"]
        e.bc1 = 1.0 if _adams else 1.0 - r["beta1"] ** step
        e.bc2 = 1.0 if _adams else 1.0 - r["beta2"] ** step
        e.lr_inactive = r["lr"] * float(r.get("inactive_lr_scale", 1.0))
        e.flags = flags
        table.append(e)
        keep.append(mk)
        spans += -(-n // _SPAN)
    if not table:
        return
    arr = (GcRecord * len(table))(*table)
    dev = records[0]["p"].device
    key = (dev, C.sizeof(arr))
    up = _uploaders.get(key)
    if up is None:
        up = _uploaders[key] = L.TableUploader(C.sizeof(arr), dev)
    up.upload(arr)
    L.call("sga_adamw_grad_correct_multi", L.ptr(up.dev), len(table), spans, L.f32(coeff),
           L.f32(interval), SCORE_MAP[emit_score] if emit_score is not None else -1, L.stream())


def build_dir_table(idx, total_n):
    """``table[j] == lower_bound(idx, j*1024)``, ``(total_n >> 10) + 2`` int32
    entries (``adamw.py:472-499``)."""
    k = idx.numel()
    n_table = (total_n >> 10) + 2
    assert (n_table - 1) * _BLOCK_SIZE < 2 ** 31, (
        f"build_dir_table: (n_table-1)*BLOCK = {(n_table - 1) * _BLOCK_SIZE} must "
        "stay < 2^31 (int32 table keys)")
    L.require_dev(idx)
    L.require_contig(idx=idx)
    if idx.dtype != torch.int32:
        raise TypeError("build_dir_table: int32 idx")
    table = torch.empty(n_table, dtype=torch.int32, device=idx.device)
    L.call("sga_build_dir_table", L.ptr(idx), k, L.ptr(table), n_table, L.stream())
    return table


def _gcc_prepare(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, idx, values,
                 rec_start, dir_table):
    """The refusals of ``adamw.py:676-750``; returns ``(n, k_total, n_table)``."""
    if not idx.is_contiguous() or not values.is_contiguous():
        raise ValueError("adamw_grad_correct_compact requires contiguous idx/values")
    n = param_buffer.numel()
    if n == 0:
        return 0, 0, 0
    k_total = idx.numel()
    assert k_total + _BLOCK_SIZE < 2 ** 31, (
        f"adamw_grad_correct_compact: k_total + BLOCK_SIZE = {k_total + _BLOCK_SIZE} "
        "must stay < 2^31 (int32 idx offsets)")
    assert rec_start + n + _BLOCK_SIZE < 2 ** 31, (
        f"adamw_grad_correct_compact: rec_start + n_elements + BLOCK_SIZE = "
        f"{rec_start + n + _BLOCK_SIZE} must stay < 2^31 (int32 coordinate offsets)")
    L.require_dev(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, idx, values)
    _flat32(param_buffer=param_buffer, grad_buffer=grad_buffer,
            exp_avg_buffer=exp_avg_buffer, exp_avg_sq_buffer=exp_avg_sq_buffer)
    if idx.dtype != torch.int32:
        raise TypeError("adamw_grad_correct_compact: int32 idx")
    n_table = 0
    if dir_table is not None:
        assert dir_table.dtype == torch.int32 and dir_table.is_contiguous(), (
            f"adamw_grad_correct_compact: dir_table must be contiguous int32, got "
            f"{dir_table.dtype}, contiguous={dir_table.is_contiguous()}")
        assert dir_table.numel() >= ((rec_start + n - 1) >> 10) + 2, (
            f"adamw_grad_correct_compact: dir_table has {dir_table.numel()} entries "
            f"but the record's last block needs >= {((rec_start + n - 1) >> 10) + 2}")
        n_table = dir_table.numel()
    return n, k_total, n_table


def adamw_grad_correct_compact(param_buffer, grad_buffer, exp_avg_buffer,
                               exp_avg_sq_buffer, idx, values, rec_start, lr, beta1,
                               beta2, eps, weight_decay, step, coeff=1.0, fold=False,
                               interval=1.0, dir_table=None, _adams=False):
    """Compact-emission commit: the gradient comes from the bucket-level sorted
    ``(idx, values)`` by merge-join (``adamw.py:637-792``).  ``values`` may be
    fp32 or bf16."""
    bias_correction1 = 1.0 - beta1 ** step
    bias_correction2 = 1.0 - beta2 ** step
    n, k_total, n_table = _gcc_prepare(param_buffer, grad_buffer, exp_avg_buffer,
                                       exp_avg_sq_buffer, idx, values, rec_start, dir_table)
    if n == 0:
        return
    flags = ((L.GC_APPLY_COEFF if coeff != 1.0 else 0) | (L.GC_FOLD if fold else 0)
             | (L.GC_ADAMS if _adams else 0))
    L.call("sga_adamw_grad_correct_compact", L.ptr(param_buffer), L.ptr(grad_buffer),
           L.ptr(exp_avg_buffer), L.ptr(exp_avg_sq_buffer), L.ptr(idx), L.ptr(values),
           L.dtype_code(values), rec_start, n, k_total, L.f32(lr), L.f32(beta1),
           L.f32(1.0 - beta1), L.f32(beta2), L.f32(1.0 - beta2), L.f32(eps),
           L.f32(weight_decay), L.f32(bias_correction1), L.f32(bias_correction2),
           L.f32(coeff), L.f32(interval), flags, L.ptr(dir_table), n_table, L.stream())


class GccRecord(C.Structure):
    """struct sga_gcc_record"""
    _fields_ = [(k, C.c_void_p) for k in ("p", "g", "m", "v", "idx", "values", "table")] + \
               [(k, C.c_int64) for k in ("rec_start", "n", "k_total", "n_table", "first_span")] + \
               [(k, C.c_float) for k in ("lr", "beta1", "om1", "beta2", "om2", "eps", "wd",
                                         "bc1", "bc2")] + [("flags", C.c_int)]


def adamw_grad_correct_compact_multi(records, coeff=1.0, fold=False, interval=1.0, _adams=False):
    """``adamw_grad_correct_compact`` over many records in one launch per values
    dtype.  ``records``: dicts with ``p, g, m, v, idx, values, rec_start,
    dir_table`` and ``lr, beta1, beta2, eps, weight_decay, step``."""
    by_dtype = {}
    for r in records:
        n, k_total, n_table = _gcc_prepare(r["p"], r["g"], r["m"], r["v"], r["idx"], r["values"],
                                           r["rec_start"], r.get("dir_table"))
        if n == 0:
            continue
        lst = by_dtype.setdefault(r["values"].dtype, [])
        e = GccRecord()
        e.p, e.g, e.m, e.v = (t.data_ptr() for t in (r["p"], r["g"], r["m"], r["v"]))
        e.idx, e.values = r["idx"].data_ptr(), r["values"].data_ptr()
        e.table = r["dir_table"].data_ptr() if r.get("dir_table") is not None else None
        e.rec_start, e.n, e.k_total, e.n_table = r["rec_start"], n, k_total, n_table
        e.lr, e.beta1, e.om1 = r["lr"], r["beta1"], 1.0 - r["beta1"]
        e.beta2, e.om2 = r["beta2"], 1.0 - r["beta2"]
        e.eps, e.wd = r["eps"], r["weight_decay"]
        e.bc1 = 1.0 if _adams else 1.0 - r["beta1"] ** r["step"]
        e.bc2 = 1.0 if _adams else 1.0 - r["beta2"] ** r["step"]
        e.flags = ((L.GC_APPLY_COEFF if coeff != 1.0 else 0) | (L.GC_FOLD if fold else 0)
                   | (L.GC_ADAMS if _adams else 0))
        lst.append(e)
    for dtype, lst in by_dtype.items():
        spans = 0
        for e in lst:
            e.first_span = spans
            spans += -(-e.n // _SPAN)
        arr = (GccRecord * len(lst))(*lst)
        dev = records[0]["p"].device
        key = (dev, "gcc", C.sizeof(arr))
        up = _uploaders.get(key)
        if up is None:
            up = _uploaders[key] = L.TableUploader(C.sizeof(arr), dev)
        up.upload(arr)
        L.call("sga_adamw_grad_correct_compact_multi", L.ptr(up.dev), len(lst), spans,
               0 if dtype == torch.float32 else 1, L.f32(coeff), L.f32(interval), L.stream())


@dataclass
class ParamRecord:
    """One (model param, fp32 main param) pair and its hyper-parameters
    (``sga/plugins/optimizer/__init__.py:20-60``)."""
    model_param: object
    main_param: object
    bucket_state: object
    start: int
    end: int
    lr: float
    beta1: float
    beta2: float
    eps: float
    weight_decay: float
    step: int
    _state: dict = field(default=None, repr=False)

    @property
    def grad(self):
        return self.main_param.grad

    @property
    def m(self):
        return self._state["exp_avg"]

    @property
    def v(self):
        return self._state["exp_avg_sq"]

    def mask_u8(self):
        bs = self.bucket_state
        if bs is None or bs.active_mask_u8 is None:
            return None
        return bs.active_mask_u8[self.start:self.end]


@dataclass
class OptContext:
    """What the optimizer sees for one step
    (``sga/plugins/optimizer/__init__.py:63-87``)."""
    records: list
    phase: str
    support: object = None
    bucket_states: list = None
    fold_window: int = 1
    next_step_is_full: bool = False
    apply_coeff: float = 1.0
    compact_values: dict = None


class SgaAdamW:
    """grad-correct + residual reset (``adamw.py:795-986``).  Reads its
    ``sga_*`` flags from the args singleton, like the reference (``:798-799``)."""

    def __init__(self):
        args = get_args()
        self.residual_mean = bool(getattr(args, "sga_optimizer_residual_mean", False))
        self.compact_search = getattr(args, "sga_optimizer_compact_search", "table")
        s = float(getattr(args, "sga_optimizer_full_sync_inactive_lr_scale", 1.0))
        if s == 0.0:
            s = 0.0
        if not (math.isfinite(s) and s >= 0.0):
            raise ValueError("sga_optimizer_full_sync_inactive_lr_scale must be a "
                             f"finite float >= 0.0 (got {s!r})")
        self.full_sync_inactive_lr_scale = s
        self.emit_score = getattr(args, "sga_score", "update")
        if self.emit_score not in SCORE_MAP:
            raise ValueError(
                f"adamw kernel has no EMIT_MODE branch for score '{self.emit_score}' "
                f"(implemented: {sorted(SCORE_MAP)})")

    def ensure_state(self, bucket_states):
        pass

    # the two commit entry points (SgaAdamS swaps in the AdamS recursion)
    _commit = staticmethod(adamw_grad_correct)
    _commit_compact = staticmethod(adamw_grad_correct_compact)

    @staticmethod
    def _state(rec):
        st = rec._state
        if len(st) == 0:
            st["exp_avg"] = torch.zeros_like(rec.main_param.data)
            st["exp_avg_sq"] = torch.zeros_like(rec.main_param.data)
        return st

    _adams = False            # SgaAdamS: the AdamS recursion in the same kernels

    def _records_pass(self, ctx, emit_score, use_mask, coeff=1.0, clear=False,
                      fold=False, interval=1.0, inactive_lr_scale=1.0):
        # every record of the step in ONE launch (the reference issues one kernel
        # per record, adamw.py:869-905); per-record knobs as in that loop
        table = []
        for rec in ctx.records:
            st = self._state(rec)
            m = rec.mask_u8() if use_mask else None
            table.append(dict(
                p=rec.main_param.data.view(-1), g=rec.grad.data.view(-1),
                m=st["exp_avg"].view(-1), v=st["exp_avg_sq"].view(-1), mask=m, lr=rec.lr,
                beta1=rec.beta1, beta2=rec.beta2, eps=rec.eps, weight_decay=rec.weight_decay,
                step=rec.step, coeff_on=m is not None, clear=clear and m is not None,
                fold=fold and m is not None,
                inactive_lr_scale=inactive_lr_scale if m is not None else 1.0))
        adamw_grad_correct_multi(table, emit_score=emit_score, coeff=coeff, interval=interval,
                                 _adams=self._adams)

    def _records_pass_compact(self, ctx, coeff=1.0, fold=False, interval=1.0):
        # records of buckets with communicated values: one merge-join launch;
        # the others (no support in their bucket): one plain-commit launch
        compact, plain = [], []
        for rec in ctx.records:
            st = self._state(rec)
            bs = rec.bucket_state
            values = ctx.compact_values.get(id(bs))
            base = dict(p=rec.main_param.data.view(-1), g=rec.grad.data.view(-1),
                        m=st["exp_avg"].view(-1), v=st["exp_avg_sq"].view(-1), lr=rec.lr,
                        beta1=rec.beta1, beta2=rec.beta2, eps=rec.eps,
                        weight_decay=rec.weight_decay, step=rec.step)
            if values is None:
                plain.append(dict(base, mask=None, coeff_on=False))
                continue
            bucket = ctx.support.buckets[bs.support_index]
            table = bucket.dir_table if self.compact_search == "table" else None
            compact.append(dict(base, idx=bucket.idx, values=values, rec_start=rec.start,
                                dir_table=table))
        adamw_grad_correct_multi(plain, _adams=self._adams)
        adamw_grad_correct_compact_multi(compact, coeff=coeff, fold=fold, interval=interval,
                                         _adams=self._adams)

    @torch.no_grad()
    def full_step(self, ctx):
        split = self.full_sync_inactive_lr_scale != 1.0
        self._records_pass(ctx, emit_score=self.emit_score, use_mask=split,
                           inactive_lr_scale=(self.full_sync_inactive_lr_scale
                                              if split else 1.0))

    @torch.no_grad()
    def sparse_step(self, ctx):
        fold = self.residual_mean and ctx.next_step_is_full
        if ctx.compact_values:
            self._records_pass_compact(ctx, coeff=float(ctx.apply_coeff), fold=fold,
                                       interval=float(ctx.fold_window))
            return
        self._records_pass(ctx, emit_score=None, use_mask=True,
                           coeff=float(ctx.apply_coeff), clear=True, fold=fold,
                           interval=float(ctx.fold_window))

    def reset(self, ctx, was_full):
        for bs in ctx.bucket_states:
            if was_full or bs.active_mask_u8 is None:
                bs.grad_data.zero_()
            for grad in bs.extra_main_grads:
                grad.zero_()
