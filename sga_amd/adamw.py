"""The SGA AdamW optimizer template on MI355X
(``sga/plugins/optimizer/adamw.py``): ``adamw_grad_correct``,
``adamw_grad_correct_compact``, ``build_dir_table`` and ``SgaAdamW`` with the
reference's signatures, refusals and step order."""
import math
from dataclasses import dataclass, field
from types import SimpleNamespace
from typing import Optional

import torch

from . import _lib as L
from .scores import SCORE_MAP

_BLOCK_SIZE = 1024


def _flat32(**named):
    for name, t in named.items():
        if t is None:
            continue
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be fp32")
    L.require_contig(**named)


def adamw_grad_correct(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer,
                       lr, beta1, beta2, eps, weight_decay, step, mask=None,
                       emit_score: Optional[str] = None, coeff=1.0, clear=False,
                       fold=False, interval=1.0, inactive_lr_scale=1.0, _adams=False):
    """One fused commit on contiguous same-size 1-D fp32 buffers
    (``adamw.py:502-634``).  ``emit_score=None`` is the sparse step; a score
    name is the full step that also writes that score into ``grad_buffer``."""
    bias_correction1 = 1.0 - beta1 ** step
    bias_correction2 = 1.0 - beta2 ** step
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
        return
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
    if _adams:
        flags |= L.GC_ADAMS
    L.call("sga_adamw_grad_correct", L.ptr(param_buffer), L.ptr(grad_buffer),
           L.ptr(exp_avg_buffer), L.ptr(exp_avg_sq_buffer), L.ptr(mk), n, L.f32(lr),
           L.f32(beta1), L.f32(1.0 - beta1), L.f32(beta2), L.f32(1.0 - beta2),
           L.f32(eps), L.f32(weight_decay), L.f32(bias_correction1),
           L.f32(bias_correction2), L.f32(coeff), L.f32(interval),
           L.f32(lr * inactive_lr_scale),
           SCORE_MAP[emit_score] if emit_score is not None else -1, flags, L.stream())


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


def adamw_grad_correct_compact(param_buffer, grad_buffer, exp_avg_buffer,
                               exp_avg_sq_buffer, idx, values, rec_start, lr, beta1,
                               beta2, eps, weight_decay, step, coeff=1.0, fold=False,
                               interval=1.0, dir_table=None, _adams=False):
    """Compact-emission commit: the gradient comes from the bucket-level sorted
    ``(idx, values)`` by merge-join (``adamw.py:637-792``).  ``values`` may be
    fp32 or bf16."""
    if not idx.is_contiguous() or not values.is_contiguous():
        raise ValueError("adamw_grad_correct_compact requires contiguous idx/values")
    bias_correction1 = 1.0 - beta1 ** step
    bias_correction2 = 1.0 - beta2 ** step
    n = param_buffer.numel()
    if n == 0:
        return
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
    flags = ((L.GC_APPLY_COEFF if coeff != 1.0 else 0) | (L.GC_FOLD if fold else 0)
             | (L.GC_ADAMS if _adams else 0))
    L.call("sga_adamw_grad_correct_compact", L.ptr(param_buffer), L.ptr(grad_buffer),
           L.ptr(exp_avg_buffer), L.ptr(exp_avg_sq_buffer), L.ptr(idx), L.ptr(values),
           L.dtype_code(values), rec_start, n, k_total, L.f32(lr), L.f32(beta1),
           L.f32(1.0 - beta1), L.f32(beta2), L.f32(1.0 - beta2), L.f32(eps),
           L.f32(weight_decay), L.f32(bias_correction1), L.f32(bias_correction2),
           L.f32(coeff), L.f32(interval), flags, L.ptr(dir_table), n_table, L.stream())


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
    """grad-correct + residual reset (``adamw.py:795-986``).  Constructed from
    an args namespace carrying the ``sga_*`` flags it reads."""

    def __init__(self, args=None):
        args = args or SimpleNamespace()
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

    def _records_pass(self, ctx, emit_score, use_mask, coeff=1.0, clear=False,
                      fold=False, interval=1.0, inactive_lr_scale=1.0):
        for rec in ctx.records:
            st = self._state(rec)
            m = rec.mask_u8() if use_mask else None
            self._commit(
                rec.main_param.data.view(-1), rec.grad.data.view(-1),
                st["exp_avg"].view(-1), st["exp_avg_sq"].view(-1), rec.lr, rec.beta1,
                rec.beta2, rec.eps, rec.weight_decay, rec.step, mask=m,
                emit_score=emit_score, coeff=coeff if m is not None else 1.0,
                clear=clear and m is not None, fold=fold and m is not None,
                interval=interval,
                inactive_lr_scale=inactive_lr_scale if m is not None else 1.0)

    def _records_pass_compact(self, ctx, coeff=1.0, fold=False, interval=1.0):
        for rec in ctx.records:
            st = self._state(rec)
            bs = rec.bucket_state
            values = ctx.compact_values.get(id(bs))
            if values is None:
                self._commit(
                    rec.main_param.data.view(-1), rec.grad.data.view(-1),
                    st["exp_avg"].view(-1), st["exp_avg_sq"].view(-1), rec.lr,
                    rec.beta1, rec.beta2, rec.eps, rec.weight_decay, rec.step)
                continue
            bucket = ctx.support.buckets[bs.support_index]
            table = bucket.dir_table if self.compact_search == "table" else None
            self._commit_compact(
                rec.main_param.data.view(-1), rec.grad.data.view(-1),
                st["exp_avg"].view(-1), st["exp_avg_sq"].view(-1), bucket.idx, values,
                rec.start, rec.lr, rec.beta1, rec.beta2, rec.eps, rec.weight_decay,
                rec.step, coeff=coeff, fold=fold, interval=interval, dir_table=table)

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
