"""The SGA AdamS optimizer template on MI355X
(``sga/plugins/optimizer/adams.py``): the AdamW commit with the second moment
rebuilt from the PRE-commit first moment, ``v' = beta2*m*m + (1-beta2)*g*g``,
and no bias corrections (hence no ``step`` argument)."""
from typing import Optional

from .adamw import SgaAdamW, adamw_grad_correct, adamw_grad_correct_compact


def adams_grad_correct(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, lr,
                       beta1, beta2, eps, weight_decay, mask=None,
                       emit_score: Optional[str] = None, coeff=1.0, clear=False, fold=False,
                       interval=1.0, inactive_lr_scale=1.0):
    """``adams.py:392-504``: same knobs and refusals as ``adamw_grad_correct``."""
    adamw_grad_correct(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer, lr, beta1,
                       beta2, eps, weight_decay, 1, mask=mask, emit_score=emit_score,
                       coeff=coeff, clear=clear, fold=fold, interval=interval,
                       inactive_lr_scale=inactive_lr_scale, _adams=True)


def adams_grad_correct_compact(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer,
                               idx, values, rec_start, lr, beta1, beta2, eps, weight_decay,
                               coeff=1.0, fold=False, interval=1.0, dir_table=None):
    """``adams.py:507-654``."""
    adamw_grad_correct_compact(param_buffer, grad_buffer, exp_avg_buffer, exp_avg_sq_buffer,
                               idx, values, rec_start, lr, beta1, beta2, eps, weight_decay, 1,
                               coeff=coeff, fold=fold, interval=interval, dir_table=dir_table,
                               _adams=True)


def _commit(p, g, m, v, lr, b1, b2, eps, wd, step, **kw):
    adams_grad_correct(p, g, m, v, lr, b1, b2, eps, wd, **kw)


def _commit_compact(p, g, m, v, idx, values, rec_start, lr, b1, b2, eps, wd, step, **kw):
    adams_grad_correct_compact(p, g, m, v, idx, values, rec_start, lr, b1, b2, eps, wd, **kw)


class SgaAdamS(SgaAdamW):
    """``adams.py:657-850``: feature-identical to SgaAdamW, AdamS step math."""
    _adams = True
    _commit = staticmethod(_commit)
    _commit_compact = staticmethod(_commit_compact)
