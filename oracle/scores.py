"""Oracle score formulas (test infrastructure; torch CPU).

Restates the four registry scores of the reference
(``sga/plugins/scores.py:147-269``) as straight-line torch expressions.  Every
binary op below is one separately rounded fp32 elementwise op, in the same
order as the reference chain, so on the same host the bits agree with the
reference's torch path by construction:

    sa = (m*b1 + g*(1-b1)) / bc1
    sb = (v*b2 + (g*(1-b2))*g) / bc2            (AdamW, scores.py:183-190)
    sb = (m*m)*b2 + (g*(1-b2))*g                (AdamS, scores.py:191-197)
    U  = sa / (sqrt(sb) + eps)
    update = wd*w + U                           (scores.py:216-226)
    coi    = |U(g) - U(0)|                      (scores.py:253-269)

``abs_gr_over_sqrt_v`` is a build-side variant (|g|/sqrt(v+eps)) that has NO
reference counterpart: parity unpinned, checked only against its own closed
form in float64.
"""
import torch

from . import ieee

SCORE_IDS = {"update": 0, "abs_g": 1, "abs_m": 2, "coi": 3}  # adamw.py:75-80


def _moments(m, v, g, b1, b2, bc1, bc2, optimizer):
    """Folded, bias-corrected first/second moments (scores.py:167-199)."""
    sa = m * b1 + g * (1.0 - b1)
    gg = (g * (1.0 - b2)) * g
    if optimizer == "adamw":
        sb = v * b2 + gg
        sa = sa / bc1
        sb = sb / bc2
    elif optimizer == "adams":
        sb = (m * m) * b2 + gg
    else:
        raise ValueError(
            f"Unknown SGA optimizer '{optimizer}' for the score formulas "
            "(registered: adamw, adams)")
    return sa, sb


def abs_g(w, m, v, g, b1, b2, eps, wd, bc1, bc2, update_includes_wd=True,
          optimizer="adamw"):
    """|g| (scores.py:147-154)."""
    return g.abs()


def abs_m(w, m, v, g, b1, b2, eps, wd, bc1, bc2, update_includes_wd=True,
          optimizer="adamw"):
    """|m| of the pre-commit first moment (scores.py:157-164)."""
    return m.abs()


def update(w, m, v, g, b1, b2, eps, wd, bc1, bc2, update_includes_wd=True,
           optimizer="adamw"):
    """Signed materialized update ``wd*w + U(g)`` (scores.py:202-231)."""
    sa, sb = _moments(m, v, g, b1, b2, bc1, bc2, optimizer)
    den = ieee.sqrt(sb) + eps
    u = sa / den
    if update_includes_wd:
        return wd * w + u
    return u


def coi(w, m, v, g, b1, b2, eps, wd, bc1, bc2, update_includes_wd=True,
        optimizer="adamw"):
    """|U(g) - U(0)| (scores.py:234-269)."""
    sa, sb = _moments(m, v, g, b1, b2, bc1, bc2, optimizer)
    if optimizer == "adams":
        num0 = m * b1
        den0 = (m * m) * b2
    else:
        num0 = (m * b1) / bc1
        den0 = (v * b2) / bc2
    u0 = num0 / (ieee.sqrt(den0) + eps)
    ug = sa / (ieee.sqrt(sb) + eps)
    return (ug - u0).abs()


FORMULAS = {"update": update, "abs_g": abs_g, "abs_m": abs_m, "coi": coi}


def get_formula(name):
    """Registry lookup with the reference's error text (scores.py:119-126)."""
    try:
        return FORMULAS[name]
    except KeyError:
        raise ValueError(
            f"Unknown SGA score '{name}'. Registered: {sorted(FORMULAS)}"
        ) from None


def score_formula(name, w, m, v, g, b1, b2, eps, wd, bc1, bc2, optimizer,
                  update_includes_wd=False):
    """Replay-side routing (replay.py:486-505): AdamS substitutes v := m*m and
    pins both bias corrections to 1.0, then calls the AdamW-shaped formula."""
    f = get_formula(name)
    if optimizer == "adamw":
        return f(w, m, v, g, b1, b2, eps, wd, bc1, bc2,
                 update_includes_wd=update_includes_wd)
    return f(w, m, m * m, g, b1, b2, eps, wd, 1.0, 1.0,
             update_includes_wd=update_includes_wd)


def abs_gr_over_sqrt_v(g_plus_r, v, eps):
    """Build-side literal ``|g+r| / sqrt(v + eps)`` as three separately rounded
    fp32 ops (add, correctly rounded root, divide).  No reference
    implementation exists: PARITY UNPINNED (closed form only)."""
    return g_plus_r.abs() / ieee.sqrt(v + eps)


EXTRA_SCORES = ("abs_g_blind", "abs_gr_over_sqrt_v")


def step_score(name, w, m, v, q, g_alone, b1, b2, eps, wd, bc1, bc2, optimizer):
    """|score| as the fused step and the replay re-selection rank it: the
    four registry names through ``score_formula`` (update with its wd term),
    plus the two build-side benchmark scores -- ``abs_g_blind`` = |g_alone|
    (the gradient term without the residual) and ``abs_gr_over_sqrt_v`` (AdamS:
    v := m*m).  PARITY UNPINNED for the two extras (no reference counterpart)."""
    if name == "abs_g_blind":
        return g_alone.abs()
    if name == "abs_gr_over_sqrt_v":
        return abs_gr_over_sqrt_v(q, v if optimizer == "adamw" else m * m, eps)
    return score_formula(name, w, m, v, q, b1, b2, eps, wd, bc1, bc2, optimizer,
                         update_includes_wd=True).abs()
