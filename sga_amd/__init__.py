"""sga_amd -- MI355X-native kernels for SGA's per-rank sparse-gradient path.

Host side mirrors the reference's operator boundary (``sga/kernels.py``,
``sga/replay_kernels.py``, ``adamw_grad_correct*``, the selection / score
plugin API); every operator calls hand-written gfx950 kernels through the C
ABI in ``include/sga_hip.h``.  No Triton, no CPU fallback.
"""
from . import _lib  # noqa: F401

__all__ = ["kernels", "support", "scores", "adamw", "selection", "replay",
           "replay_kernels", "replay_fused", "fused_step", "backends"]
