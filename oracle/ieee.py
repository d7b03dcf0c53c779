"""Correctly rounded elementary operations for the oracle -- TEST INFRASTRUCTURE ONLY.

The reference's chains (``sga/plugins/scores.py:202-231``,
``sga/replay.py:687-744``) are sequences of IEEE-754 fp32 operations, one
rounding each.  On the CPU ``+ - * /`` of torch are exactly that, but
``torch.sqrt`` goes through a vector math library that is not correctly
rounded (on the build this was written on it differs from the IEEE result on
about one lane in five for arguments around 1e-10).  The oracle therefore
takes its square roots here: numpy's ``sqrt`` is the hardware instruction,
which IEEE-754 requires to be correctly rounded.

Pinned by ``tests/test_oracle_numeric.py::test_ieee_sqrt_is_correctly_rounded``:
for every result s the exact inequality ``(s - ulp/2)^2 <= x <= (s + ulp/2)^2``
holds (the squares of the 25-bit midpoints are exact in float64).
"""
import numpy as np
import torch


def sqrt(t):
    """Correctly rounded square root of a CPU float tensor, same dtype."""
    if t.device.type != "cpu":
        raise ValueError("oracle.ieee.sqrt: CPU tensors only")
    if t.numel() == 0:
        return t.clone()
    with np.errstate(invalid="ignore"):
        return torch.from_numpy(np.sqrt(t.detach().contiguous().numpy())).reshape(t.shape)
