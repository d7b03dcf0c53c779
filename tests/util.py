import numpy as np
import torch


def adv(n, seed, nonneg=False):
    """Adversarial fp32 lanes: specials (+-0, min/max normal, min denormal,
    1e+-20, near-tie constants) + random finite bit patterns -- the lane
    families of the reference's tests/test_replay_kernels.py:49-64."""
    g = np.random.default_rng(seed)
    parts = [np.array([0.0, -0.0, 1.0, -1.0, 2.0 ** -126, 2.0 ** -149, 2.0 ** 127,
                       -(2.0 ** 127), 1e-8, 1e-20, 1e20, 0.9, 0.999], dtype=np.float32)]
    got = parts[0].size
    while got < n:
        b = g.integers(-2 ** 31, 2 ** 31, size=n, dtype=np.int32)
        f = b.view(np.float32)
        f = f[np.isfinite(f)]
        parts.append(f)
        got += f.size
    v = np.concatenate(parts)[:n]
    return torch.from_numpy(np.abs(v) if nonneg else v.copy())


def student_t(n, seed, nu=3, scale=1e-3):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(n, generator=g)
    chi = torch.randn(nu, n, generator=g).pow(2).sum(0)
    return z / torch.sqrt(chi / nu) * scale


def same_bits(a, b):
    """Bitwise equality of two float tensors (signed zeros and NaN payloads
    included): the device ran the same IEEE-754 chain as the oracle."""
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    it = {torch.float32: torch.int32, torch.float64: torch.int64, torch.bfloat16: torch.int16}[a.dtype]
    return bool(torch.equal(a.view(it), b.view(it)))


def rel_close(a, b, rtol=1e-6, atol=0.0, scale=None):
    """|a-b| <= rtol*max(|a|,|b|,scale) + atol, elementwise.  ``scale`` carries
    the magnitude of the operands of a final subtraction (p' = p - lr*update):
    where that subtraction cancels, 1e-6 "relative" is only meaningful against
    its operands.  Returns (#bad lanes, worst abs error)."""
    a, b = a.double().cpu(), b.double().cpu()
    err = (a - b).abs()
    mag = torch.maximum(a.abs(), b.abs())
    if scale is not None:
        mag = torch.maximum(mag, scale.double().cpu().abs())
    bad = err > rtol * mag + atol
    return int(bad.sum()), float(err.max()) if err.numel() else 0.0


def sub_scale(p_old, p_new_ref):
    """Operand scale of p' = p - step: max(|p|, |step|)."""
    return torch.maximum(p_old.abs(), (p_new_ref - p_old).abs())
