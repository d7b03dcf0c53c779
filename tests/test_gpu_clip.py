"""Masked clip service on the device vs the oracle (engine.py:1052-1218)."""
import copy
from types import SimpleNamespace

import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [40_001, 7, 65_536, 100_009]


class Rec:
    def __init__(self, grad, bucket, start, end):
        self.main_param = SimpleNamespace(grad=grad)
        self.bucket_state, self.start, self.end = bucket, start, end

    @property
    def grad(self):
        return self.main_param.grad

    def mask_u8(self):
        m = self.bucket_state.active_mask_u8
        return None if m is None else m[self.start:self.end]


def build(dev, with_mask=True, seed=0, maskless_tail=False):
    gen = torch.Generator().manual_seed(seed)
    n = sum(SIZES)
    flat = torch.randn(n, generator=gen) * 0.02
    mask = (torch.rand(n, generator=gen) < 0.05).to(torch.uint8) if with_mask else None
    b = SimpleNamespace(active_mask_u8=None if mask is None else mask.to(dev))
    b2 = SimpleNamespace(active_mask_u8=None)
    flat = flat.to(dev)
    recs, off = [], 0
    for i, s in enumerate(SIZES):
        bucket = b2 if (maskless_tail and i == len(SIZES) - 1) else b
        recs.append(Rec(flat[off:off + s], bucket, off, off + s))
        off += s
    return recs, flat, b


def norm64(recs, was_full):
    t = 0.0
    for r in recs:
        g = r.grad.double().cpu()
        m = None if was_full else r.mask_u8()
        t += float((g * g).sum() if m is None else (g[m.cpu() > 0] ** 2).sum())
    return t ** 0.5


@pytest.mark.parametrize("route", ["full", "sparse_fused", "sparse_dump", "maskless_tail", "noclip"])
def test_masked_clip_routes(dev, route):
    from oracle.clip import masked_clip_grad_norm as ref_clip
    from sga_amd.clip import masked_clip_grad_norm
    was_full = route == "full"
    recs, flat, _ = build(dev, seed=3, maskless_tail=route == "maskless_tail")
    cpu_recs, cpu_flat, _ = build(torch.device("cpu"), seed=3,
                                  maskless_tail=route == "maskless_tail")
    before = flat.clone()
    exact = norm64(cpu_recs, was_full)
    clip = 0.0 if route == "noclip" else 0.5 * exact
    dumps = route == "sparse_dump"
    n_d, c_d = masked_clip_grad_norm(recs, clip, was_full, trace_dumps=dumps)
    n_r, c_r = ref_clip(cpu_recs, clip, was_full, trace_dumps=dumps)
    assert abs(n_d - exact) <= 1e-5 * exact and abs(n_r - exact) <= 1e-5 * exact
    if route == "noclip":
        assert c_d == 1.0 and torch.equal(flat, before)
        return
    coeff = clip / (n_d + 1.0e-6)
    if route in ("sparse_fused", "maskless_tail"):
        assert c_d == float(coeff) and abs(c_d - c_r) <= 1e-5
    else:
        assert c_d == 1.0 and c_r == 1.0
    # which coordinates moved is the reference's; each is one fp32 multiply
    want = before.clone()
    c32 = torch.tensor(coeff, dtype=torch.float32, device=dev)
    for r in recs:
        m = None if was_full else r.mask_u8()
        seg = want[r.start:r.end]
        if route == "full" or (m is None and route == "maskless_tail"):
            seg.mul_(c32)
        elif route == "sparse_dump":
            seg[m > 0] *= c32
    assert torch.equal(flat, want)
    moved_ref = cpu_flat != before.cpu()
    assert torch.equal(moved_ref, (flat != before).cpu())


def test_masked_clip_compact(dev):
    from sga_amd.clip import masked_clip_grad_norm
    recs, flat, b = build(dev, seed=9)
    idx = b.active_mask_u8.nonzero().reshape(-1)
    vals = flat[idx].clone()
    exact = float(vals.double().pow(2).sum().sqrt())
    before, vbefore = flat.clone(), vals.clone()
    n_d, c_d = masked_clip_grad_norm(recs, 0.25 * exact, False,
                                     compact_values={id(b): vals})
    assert abs(n_d - exact) <= 1e-5 * exact
    assert c_d == float(0.25 * exact / (n_d + 1e-6)) and c_d < 1.0
    assert torch.equal(flat, before) and torch.equal(vals, vbefore)
    n2, c2 = masked_clip_grad_norm(recs, 0.25 * exact, False,
                                   compact_values={id(b): vals}, trace_dumps=True)
    assert n2 == n_d and c2 == 1.0
    assert torch.equal(vals, vbefore * torch.tensor(c_d, dtype=torch.float32, device=dev))
    with pytest.raises(RuntimeError):
        masked_clip_grad_norm(recs, 1.0, False, compact_values={123: vals})


def test_scale_masked_ragged(dev):
    from sga_amd.clip import scale_masked_
    gen = torch.Generator().manual_seed(1)
    for n in (1, 3, 1023, 4097):
        base = torch.randn(n + 1, generator=gen).to(dev)
        g = base[1:]                                   # misaligned view
        m = (torch.rand(n, generator=gen) < 0.5).to(torch.uint8).to(dev)
        want = torch.where(m > 0, g * torch.tensor(0.37, device=dev), g)
        scale_masked_(g, m, 0.37)
        assert torch.equal(g, want) and base[0] == base[0]
