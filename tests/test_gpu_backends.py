"""GPU parity of the two sparse-sync layouts' data movement (what one rank
hands to and takes back from the all-reduce) against the CPU oracle:
mask layout (`torch_pipelined_mask.py:91-138`: per slice [i*(N//s), ...) the
ordered compaction grad[s:e][mask] * factor, later written back in place) and
index layout (`torch_pipelined_index.py:314-325, 483-520`: sorted int32 idx,
values packed slice by slice, bucket-midpoint split for two slices).  All
results are data movement plus one fp32 multiply: bitwise."""
import pytest
import torch

from oracle import kernels as OK
from tests.util import adv, same_bits

pytestmark = pytest.mark.gpu


def _case(n, dens, seed, adversarial=False):
    gen = torch.Generator().manual_seed(seed)
    grad = adv(n, seed) if adversarial else torch.randn(n, generator=gen)
    mask = (torch.rand(n, generator=gen) < dens).to(torch.uint8)
    return grad, mask


@pytest.mark.parametrize("slices", [1, 2, 3])
@pytest.mark.parametrize("factor", [1.0, 0.5, 0.125])
@pytest.mark.parametrize("n,dens,off", [(1001, 0.25, 0), (300_001, 0.25, 0), (70_003, 0.9, 1),
                                        (4097, 0.0, 0), (5, 1.0, 0)])
def test_mask_layout_matches_oracle(dev, n, dens, off, factor, slices):
    """Odd n (the N // slices cut falls inside the bucket), factor != 1, an
    unaligned base pointer (off = 1), empty and full masks."""
    from sga_amd import backends
    grad_full, mask_full = _case(n + off, dens, 11 + slices)
    grad, mask = grad_full[off:], mask_full[off:]
    ref = OK.mask_layout_pack(grad, mask, factor, slices)
    dgrad, dmask = grad_full.to(dev)[off:], mask_full.to(dev)[off:]
    payloads, idx = backends.mask_layout_pack(dgrad, dmask, factor=factor, slices=slices)
    assert len(payloads) == len(ref) == slices
    for got, want in zip(payloads, ref):
        assert got.dtype == torch.float32 and same_bits(got, want)
    assert torch.equal(dgrad.cpu(), grad)                       # the pack is a pure read
    assert torch.equal(idx.cpu(), OK.compact_mask_u8(mask))
    # "reduced" payloads (what the all-reduce would hand back) written in place
    red_ref = [p * 3.0 + 1.0 for p in ref]
    want = grad.clone()
    OK.mask_layout_unpack(want, mask, red_ref, slices)
    backends.mask_layout_unpack(dgrad, idx, [p.to(dev) for p in red_ref])
    assert same_bits(dgrad, want)


def test_mask_layout_adversarial_lanes(dev):
    from sga_amd import backends
    grad, mask = _case(65_537, 0.5, 3, adversarial=True)
    ref = OK.mask_layout_pack(grad, mask, 0.125, 2)
    payloads, _ = backends.mask_layout_pack(grad.to(dev), mask.to(dev), factor=0.125, slices=2)
    for got, want in zip(payloads, ref):
        assert same_bits(got, want)


@pytest.mark.parametrize("vdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("slices", [1, 2, 3])
@pytest.mark.parametrize("factor", [1.0, 0.5])
def test_index_layout_matches_oracle(dev, vdtype, slices, factor):
    """Compact emission: values = gather * factor in idx order, packed
    positions zeroed; slice ranges = midpoint split (2) or even split."""
    from sga_amd import backends
    n = 200_003
    grad, mask = _case(n, 0.1, 5)
    mask[: n // 2 - 7000] = 0                        # lopsided: the midpoint split is far from k // 2
    idx = OK.compact_mask_u8(mask)
    k = idx.numel()
    g_ref, v_ref = grad.clone(), torch.empty(k, dtype=vdtype)
    b_ref = OK.index_layout_pack(g_ref, idx, v_ref, factor, slices)
    g_dev, v_dev = grad.to(dev), torch.empty(k, dtype=vdtype, device=dev)
    b_dev = backends.index_layout_pack(g_dev, idx.to(dev), v_dev, factor, slices)
    assert b_dev == b_ref and b_ref[-1][1] == k
    if slices == 2:
        assert b_ref[0][1] == int((idx < n // 2).sum()) != k // 2
    assert same_bits(v_dev, v_ref) and same_bits(g_dev, g_ref)
    # writeback emission: the reduced values scattered back over the zeroed positions
    red = (v_ref.float() * 2.0)
    OK.scatter_selected(g_ref, idx, red)
    backends.index_layout_writeback(g_dev, idx.to(dev), red.to(dev))
    assert same_bits(g_dev, g_ref)


def test_index_layout_empty_and_single(dev):
    from sga_amd import backends
    grad = torch.arange(10, dtype=torch.float32)
    for ix in (torch.empty(0, dtype=torch.int32), torch.tensor([7], dtype=torch.int32)):
        g_ref, v_ref = grad.clone(), torch.empty(ix.numel())
        OK.index_layout_pack(g_ref, ix, v_ref, 0.5, 2)
        g_dev, v_dev = grad.to(dev), torch.empty(ix.numel(), device=dev)
        assert backends.index_layout_pack(g_dev, ix.to(dev), v_dev, 0.5, 2) == \
            OK.index_layout_bounds(ix, 10, 2)
        assert same_bits(v_dev, v_ref) and same_bits(g_dev, g_ref)
