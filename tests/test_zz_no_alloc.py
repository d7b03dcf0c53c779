"""The allocation-free compact norm (sga_compact_norm_sq_noalloc) against the
entry point it is a variant of (sga_compact_norm_sq with a caller workspace),
through the C ABI: same bits in the total, on two calls in a row with the
second input smaller, and the refusal of sizes beyond the stated maximum."""
import ctypes as C

import pytest
import torch

from sga_amd import _lib as L

pytestmark = pytest.mark.gpu


def _ref_total(vals, start):
    """sga_compact_norm_sq on a fresh caller-provided partials workspace."""
    k = vals.numel()
    total = torch.full((1,), start, dtype=torch.float32, device=vals.device)
    partials = torch.empty(int(L.raw("sga_norm_partials", k)), dtype=torch.float32,
                           device=vals.device)
    L.call("sga_compact_norm_sq", L.ptr(vals), k, L.ptr(partials), L.ptr(total), L.stream())
    return total


def _noalloc_total(vals, start):
    total = torch.full((1,), start, dtype=torch.float32, device=vals.device)
    L.call("sga_compact_norm_sq_noalloc", L.ptr(vals), vals.numel(), L.ptr(total), L.stream())
    return total


def test_noalloc_norm_matches_workspace_norm_twice(dev):
    gen = torch.Generator().manual_seed(7)
    big = (torch.randn(3_000_001, generator=gen) * 1e-2).to(dev)      # many workgroups, ragged tail
    small = (torch.randn(1_237, generator=gen) * 3.0).to(dev)         # two workgroups: stale slots beyond
    for vals, start in ((big, 0.0), (small, 0.25)):
        got = _noalloc_total(vals, start)
        want = _ref_total(vals, start)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (got.item(), want.item())
        ref64 = float((vals.double() ** 2).sum()) + start
        assert abs(got.item() - ref64) <= 1e-5 * ref64
    # an unaligned view (scalar load path) and the accumulate-into-total contract
    view = big[1:70_001]
    got = _noalloc_total(view, 1.5)
    want = _ref_total(view, 1.5)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


def test_noalloc_norm_refuses_and_skips(dev):
    lib = L.load()
    total = torch.zeros(1, device=dev)
    vals = torch.ones(8, device=dev)
    # k == 0 is a silent no-op, like the reference's dispatcher (kernels.py:256-258)
    assert lib.sga_compact_norm_sq_noalloc(L.ptr(vals), 0, L.ptr(total), L.stream()) == 0
    # beyond the stated maximum: refused on the host, nothing is launched
    rc = lib.sga_compact_norm_sq_noalloc(L.ptr(vals), 1 << 31, L.ptr(total), L.stream())
    assert rc == -1 and b"exceeds the supported maximum" in lib.sga_last_error()
    rc = lib.sga_compact_norm_sq_noalloc(None, 8, L.ptr(total), L.stream())
    assert rc == -1
    torch.cuda.synchronize()
    assert total.item() == 0.0
