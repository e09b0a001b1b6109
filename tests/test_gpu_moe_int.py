"""GPU parity, integer parts of the MoE layer: histogram, stable expert sort, offsets.  Bit-exact."""

import pytest
import torch

from helpers import announce
from oracle import cute_oracle as O


pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n", [0, 1, 63, 64, 65, 1000, 4099, 100000])
@pytest.mark.parametrize("size", [1, 8, 72, 4096, 5000])
def test_contiguous_count(gpu, dtype, n, size):
    from cute_kernels import contiguous_count_cute

    announce("contiguous_count", dtype, n, size)
    x = torch.randint(0, size, (n,), generator=torch.Generator().manual_seed(n + size)).to(dtype)
    out = contiguous_count_cute(x.to(gpu), size)
    assert out.dtype == torch.int32 and out.shape == (size,)
    assert torch.equal(out.cpu(), O.contiguous_count(x, size))
    assert torch.equal(out.cpu().long(), x.long().bincount(minlength=size))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("M,E", [(0, 8), (1, 1), (2, 8), (64, 2), (1000, 6), (16384, 8), (98304, 64), (5000, 72), (3000, 300), (70000, 1000),
                                 (16383, 8), (16385, 5), (32768, 8), (32769, 3), (100000, 300), (40000, 512), (50000, 1), (131071, 65)])
def test_moe_sort(gpu, dtype, M, E):
    from cute_kernels.kernels.scattermoe import moe_sort

    announce("moe_sort", dtype, M, E)
    g = torch.Generator().manual_seed(M + E)
    ids = torch.randint(0, E, (M,), generator=g).to(dtype)
    if E > 4 and M > 0:
        ids[ids == 3] = 2  # an expert that receives nothing
    s, idx, off = moe_sort(ids.to(gpu), E)
    es, eidx, eoff = O.moe_sort(ids, E)
    assert s.dtype == idx.dtype == off.dtype == torch.int64
    assert torch.equal(s.cpu(), es)
    assert torch.equal(idx.cpu(), eidx)
    assert torch.equal(off.cpu(), eoff)
    # same result as torch's stable sort and cumsum(bincount)
    ts, tidx = torch.sort(ids.long(), stable=True)
    assert torch.equal(s.cpu(), ts) and torch.equal(idx.cpu(), tidx)
    assert torch.equal(off.cpu(), ids.long().bincount(minlength=E).cumsum(-1))


def test_moe_sort_on_topk_output(gpu):
    """[T, k] selected experts exactly as the layer produces them (skewed: some experts empty)."""
    from cute_kernels.kernels.scattermoe import moe_sort

    announce("moe_sort topk")
    T, k, E = 4096, 6, 64
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g) + torch.linspace(3, -8, E)
    sel = logits.topk(k, dim=-1).indices
    s, idx, off = moe_sort(sel.to(gpu), E)
    es, eidx, eoff = O.moe_sort(sel, E)
    assert torch.equal(s.cpu(), es) and torch.equal(idx.cpu(), eidx) and torch.equal(off.cpu(), eoff)
    assert (eoff.diff() == 0).any(), "the case is meant to contain empty experts"


def test_offsets_from_sorted(gpu):
    from cute_kernels import _C

    announce("offsets_from_sorted")
    for M, E in [(0, 5), (10, 3), (5000, 72), (100000, 8)]:
        ids = torch.randint(0, E, (M,), generator=torch.Generator().manual_seed(M)).sort().values
        off = torch.empty(E, dtype=torch.int64, device=gpu)
        _C.offsets_from_sorted(ids.to(gpu), off)
        assert torch.equal(off.cpu(), ids.bincount(minlength=E).cumsum(-1))
