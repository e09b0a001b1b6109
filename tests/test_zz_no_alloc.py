"""The expert sort for callers that cannot allocate (``ck_moe_sort_noalloc``): its workspace is a device array
inside the library, so the call itself must make no allocation and must give what ``ck_moe_sort`` gives.

Called through the C ABI (the ctypes handle, raw pointers).  Every case runs two sorts in a row through the
shared array, the second with a smaller input, and a third that uses the array in its other role (the key /
value ping-pong buffers of a multi-pass single-workgroup sort), each compared bit for bit with ``ck_moe_sort``
on a workspace of its own.  This file is collected last on purpose."""

import pytest
import torch

from helpers import announce

pytestmark = pytest.mark.gpu


def _reference_sort(lib, ids, E, stream):
    M = ids.numel()
    out = [torch.full((M,), -1, dtype=torch.int64, device=ids.device) for _ in range(2)]
    offsets = torch.full((E,), -1, dtype=torch.int64, device=ids.device)
    need = lib.ck_moe_sort_workspace_size(M, E)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=ids.device)
    status = lib.ck_moe_sort(ids.data_ptr(), int(ids.dtype == torch.int32), out[0].data_ptr(), out[1].data_ptr(),
                             offsets.data_ptr(), ws.data_ptr(), ws.numel(), M, E, stream)
    assert status == 0
    return out[0], out[1], offsets


def _skewed_ids(M, E, seed, dtype, device):
    g = torch.Generator().manual_seed(seed)
    weights = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.2
    weights[E // 2] = 0.0  # an expert nobody selects
    return torch.multinomial(weights, M, replacement=True, generator=g).to(dtype).to(device)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_moe_sort_noalloc_matches_moe_sort(gpu, dtype):
    from cute_kernels import _C

    lib = _C.load_library()
    stream = torch.cuda.current_stream().cuda_stream
    # (M, E): grid-wide sort; the same, smaller; multi-pass single-workgroup sort (E > 256, M below the grid
    # threshold); one pass without any workspace; nothing to sort
    cases = [(98304, 64), (20000, 8), (5000, 300), (1000, 8), (0, 8)]
    # The first call on a device looks the array's address up (and has the code object loaded): it is the set-up
    # call, made outside any stream capture, and is not one of the measured ones.
    warm = _skewed_ids(4096, 8, 99, dtype, gpu)
    w_out = [torch.empty(4096, dtype=torch.int64, device=gpu) for _ in range(3)]
    assert lib.ck_moe_sort_noalloc(warm.data_ptr(), int(dtype == torch.int32), w_out[0].data_ptr(), w_out[1].data_ptr(),
                                   w_out[2].data_ptr(), 4096, 8, stream) == 0
    torch.cuda.synchronize()
    for i, (M, E) in enumerate(cases):
        announce("ck_moe_sort_noalloc", f"M={M} E={E} {dtype}")
        ids = _skewed_ids(M, E, 100 + i, dtype, gpu) if M else torch.empty(0, dtype=dtype, device=gpu)
        expected = _reference_sort(lib, ids, E, stream)
        got = [torch.full((M,), -1, dtype=torch.int64, device=gpu) for _ in range(2)]
        offsets = torch.full((E,), -1, dtype=torch.int64, device=gpu)
        # Once unmeasured with this case's shape, so that whatever the runtime sets up lazily for a launch configuration
        # it has not seen (argument buffers, code) exists before the measured call; a library that allocated per call
        # would do so again there.
        assert lib.ck_moe_sort_noalloc(ids.data_ptr(), int(dtype == torch.int32), got[0].data_ptr(), got[1].data_ptr(),
                                       offsets.data_ptr(), M, E, stream) == 0
        torch.cuda.synchronize()
        for t in (*got, offsets):
            t.fill_(-1)
        torch.cuda.synchronize()
        # torch's allocator counters see nothing the library would allocate by itself; the driver's count of free
        # device memory does
        before = torch.cuda.memory_stats(gpu)["allocation.all.allocated"], torch.cuda.memory_reserved(gpu)
        free_before = torch.cuda.mem_get_info(gpu)[0]
        status = lib.ck_moe_sort_noalloc(ids.data_ptr(), int(dtype == torch.int32), got[0].data_ptr(),
                                         got[1].data_ptr(), offsets.data_ptr(), M, E, stream)
        free_during = torch.cuda.mem_get_info(gpu)[0]
        after = torch.cuda.memory_stats(gpu)["allocation.all.allocated"], torch.cuda.memory_reserved(gpu)
        assert status == 0, lib.ck_status_string(status)
        assert before == after  # nothing taken from torch's allocator either
        torch.cuda.synchronize()
        assert free_during == free_before == torch.cuda.mem_get_info(gpu)[0], "device memory taken or given back by the call"
        assert torch.equal(got[0], expected[0]), f"sorted ids differ (M={M}, E={E})"
        assert torch.equal(got[1], expected[1]), f"sorted positions differ (M={M}, E={E})"
        assert torch.equal(offsets, expected[2]), f"offsets differ (M={M}, E={E})"
        if M:
            assert torch.equal(ids.long()[got[1]], got[0])  # the permutation really sorts the input
            assert torch.equal(offsets, torch.bincount(ids.long(), minlength=E).cumsum(0))


def test_moe_sort_noalloc_binding_and_limit(gpu):
    from cute_kernels import _C

    ids = _skewed_ids(16384, 8, 7, torch.int64, gpu)
    out = [torch.empty_like(ids) for _ in range(2)]
    offsets = torch.empty(8, dtype=torch.int64, device=gpu)
    _C.moe_sort_noalloc(ids, out[0], out[1], offsets, 8)
    values, positions = torch.sort(ids, stable=True)
    assert torch.equal(out[0], values) and torch.equal(out[1], positions)
    # beyond the array: refused with the status for it, nothing launched
    big = torch.zeros((1 << 20) + 1, dtype=torch.int32, device=gpu)
    o = [torch.empty(big.numel(), dtype=torch.int64, device=gpu) for _ in range(2)]
    offs = torch.full((512,), -5, dtype=torch.int64, device=gpu)
    with pytest.raises(RuntimeError, match="scratch"):
        _C.moe_sort_noalloc(big, o[0], o[1], offs, 512)
    torch.cuda.synchronize()
    assert bool((offs == -5).all())
