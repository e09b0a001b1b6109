"""The short prelude of the embedding backward (CK_EMBEDDING_BWD_PRELUDE=short: clear marks | set marks | one-workgroup
sort with the run heads, the zero fill riding on all three) against the default one (the grid-wide sort, seven launches):
both leave the same sorted pairs and run heads, so the row sums add the same values in the same order and the table
gradients are equal bit for bit.

Not collected by pytest (the file name): the variant has run on the CPU emulation only (tests/test_emulated_device.py
calls these bodies).  Run it by name on a GPU,
    python -m pytest tests/wip_embedding_short_prelude.py -x -q
and rename it to test_gpu_embedding_short_prelude.py once it passes there."""

import pytest
import torch

from helpers import acc_dtype, announce, assert_close, randn
from oracle import cute_oracle as O

pytestmark = pytest.mark.gpu


def ids_of(kind, V):
    if kind == "uniform":
        return torch.randint(0, V, (3, 700), generator=torch.Generator().manual_seed(31))
    if kind == "zipf":
        return O.zipf_ids((4, 2048), V, 1.1, seed=32)
    if kind == "one_row":
        return torch.full((3000,), 77, dtype=torch.long)
    if kind == "outside":  # ids outside the table are skipped (the forward writes zeros for them)
        ids = torch.randint(0, V, (900,), generator=torch.Generator().manual_seed(33))
        ids[::7] = V + 5
        ids[3::11] = -1
        return ids
    if kind == "int32":
        return torch.randint(0, V, (2, 300), generator=torch.Generator().manual_seed(34)).int()
    return torch.zeros((1,), dtype=torch.long)  # a single id


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("kind", ["uniform", "zipf", "one_row", "outside", "int32", "single"])
@pytest.mark.parametrize("table", [(5000, 1024), (300, 64), (131072 + 9, 8)])
def test_short_prelude_equals_the_default(gpu, monkeypatch, dtype, kind, table):
    from cute_kernels import _C

    V, H = table
    announce("embedding backward, short prelude", dtype, kind, table)
    ids = ids_of(kind, V)
    dy = randn((ids.numel(), H), dtype, 35)
    got = {}
    for prelude in ("grid", "short"):
        monkeypatch.setenv("CK_EMBEDDING_BWD_PRELUDE", prelude)
        dw = torch.full((V, H), float("nan"), dtype=dtype, device=gpu)
        ws = torch.empty(_C.embedding_backward_workspace_size(ids.numel(), V, H), dtype=torch.uint8, device=gpu)
        _C.embedding_backward(ids.reshape(-1).to(gpu), dy.to(gpu), dw, ws)
        got[prelude] = dw
    assert torch.equal(got["short"], got["grid"])
    inside = (ids.reshape(-1) >= 0) & (ids.reshape(-1) < V)
    expected = O.embedding_backward(ids.reshape(-1)[inside].long(), dy[inside], V, acc_dtype(dtype))
    assert_close(got["short"], expected, dtype, "weight_grad")
