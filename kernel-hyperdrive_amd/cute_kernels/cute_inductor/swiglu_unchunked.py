"""Graph rewrite: ``a, b = x.chunk(2, dim=-1); a * F.silu(b)`` -> ``swiglu_unchunked_cute(x)``.

Pattern of cute_kernels/cute_inductor/swiglu_unchunked.py:12-72: a chunk into two along the last dimension
whose second half feeds exactly one ``silu`` and whose first half is multiplied with that ``silu``; none of
the intermediate values may have another user.
"""

import operator

import torch
import torch.nn.functional as F
from torch.fx import Node
from torch.fx.graph_module import GraphModule

from ..kernels.swiglu_unchunked import swiglu_unchunked_cute


_MUL_TARGETS = (torch.mul, operator.mul)
_SILU_TARGETS = (F.silu, torch.nn.functional.silu)


def _chunk_arguments(node: Node):
    """(input, chunks, dim) of a ``chunk`` node, or None."""
    is_method = node.op == "call_method" and node.target == "chunk"
    is_function = node.op == "call_function" and node.target is torch.chunk
    if not (is_method or is_function):
        return None
    bound = dict(zip(("input", "chunks", "dim"), node.args))
    bound.update(node.kwargs)
    return bound.get("input"), bound.get("chunks"), bound.get("dim", 0)


def _sole_user(node: Node):
    return next(iter(node.users)) if len(node.users) == 1 else None


def _is_getitem(node: Node, index: int) -> bool:
    return node.op == "call_function" and node.target is operator.getitem and node.args[1] == index


def _match(chunk: Node):
    """Return the multiply node that ends the pattern rooted at ``chunk``, or None."""
    if len(chunk.users) != 2:
        return None
    halves = {}
    for user in chunk.users:
        for index in (0, 1):
            if _is_getitem(user, index):
                halves[index] = user
    if set(halves) != {0, 1}:
        return None
    up, gate = halves[0], halves[1]

    silu = _sole_user(gate)
    if silu is None or silu.op != "call_function" or silu.target not in _SILU_TARGETS:
        return None
    product = _sole_user(silu)
    if product is None or product.op != "call_function" or product.target not in _MUL_TARGETS:
        return None
    if _sole_user(up) is not product:
        return None
    if set(product.all_input_nodes) != {up, silu}:
        return None
    return product


def replace_swiglu_unchunked(gm: GraphModule, node: Node) -> None:
    arguments = _chunk_arguments(node)
    if arguments is None:
        return
    x, chunks, dim = arguments
    if chunks != 2 or dim != -1:
        return
    product = _match(node)
    if product is None:
        return

    print("replacing with swiglu_unchunked_cute")
    with gm.graph.inserting_after(product):
        new_node = gm.graph.call_function(swiglu_unchunked_cute, args=(x,))
    product.replace_all_uses_with(new_node)
    gm.graph.eliminate_dead_code()
