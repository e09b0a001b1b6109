"""Graph rewrite: ``torch.rms_norm(x, normalized_shape, weight, eps)`` -> ``rmsnorm_cute(x, weight, eps)``.

Same rewrite as cute_kernels/cute_inductor/rmsnorm.py:9-31.  ``F.rms_norm`` shows up in dynamo graphs as a
call to ``torch.rms_norm``; only normalisation over the last dimension is expressible by ``rmsnorm_cute``,
which is also all the reference handles.
"""

import torch
import torch.nn.functional as F
from torch.fx import Node
from torch.fx.graph_module import GraphModule

from ..kernels.rmsnorm import rmsnorm_cute


_RMS_NORM_TARGETS = (torch.rms_norm, F.rms_norm)
_ARG_NAMES = ("input", "normalized_shape", "weight", "eps")


def replace_rmsnorm(gm: GraphModule, node: Node) -> None:
    if node.op != "call_function" or node.target not in _RMS_NORM_TARGETS:
        return

    # normalise positional / keyword use into one dict, then drop normalized_shape
    bound = dict(zip(_ARG_NAMES, node.args))
    bound.update(node.kwargs)
    normalized_shape = bound.pop("normalized_shape", None)
    if normalized_shape is not None and len(normalized_shape) != 1:
        return  # more than the last dimension: leave it to torch

    x = bound.pop("input")
    kwargs = {"weight": bound.pop("weight", None), "eps": bound.pop("eps", None)}
    if bound:
        return  # unknown arguments: not the call we know how to replace

    with gm.graph.inserting_after(node):
        new_node = gm.graph.call_function(rmsnorm_cute, args=(x,), kwargs=kwargs)

    print("replacing with rmsnorm_cute")
    node.replace_all_uses_with(new_node)
    gm.graph.erase_node(node)
