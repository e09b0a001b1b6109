"""``torch.compile`` backend that swaps known sub-graphs for this library's kernels.

Usage is the reference's (cute_kernels/cute_inductor/compiler.py:14-46):

    model = torch.compile(model, backend=CuteInductor().compiler)

Each replace function is called as ``f(gm, node)`` for every node of the captured FX graph and may rewrite
the graph in place.  Afterwards the graph is handed to Inductor (default) or run as is.
"""

from typing import Callable, Sequence

import torch
from torch._dynamo import lookup_backend

from ..utils import get_boolean_env_variable, set_cute_tracing
from .rmsnorm import replace_rmsnorm
from .swiglu_unchunked import replace_swiglu_unchunked


_DEBUG_CUTEINDUCTOR = get_boolean_env_variable("DEBUG_CUTEINDUCTOR", True)


class CuteInductor:
    def __init__(
        self,
        use_torch_inductor_after_cute_inductor: bool = True,
        replace_functions: Sequence[Callable] = (replace_rmsnorm, replace_swiglu_unchunked),
    ) -> None:
        self.use_torch_inductor_after_cute_inductor = use_torch_inductor_after_cute_inductor
        self.replace_functions = list(replace_functions)

    def compiler(self, gm: torch.fx.GraphModule, example_inputs: list[torch.Tensor]) -> Callable:
        # while set, cute ops go through their registered custom op, which later compilation can trace
        set_cute_tracing(True)
        try:
            if _DEBUG_CUTEINDUCTOR:
                print("graph before cute inductor")
                gm.print_readable()

            for replace_function in self.replace_functions:
                for node in list(gm.graph.nodes):
                    replace_function(gm, node)
            gm.graph.lint()
            gm.recompile()

            if _DEBUG_CUTEINDUCTOR:
                print("graph after cute inductor")
                gm.print_readable()

            if self.use_torch_inductor_after_cute_inductor:
                compiled = lookup_backend("inductor")(gm, example_inputs)
            else:
                compiled = gm.forward
        finally:
            set_cute_tracing(False)
        return compiled
