"""The backend object handed to torch.compile(backend=CuteInductor(...).compiler).

Follows cute_kernels/cute_inductor/compiler.py:18-47 (reference): walk the dynamo graph, let every replace function look
at every node, then either hand the rewritten graph to torch's inductor or run it as it is. The rewritten nodes call
this package's public functions; while inductor (AOTAutograd) re-traces the graph those functions dispatch to their
torch.library custom ops, which is what `enable_cute_tracing` switches on.
"""

import os
from typing import Callable

import torch
from torch._dynamo import lookup_backend

from ..utils import enable_cute_tracing
from .rmsnorm import replace_rmsnorm
from .swiglu_packed import replace_swiglu_unchunked


def _debug() -> bool:
    # the reference prints both graphs unless DEBUG_CUTEINDUCTOR is switched off (compiler.py:15); quiet by default here
    return os.environ.get("DEBUG_CUTEINDUCTOR", "0").lower() in ("1", "true", "yes")


class CuteInductor:
    def __init__(
        self,
        use_torch_inductor_after_cute_inductor: bool = True,
        replace_functions=(replace_rmsnorm, replace_swiglu_unchunked),
    ) -> None:
        self.use_torch_inductor_after_cute_inductor = use_torch_inductor_after_cute_inductor
        self.replace_functions = list(replace_functions)

    def compiler(self, gm: torch.fx.GraphModule, example_inputs: list[torch.Tensor]) -> Callable:
        with enable_cute_tracing():
            if _debug():
                print("graph before cute inductor")
                gm.print_readable()

            for replace_function in self.replace_functions:
                for node in list(gm.graph.nodes):  # a copy: replace functions erase nodes while we walk
                    if node.graph is gm.graph and not getattr(node, "_erased", False):
                        replace_function(gm, node)

            gm.graph.lint()
            gm.recompile()

            if _debug():
                print("graph after cute inductor")
                gm.print_readable()

            if self.use_torch_inductor_after_cute_inductor:
                return lookup_backend("inductor")(gm, example_inputs)
            return gm.forward
