"""torch.fx tracing of samplers written against Matrix / BatchMatrix.

A Matrix argument is rebuilt inside the traced function from its operator
object (`_graph`), so every Matrix method unfolds into `call_method` nodes whose
target is the `_CAPI_*` operator name -- the representation all rewrite passes
work on (same approach as the reference, python/gs/jit/trace.py:9-35)."""
import math

import torch
from torch.fx import GraphModule, Tracer

from ..matrix_api import Matrix


class GSTracer(Tracer):
    def __init__(self, autowrap_modules=(math,), autowrap_functions=(),
                 param_shapes_constant=False) -> None:
        super().__init__(autowrap_modules, autowrap_functions, param_shapes_constant)

    def create_arg(self, a):
        # a Matrix that escapes into a node argument is re-created from its graph
        if isinstance(a, Matrix):
            return self.create_proxy("call_function", a.__class__, (a._graph,), {}, None).node
        return super().create_arg(a)


def gs_symbolic_trace(root, concrete_args=None) -> GraphModule:
    tracer = GSTracer()
    graph = tracer.trace(root, concrete_args)
    name = root.__class__.__name__ if isinstance(root, torch.nn.Module) else root.__name__
    return GraphModule(tracer.root, graph, name)
