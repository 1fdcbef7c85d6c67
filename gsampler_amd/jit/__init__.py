from .module import compile  # noqa: F401
from .trace import GSTracer, gs_symbolic_trace  # noqa: F401
