from .sddmm import *  # noqa: F401,F403
from .spmm import *  # noqa: F401,F403
from .fused_op import *  # noqa: F401,F403
