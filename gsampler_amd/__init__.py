"""gsampler_amd -- MI355X-native implementation of gSampler's matrix-centric
sampling hot path.  `import gsampler_amd as gs` mirrors the reference's `gs`
package for that path: gs.Matrix, gs.BatchMatrix, gs.ops, gs.jit.compile,
gs.Graph.  Kernels live behind the C ABI of include/gsampler_hip.h
(libgsampler_hip.so); libgs.so registers the operator class with PyTorch."""
from . import _library

_library.load()

import torch  # noqa: E402

from . import capi, jit, ops, utils  # noqa: E402,F401
from .jit import GSTracer, compile, gs_symbolic_trace  # noqa: E402,F401
from .format import _COO, _CSC, _CSR  # noqa: E402,F401
from .matrix_api import BatchMatrix, Matrix  # noqa: E402,F401

Graph = torch.classes.gs_classes.Graph


def manual_seed(seed: int) -> None:
    """Seeds the sampler: every sampling call afterwards uses Philox streams
    (seed, call id) with call ids counted from 0."""
    torch.ops.gs_ops._CAPI_SetRandomSeed(int(seed))


def random_state():
    """(seed, id the next sampling call will use)."""
    return tuple(torch.ops.gs_ops._CAPI_GetRandomState())


def set_sampling_algorithm(name: str) -> None:
    """'auto' (Floyd for fanout <= 64, else reservoir), 'reservoir' or 'floyd'."""
    torch.ops.gs_ops._CAPI_SetSamplingAlgorithm({"auto": 0, "reservoir": 1, "floyd": 2}[name])
