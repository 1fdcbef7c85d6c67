"""A matrix whose CSC arrays stay in pinned host memory (the reference's UVA
mode, examples/graphsage/graphsage_e2e.py:62-66): the kernels read it in place
and every result equals the one from the same matrix in device memory."""
import pytest
import torch

import gsampler_amd as gs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def matrices():
    from gsampler_amd.utils import rmat_csc
    indptr, indices = rmat_csc(20000, 400000, seed=1)
    on_gpu, pinned = gs.Matrix(), gs.Matrix()
    on_gpu.load_graph("CSC", [indptr.to(DEV), indices.to(DEV)])
    pinned.load_graph("CSC", [indptr.pin_memory(), indices.pin_memory()])
    return on_gpu, pinned


def graphsage(A, seeds, fanouts):
    blocks = []
    for K in fanouts:
        sub = A[:, seeds].individual_sampling(K, None, False)
        seeds = sub.all_nodes()
        blocks.append(sub.to_dgl_block())
    return seeds, blocks


def same_blocks(a, b):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert torch.equal(x.row, y.row) and torch.equal(x.col, y.col)
        assert torch.equal(x.srcdata["_ID"], y.srcdata["_ID"])


def test_graphsage_eager_and_compiled(matrices):
    on_gpu, pinned = matrices
    seeds = torch.arange(0, 20000, 39, device=DEV)
    gs.manual_seed(5)
    want_nodes, want = graphsage(on_gpu, seeds, [15, 10, 5])
    gs.manual_seed(5)
    got_nodes, got = graphsage(pinned, seeds, [15, 10, 5])
    assert got_nodes.is_cuda and torch.equal(got_nodes, want_nodes)
    same_blocks(got, want)
    compiled = gs.jit.compile(func=graphsage, args=(pinned, seeds, [15, 10, 5]))
    gs.manual_seed(5)
    jit_nodes, jit_blocks = compiled(pinned, seeds, [15, 10, 5])
    assert torch.equal(jit_nodes, want_nodes)
    same_blocks(jit_blocks, want)


def test_column_slice_and_walks(matrices):
    on_gpu, pinned = matrices
    seeds = torch.arange(5, 20000, 97, device=DEV)
    a, b = on_gpu[:, seeds], pinned[:, seeds]
    for x, y in zip(a._graph._CAPI_GetCSCIndptr(), b._graph._CAPI_GetCSCIndptr()):
        assert x == y
    assert torch.equal(a._graph._CAPI_GetCSCIndices(), b._graph._CAPI_GetCSCIndices())
    gs.manual_seed(9)
    want = on_gpu.random_walk(seeds, 6)
    gs.manual_seed(9)
    got = pinned.random_walk(seeds, 6)
    assert got.is_cuda and torch.equal(got, want)


def test_format_conversion_is_refused(matrices):
    _, pinned = matrices
    with pytest.raises(RuntimeError, match="pinned host memory"):
        pinned._graph._CAPI_GetCSRIndptr()
