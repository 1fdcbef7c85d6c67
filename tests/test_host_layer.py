"""Host-side checks that need no GPU: the operator library loads, registers the
reference's class / operator names, and rejects bad input with exceptions."""
import pytest
import torch

import gsampler_amd as gs

REFERENCE_METHODS = """_CAPI_LoadCSC _CAPI_LoadCOO _CAPI_LoadCSR _CAPI_GetNumRows _CAPI_GetNumCols
_CAPI_GetNumEdges _CAPI_GetCSCIndptr _CAPI_GetCSCIndices _CAPI_GetCSCEids _CAPI_GetCOORows
_CAPI_GetCOOCols _CAPI_GetCOOEids _CAPI_GetCSRIndptr _CAPI_GetCSRIndices _CAPI_GetCSREids
_CAPI_Slicing _CAPI_Sampling _CAPI_SamplingProbs _CAPI_RandomWalk _CAPI_Node2Vec _CAPI_SDDMM
_CAPI_SpMM _CAPI_Compact _CAPI_GraphRelabel _CAPI_GetValidNodes _CAPI_SlicingSampling
_CAPI_FusedUOPV _CAPI_FusedESquareSum _CAPI_FusedEDivUSum _CAPI_SortCSCIndices
_CAPI_BatchColSlicing _CAPI_BatchRowSlicing _CAPI_BatchColRowSlcing _CAPI_BatchRowSampling
_CAPI_BatchRowSamplingProbs _CAPI_BatchGraphRelabel _CAPI_BatchFusedSlicingSampling
_CAPI_GetEdgeBptr _CAPI_GetColBptr _CAPI_GetRowBptr _CAPI_SetEdgeBptr _CAPI_SetColBptr
_CAPI_SetRowBptr _CAPI_BatchSetRows _CAPI_BatchSetCols _CAPI_BatchGetRows _CAPI_BatchGetCols
_CAPI_BatchGetCSCIndptr _CAPI_BatchGetCSCIndices _CAPI_BatchGetCSCEids _CAPI_BatchGetCOORows
_CAPI_BatchGetCOOCols _CAPI_BatchGetCOOEids _CAPI_BatchGetColCounts
_CAPI_BatchGetValidNodes""".split()

REFERENCE_OPS = """_CAPI_ListSampling _CAPI_ListSamplingWithProbs _CAPI_BatchListSamplingWithProbs
_CAPI_BatchListSampling _CAPI_BatchSplitByOffset _CAPI_BatchIndptrSplitByOffset""".split()


def test_graph_class_has_every_reference_method():
    g = gs.Graph(4, 4)
    for name in REFERENCE_METHODS:
        assert hasattr(g, name), name
    assert len(REFERENCE_METHODS) == 55
    assert g._CAPI_GetNumRows() == 4 and g._CAPI_GetNumCols() == 4


def test_free_operators_registered():
    for name in REFERENCE_OPS:
        assert hasattr(torch.ops.gs_ops, name), name


def test_format_constants():
    assert (gs._COO, gs._CSC, gs._CSR) == (1, 2, 4)


def test_cpu_tensors_are_rejected_with_an_exception():
    g = gs.Graph(3, 3)
    with pytest.raises(RuntimeError, match="GPU"):
        g._CAPI_LoadCSC(torch.tensor([0, 1, 2, 3]), torch.tensor([0, 1, 2]))
    with pytest.raises(RuntimeError, match="no sparse format"):
        g._CAPI_GetCSCIndptr()


def test_sampler_state():
    gs.manual_seed(42)
    assert gs.random_state() == (42, 0)
    gs.manual_seed(7777)
    with pytest.raises(KeyError):
        gs.set_sampling_algorithm("bogus")
    gs.set_sampling_algorithm("auto")


def test_split_by_offset_on_cpu_data():
    parts = torch.ops.gs_ops._CAPI_BatchSplitByOffset(torch.arange(10), torch.tensor([0, 3, 3, 10]))
    assert [p.tolist() for p in parts] == [[0, 1, 2], [], [3, 4, 5, 6, 7, 8, 9]]
