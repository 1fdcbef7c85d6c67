// register.cc -- the drop-in boundary: registers gs_classes.Graph and the
// gs_ops free operators under the names the reference exposes
// (src/pybind.cc:9-78 of gSampler), so Python code written against
// torch.classes.gs_classes.Graph / torch.ops.gs_ops keeps working.
#include <torch/custom_class.h>
#include <torch/script.h>

#include "abi_call.h"
#include "graph.h"

namespace gs {

// Sampler state controls (no counterpart in the reference, whose seeds are
// compile-time literals).
static void set_random_seed(int64_t seed) {
  random_state().seed = (uint64_t)seed;
  random_state().next_call = 0;
}
static std::tuple<int64_t, int64_t> get_random_state() {
  return {(int64_t)random_state().seed, (int64_t)random_state().next_call};
}
static void set_next_call_id(int64_t id) { random_state().next_call = (uint64_t)id; }
static void set_sampling_algorithm(int64_t algo) {
  TORCH_CHECK(algo >= 0 && algo <= 2, "unknown sampling algorithm ", algo);
  random_state().algo = algo;
}
static int64_t abi_version() { return gs_abi_version(); }
// After a write to a graph or weight tensor that went around torch (a raw
// pointer, another extension, a replayed HIP graph): forget everything derived
// from tensor contents.
static void invalidate_all_caches() { invalidate_caches(); }
// Whether loaded matrices may keep an int32 copy of their ids (on by default).
static void set_narrow_ids(bool on) { narrow_ids_allowed().store(on); }

}  // namespace gs

using gs::BlockBatch;
using gs::Graph;

TORCH_LIBRARY(gs_classes, m) {
  m.class_<BlockBatch>("BlockBatch")
      .def("size", &BlockBatch::Size)
      .def("totals", &BlockBatch::Totals)
      .def("offsets", &BlockBatch::Offsets)
      .def("block", &BlockBatch::Block)
      .def("blocks", &BlockBatch::Blocks)
      .def("num_src_of", &BlockBatch::NumSrcOf)
      .def("frontier", &BlockBatch::Frontier)
      .def("frontier_ptr", &BlockBatch::FrontierPtr)
      .def("row", &BlockBatch::Row)
      .def("col", &BlockBatch::Col)
      .def("indptr", &BlockBatch::Indptr)
      .def("edge_ptr", &BlockBatch::EdgePtr)
      .def("col_ptr", &BlockBatch::ColPtr)
      .def("edge_ids", &BlockBatch::EdgeIds);
  m.class_<Graph>("Graph")
      .def(torch::init<int64_t, int64_t>())
      .def("_CAPI_LoadCSC", &Graph::LoadCSC)
      .def("_CAPI_LoadCOO", &Graph::LoadCOO)
      .def("_CAPI_LoadCSR", &Graph::LoadCSR)
      .def("_CAPI_GetNumRows", &Graph::GetNumRows)
      .def("_CAPI_GetNumCols", &Graph::GetNumCols)
      .def("_CAPI_GetNumEdges", &Graph::GetNumEdges)
      .def("_CAPI_GetCSCIndptr", &Graph::GetCSCIndptr)
      .def("_CAPI_GetCSCIndices", &Graph::GetCSCIndices)
      .def("_CAPI_GetCSCEids", &Graph::GetCSCEids)
      .def("_CAPI_GetCOORows", &Graph::GetCOORows)
      .def("_CAPI_GetCOOCols", &Graph::GetCOOCols)
      .def("_CAPI_GetCOOEids", &Graph::GetCOOEids)
      .def("_CAPI_GetCSRIndptr", &Graph::GetCSRIndptr)
      .def("_CAPI_GetCSRIndices", &Graph::GetCSRIndices)
      .def("_CAPI_GetCSREids", &Graph::GetCSREids)
      .def("_CAPI_Slicing", &Graph::Slicing)
      .def("_CAPI_Sampling", &Graph::Sampling)
      .def("_CAPI_SamplingProbs", &Graph::SamplingProbs)
      .def("_CAPI_RandomWalk", &Graph::RandomWalk)
      .def("_CAPI_Node2Vec", &Graph::Node2Vec)
      .def("_CAPI_SDDMM", &Graph::SDDMM)
      .def("_CAPI_SpMM", &Graph::SpMM)
      .def("_CAPI_Compact", &Graph::Compact)
      .def("_CAPI_GraphRelabel", &Graph::GraphRelabel)
      .def("_CAPI_GetValidNodes", &Graph::GetValidNodes)
      .def("_CAPI_SlicingSampling", &Graph::FusedSlicingSampling)
      .def("_CAPI_SlicingSamplingProbs", &Graph::FusedSlicingSamplingProbs)
      .def("_CAPI_FusedUOPV", &Graph::FusedUOPV)
      .def("_CAPI_FusedESquareSum", &Graph::FusedESquareSum)
      .def("_CAPI_FusedEDivUSum", &Graph::FusedEDivUSum)
      .def("_CAPI_SlicedESquareSum", &Graph::SlicedESquareSum)
      .def("_CAPI_ColRowSlicing", &Graph::ColRowSlicing)
      .def("_CAPI_SortCSCIndices", &Graph::SortCSCIndices)
      .def("_CAPI_BatchColSlicing", &Graph::BatchColSlicing)
      .def("_CAPI_BatchRowSlicing", &Graph::BatchRowSlicing)
      .def("_CAPI_BatchColRowSlcing", &Graph::BatchColRowSlcing)
      .def("_CAPI_BatchRowSampling", &Graph::BatchRowSampling)
      .def("_CAPI_BatchRowSamplingProbs", &Graph::BatchRowSamplingProbs)
      .def("_CAPI_BatchGraphRelabel", &Graph::BatchGraphRelabel)
      .def("_CAPI_BatchFusedSlicingSampling", &Graph::BatchFusedSlicingSampling)
      .def("_CAPI_BatchFusedSlicingSamplingProbs", &Graph::BatchFusedSlicingSamplingProbs)
      .def("_CAPI_GetEdgeBptr", &Graph::GetEdgeBptr)
      .def("_CAPI_GetColBptr", &Graph::GetColBptr)
      .def("_CAPI_GetRowBptr", &Graph::GetRowBptr)
      .def("_CAPI_SetEdgeBptr", &Graph::SetEdgeBptr)
      .def("_CAPI_SetColBptr", &Graph::SetColBptr)
      .def("_CAPI_SetRowBptr", &Graph::SetRowBptr)
      .def("_CAPI_BatchSetRows", &Graph::SetOrigRowIds)
      .def("_CAPI_BatchSetCols", &Graph::SetOrigColIds)
      .def("_CAPI_BatchGetRows", &Graph::BatchGetRows)
      .def("_CAPI_BatchGetCols", &Graph::BatchGetCols)
      .def("_CAPI_BatchGetCSCIndptr", &Graph::BatchGetCSCIndptr)
      .def("_CAPI_BatchGetCSCIndices", &Graph::BatchGetCSCIndices)
      .def("_CAPI_BatchGetCSCEids", &Graph::BatchGetCSCEids)
      .def("_CAPI_BatchGetCOORows", &Graph::BatchGetCOORows)
      .def("_CAPI_BatchGetCOOCols", &Graph::BatchGetCOOCols)
      .def("_CAPI_BatchGetCOOEids", &Graph::BatchGetCOOEids)
      .def("_CAPI_BatchGetColCounts", &Graph::BatchGetColCounts)
      .def("_CAPI_BatchGetValidNodes", &Graph::BatchGetValidNodes)
      .def("_CAPI_BatchBlocks", &Graph::BatchBlocks);
}

TORCH_LIBRARY(gs_ops, m) {
  m.def("_CAPI_ListSampling", &gs::ListSampling);
  m.def("_CAPI_ListSamplingWithProbs", &gs::ListSamplingProbs);
  m.def("_CAPI_BatchListSamplingWithProbs", &gs::BatchListSamplingProbs);
  m.def("_CAPI_BatchListSampling", &gs::BatchListSampling);
  m.def("_CAPI_BatchSplitByOffset", &gs::SplitByOffset);
  m.def("_CAPI_BatchIndptrSplitByOffset", &gs::SplitIndptrByOffset);
  m.def("_CAPI_GatherRows", &gs::GatherRows);
  m.def("_CAPI_SetRandomSeed", &gs::set_random_seed);
  m.def("_CAPI_GetRandomState", &gs::get_random_state);
  m.def("_CAPI_SetNextCallId", &gs::set_next_call_id);
  m.def("_CAPI_SetSamplingAlgorithm", &gs::set_sampling_algorithm);
  m.def("_CAPI_AbiVersion", &gs::abi_version);
  m.def("_CAPI_InvalidateCaches", &gs::invalidate_all_caches);
  m.def("_CAPI_SetNarrowIds", &gs::set_narrow_ids);
}
