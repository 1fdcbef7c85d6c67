// pending.cc -- operators of the reference interface whose kernels are not
// built yet.  Each raises a clear error instead of computing on a fallback
// path.  This file shrinks as kernels land.
#include "abi_call.h"
#include "graph.h"

namespace gs {

#define GS_PENDING(what) \
  TORCH_CHECK(false, what, " is not implemented in this build of gsampler_amd")

GraphAndIndex Graph::Compact(int64_t) { GS_PENDING("Compact"); }
torch::Tensor Graph::RandomWalk(torch::Tensor, int64_t) { GS_PENDING("RandomWalk"); }
torch::Tensor Graph::Node2Vec(torch::Tensor, int64_t, double, double) {
  GS_PENDING("Node2Vec");
}
void Graph::SortCSCIndices() { GS_PENDING("SortCSCIndices"); }
GraphAndIndex Graph::BatchColRowSlcing(torch::Tensor, torch::Tensor, torch::Tensor,
                                       torch::Tensor) {
  GS_PENDING("BatchColRowSlcing");
}
}  // namespace gs
