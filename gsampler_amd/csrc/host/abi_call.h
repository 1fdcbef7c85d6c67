// abi_call.h -- glue between torch tensors and the C ABI of gsampler_hip.h.
// Tensors are plumbing here: device memory, the caching allocator and the
// current HIP stream.  All computation happens behind the C ABI.
#ifndef GS_HOST_ABI_CALL_H_
#define GS_HOST_ABI_CALL_H_

#include <c10/hip/HIPStream.h>
#include <torch/torch.h>

#include "../../../include/gsampler_hip.h"

namespace gs {

#define GS_CALL(expr)                                                        \
  do {                                                                       \
    int gs_rc__ = (expr);                                                    \
    TORCH_CHECK(gs_rc__ == GS_OK, "gsampler_hip error ", gs_rc__, ": ",      \
                gs_last_error());                                            \
  } while (0)

inline gs_stream_t cur_stream() {
  return (gs_stream_t)c10::hip::getCurrentHIPStream().stream();
}

// int64 CUDA tensor, contiguous; the reference aborts on anything else
// (src/graph_ops.cc:28 "Not implemented warning"), this raises instead.
inline torch::Tensor ids(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.defined(), name, " is undefined");
  if (t.numel() == 0 && t.scalar_type() == torch::kInt64) return t;  // "none"
  TORCH_CHECK(t.is_cuda(), name, " must live on the GPU (got ", t.device(), ")");
  TORCH_CHECK(t.scalar_type() == torch::kInt64, name, " must be int64 (got ",
              t.scalar_type(), ")");
  return t.contiguous();
}

inline const int64_t* cptr(const torch::Tensor& t) {
  return (t.defined() && t.numel() > 0) ? t.data_ptr<int64_t>() : nullptr;
}
inline int64_t* mptr(torch::Tensor& t) {
  return (t.defined() && t.numel() > 0) ? t.data_ptr<int64_t>() : nullptr;
}

inline torch::Tensor new_ids(int64_t n, const torch::Tensor& like) {
  return torch::empty({n}, like.options().dtype(torch::kInt64));
}

inline torch::Tensor new_workspace(size_t bytes, const torch::Tensor& like) {
  return torch::empty({(int64_t)(bytes > 0 ? bytes : 1)},
                      like.options().dtype(torch::kUInt8));
}

// Last element of a device prefix array (one blocking 8-byte copy).
inline int64_t read_last(const torch::Tensor& prefix) {
  return prefix[prefix.numel() - 1].item<int64_t>();
}

}  // namespace gs

#endif  // GS_HOST_ABI_CALL_H_
