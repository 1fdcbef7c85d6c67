// abi_call.h -- glue between torch tensors and the C ABI of gsampler_hip.h.
// Tensors are plumbing here: device memory, the caching allocator and the
// current HIP stream.  All computation happens behind the C ABI.
#ifndef GS_HOST_ABI_CALL_H_
#define GS_HOST_ABI_CALL_H_

#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <atomic>
#include <torch/torch.h>

#include <vector>

#include "../../../include/gsampler_hip.h"

namespace gs {

#define GS_CALL(expr)                                                        \
  do {                                                                       \
    int gs_rc__ = (expr);                                                    \
    TORCH_CHECK(gs_rc__ == GS_OK, "gsampler_hip error ", gs_rc__, ": ",      \
                gs_last_error());                                            \
  } while (0)

// Everything the operators remember between calls (the int32 copy of a matrix's
// ids, its weight CDF, offsets read back to the host, the frontier of the last
// relabel, ...) is keyed by the identity and version counter of the tensors it
// was made from.  A write that goes around torch (another extension, a raw
// pointer, a replayed HIP graph) changes the memory without moving that counter:
// whoever makes one calls invalidate_caches(), which ages everything at once.
// Entries carry the epoch they were made in and are ignored in a later one.
inline std::atomic<int64_t>& cache_epoch_counter() {
  static std::atomic<int64_t> epoch{0};
  return epoch;
}
inline int64_t cache_epoch() { return cache_epoch_counter().load(std::memory_order_relaxed); }
inline void invalidate_caches() { cache_epoch_counter().fetch_add(1); }

// Whether a loaded matrix may keep an int32 copy of its ids for the uniform
// sampler (4 bytes per edge of device memory for half the bytes behind a pick).
inline std::atomic<bool>& narrow_ids_allowed() {
  static std::atomic<bool> on{true};
  return on;
}

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

// Structure arrays of a loaded matrix may also sit in pinned host memory, which
// the kernels read in place over the host link (the reference's UVA mode:
// examples/graphsage/graphsage_e2e.py:62-66 pins indptr / indices before
// load_graph).  Everything an operator produces lives on the GPU.
inline torch::Tensor graph_ids(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.defined(), name, " is undefined");
  TORCH_CHECK(t.is_cuda() || t.is_pinned(), name,
              " must live on the GPU or in pinned host memory (got ", t.device(), ")");
  TORCH_CHECK(t.scalar_type() == torch::kInt64, name, " must be int64 (got ",
              t.scalar_type(), ")");
  return t.contiguous();
}

// Options of a fresh output: on the device of `like`, or on the current GPU
// when `like` is a pinned host tensor.
inline torch::TensorOptions device_options(const torch::Tensor& like) {
  if (like.is_cuda()) return like.options();
  return like.options()
      .device(c10::Device(c10::kCUDA, c10::hip::current_device()))
      .pinned_memory(false);
}

inline torch::Tensor new_ids(int64_t n, const torch::Tensor& like) {
  return torch::empty({n}, device_options(like).dtype(torch::kInt64));
}

inline torch::Tensor new_workspace(size_t bytes, const torch::Tensor& like) {
  return torch::empty({(int64_t)(bytes > 0 ? bytes : 1)},
                      device_options(like).dtype(torch::kUInt8));
}

// Last element of a device prefix array (one blocking 8-byte copy).
inline int64_t read_last(const torch::Tensor& prefix) {
  return prefix[prefix.numel() - 1].item<int64_t>();
}

// The same value without stalling the GPU: the copy into pinned host memory is
// queued on the current stream at once, get() waits for it.  Work launched in
// between (into buffers sized by an upper bound) keeps the GPU busy while the
// value travels.  Slots come from a small per-thread ring of pinned words that
// lives until the process ends; a slot is reused after kSlots later reads.
class AsyncCount {
 public:
  AsyncCount() = default;
  explicit AsyncCount(const torch::Tensor& prefix) {
    Ring& r = ring();
    ticket_ = r.next++;
    slot_ = (int)(ticket_ % kSlots);
    hipStream_t s = (hipStream_t)cur_stream();
    const int64_t* src = prefix.data_ptr<int64_t>() + prefix.numel() - 1;
    GS_CALL(gs_copy_i64(src, 1, r.words + slot_, (gs_stream_t)s));
    check(hipEventRecord(r.events[slot_], s));
    pending_ = true;
  }
  // For a kernel that stores the value to the host itself: hand it mirror(),
  // then arm() once it is queued.
  static AsyncCount mirrored() {
    AsyncCount c;
    Ring& r = ring();
    c.ticket_ = r.next++;
    c.slot_ = (int)(c.ticket_ % kSlots);
    return c;
  }
  bool requested() const { return slot_ >= 0; }
  int64_t* mirror() const { return ring().words + slot_; }
  void arm() {
    check(hipEventRecord(ring().events[slot_], (hipStream_t)cur_stream()));
    pending_ = true;
  }
  int64_t get() {
    TORCH_CHECK(slot_ >= 0, "AsyncCount: nothing was requested");
    Ring& r = ring();
    if (pending_) {
      // every operator reads its counts before it returns; one left waiting
      // while kSlots later requests went by would read another request's word
      TORCH_CHECK(r.next - ticket_ <= (unsigned)kSlots, "AsyncCount: the slot was reused");
      check(hipEventSynchronize(r.events[slot_]));
      value_ = r.words[slot_];
      pending_ = false;
    }
    return value_;
  }

 private:
  static constexpr int kSlots = 64;
  struct Ring {
    int64_t* words = nullptr;
    hipEvent_t events[kSlots];
    unsigned next = 0;
  };
  static void check(hipError_t e) {
    TORCH_CHECK(e == hipSuccess, "HIP error: ", hipGetErrorString(e));
  }
  static Ring& ring() {
    static thread_local Ring* r = [] {
      Ring* x = new Ring();
      check(hipHostMalloc((void**)&x->words, kSlots * sizeof(int64_t), hipHostMallocDefault));
      for (int i = 0; i < kSlots; ++i)
        check(hipEventCreateWithFlags(&x->events[i], hipEventDisableTiming));
      return x;
    }();
    return *r;
  }
  int slot_ = -1;
  unsigned ticket_ = 0;
  bool pending_ = false;
  int64_t value_ = 0;
};

// Host copies of small offset arrays (batch pointers).  Splitting results per
// batch needs them on the host; a blocking copy at that point waits for
// everything queued on the stream.  Producers therefore announce an array as
// soon as its kernel is queued (prefetch): the copy into pinned memory travels
// while later kernels run, and values() only waits for that copy.  The last few
// arrays are remembered, keyed by tensor identity + version; an entry keeps its
// tensor alive, which is what makes that key safe.  Pinned blocks are reused
// and live until the process ends.
class OffsetMirror {
 public:
  static void prefetch(const torch::Tensor& offsets) { (void)entry_for(offsets); }
  // For a kernel that stores the array to the host itself: the pinned block it
  // should write to (as many entries as `offsets` has), and arm() once that
  // kernel is queued.
  static int64_t* reserve(const torch::Tensor& offsets) {
    return entry_for(offsets, /*copy=*/false).pinned;
  }
  static void arm(const torch::Tensor& offsets) {
    Entry& e = entry_for(offsets, false);
    check(hipEventRecord(e.event, (hipStream_t)cur_stream()));
    e.pending = true;
  }
  static const std::vector<int64_t>& values(const torch::Tensor& offsets) {
    Entry& e = entry_for(offsets);
    if (e.pending) {
      check(hipEventSynchronize(e.event));
      e.host.assign(e.pinned, e.pinned + e.count);
      e.pending = false;
    }
    return e.host;
  }

 private:
  struct Entry {
    torch::Tensor tensor;
    int64_t version = -1, epoch = -1;
    int64_t* pinned = nullptr;
    size_t capacity = 0, count = 0;
    hipEvent_t event = nullptr;
    bool pending = false;
    std::vector<int64_t> host;
  };
  // Deep enough that an entry is reused several sampler steps after its copy was
  // queued (a step of a three-layer super-batched sampler announces about ten
  // arrays): reusing one whose copy is still pending would stall the host.
  static constexpr size_t kEntries = 64;
  static void check(hipError_t e) {
    TORCH_CHECK(e == hipSuccess, "HIP error: ", hipGetErrorString(e));
  }
  static Entry& entry_for(const torch::Tensor& offsets, bool copy = true) {
    static thread_local std::vector<Entry> ring(kEntries);
    static thread_local size_t next = 0;
    TORCH_CHECK(offsets.defined() && offsets.scalar_type() == torch::kInt64,
                "batch offsets must be an int64 tensor");
    for (Entry& e : ring)
      if (e.tensor.defined() && e.tensor.is_same(offsets) &&
          e.version == (int64_t)offsets._version() && e.epoch == cache_epoch())
        return e;
    Entry& e = ring[next++ % kEntries];
    if (e.pending) check(hipEventSynchronize(e.event));  // its copy must not land later
    e.tensor = offsets;
    e.version = offsets._version();
    e.epoch = cache_epoch();
    e.count = (size_t)offsets.numel();
    e.pending = false;
    if (!offsets.is_cuda() && copy) {
      torch::Tensor c = offsets.contiguous();
      e.host.assign(c.data_ptr<int64_t>(), c.data_ptr<int64_t>() + e.count);
      return e;
    }
    if (e.capacity < e.count) {
      if (e.pinned) check(hipHostFree(e.pinned));
      e.capacity = e.count < 1024 ? 1024 : e.count;
      check(hipHostMalloc((void**)&e.pinned, e.capacity * sizeof(int64_t), hipHostMallocDefault));
    }
    if (!e.event) check(hipEventCreateWithFlags(&e.event, hipEventDisableTiming));
    if (!copy) return e;
    torch::Tensor c = offsets.contiguous();
    hipStream_t s = (hipStream_t)cur_stream();
    if (e.count > 0)
      GS_CALL(gs_copy_i64(c.data_ptr<int64_t>(), (int64_t)e.count, e.pinned, (gs_stream_t)s));
    check(hipEventRecord(e.event, s));
    e.pending = true;
    return e;
  }
};

// The number of edges a sampling operator produced.  A plain operator copies the
// last entry of its prefix array to the host (AsyncCount).  A super-batched
// operator needs the per-batch edge pointer prefix[col_bptr] on the host anyway
// (its last entry is the same total), so it announces col_bptr through hint()
// before the call: the sampler then gathers the edge pointer at once, sends that
// one array to the host and leaves it in the hint.  One copy instead of two;
// a copy to the host costs the device about as much as a small kernel.
class EdgeCount {
 public:
  struct Hint {
    torch::Tensor col_bptr;    // set by the caller
    torch::Tensor edge_bptr;   // left by the sampler
    // also left by the sampler: for every edge the place of its column inside its
    // batch, which is the column's label in the batch's block while the batch's
    // seeds are distinct (the relabel pass then has nothing to do on that side)
    torch::Tensor col_labels;
  };
  static Hint& hint() {
    static thread_local Hint h;
    return h;
  }
  struct HintScope {
    explicit HintScope(const torch::Tensor& col_bptr) {
      hint().col_bptr = col_bptr;
      hint().edge_bptr = torch::Tensor();
      hint().col_labels = torch::Tensor();
    }
    ~HintScope() { hint() = Hint(); }
  };
  // Before the count pass: what to give it as total_mirror (null when the
  // per-batch edge pointer is sent instead).
  EdgeCount() {
    if (!hint().col_bptr.defined()) count_ = AsyncCount::mirrored();
  }
  int64_t* mirror() const { return hint().col_bptr.defined() ? nullptr : count_.mirror(); }
  // After the count pass is queued.
  void arm(const torch::Tensor& prefix) {
    Hint& h = hint();
    if (h.col_bptr.defined()) {
      edge_bptr_ = prefix.index_select(0, h.col_bptr);
      OffsetMirror::prefetch(edge_bptr_);
      h.edge_bptr = edge_bptr_;
    } else {
      count_.arm();
    }
  }
  int64_t get() {
    return edge_bptr_.defined() ? OffsetMirror::values(edge_bptr_).back() : count_.get();
  }

 private:
  torch::Tensor edge_bptr_;
  AsyncCount count_;
};

// Batch pointer arrays (int64[B + 1] offsets into a concatenation) reach the
// kernels unchecked, so one that a caller supplies is looked at on the host
// first: it must start at 0, never decrease and end at the length it splits.
// Arrays that this library's own operators produced are remembered and skip
// the check (and the device read-back it costs); a caller's array is read back
// once and then found in the mirror while it stays unchanged.
class BatchOffsets {
 public:
  // `total`: the last entry, when the producer knows it on the host; -1 when it
  // is still on its way from the device (looked up on first use).
  static void trust(const torch::Tensor& offsets, int64_t total = -1) {
    if (!offsets.defined()) return;
    Known& k = ring()[next()++ % kEntries];
    k.tensor = offsets;  // kept alive: neither its address nor its memory can be handed out again
    k.version = (int64_t)offsets._version();
    k.epoch = cache_epoch();
    k.total = total;
  }
  static void check(const torch::Tensor& offsets, int64_t total, const char* who) {
    TORCH_CHECK(offsets.defined() && offsets.scalar_type() == torch::kInt64 &&
                    offsets.dim() == 1 && offsets.numel() >= 2,
                who, ": batch offsets must be an int64 vector with at least two entries");
    if (Known* k = trusted(offsets)) {
      // a well-formed array, but it must also split a sequence of this length
      if (k->total < 0) k->total = OffsetMirror::values(offsets).back();
      TORCH_CHECK(k->total == total, who, ": batch offsets end at ", k->total,
                  " but split ", total, " elements");
      return;
    }
    const std::vector<int64_t>& p = OffsetMirror::values(offsets);
    bool ok = p.front() == 0 && p.back() == total;
    for (size_t i = 1; ok && i < p.size(); ++i) ok = p[i] >= p[i - 1];
    TORCH_CHECK(ok, who, ": batch offsets must start at 0, never decrease and end at ",
                total, " (found ", p.front(), " .. ", p.back(), ")");
    trust(offsets, total);
  }

 private:
  struct Known {
    torch::Tensor tensor;
    int64_t version = -1, epoch = -1;
    int64_t total = -1;
  };
  static constexpr size_t kEntries = 32;
  static std::vector<Known>& ring() {
    static thread_local std::vector<Known> r(kEntries);
    return r;
  }
  static size_t& next() {
    static thread_local size_t n = 0;
    return n;
  }
  static Known* trusted(const torch::Tensor& t) {
    for (Known& k : ring())
      if (k.tensor.defined() && k.tensor.is_same(t) && k.version == (int64_t)t._version() &&
          k.epoch == cache_epoch())
        return &k;
    return nullptr;
  }
};

// Outputs are sized by an upper bound (and trimmed afterwards) only up to this
// many elements; beyond it the count is awaited first.
constexpr int64_t kBoundLimit = int64_t(1) << 26;

}  // namespace gs

#endif  // GS_HOST_ABI_CALL_H_
