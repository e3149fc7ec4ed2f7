// Shared by the translation units of the ShmTensorLib module: tensor checks,
// the pinned read-back slots for data-dependent sizes, the hashmap wrapper,
// and what the operator surface (module.cc), the batch driver
// (batch_driver.cc) and the graph-replaying sampler (batch_sampler.cc) call
// across file boundaries. Host C++ only.
#pragma once
#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <exception>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <thread>
#include <tuple>
#include <unordered_map>
#include <utility>
#include <vector>

#include "shmt.h"

namespace py = pybind11;

namespace shim {

inline void check(int rc) { TORCH_CHECK(rc == SHMT_OK, shmt_last_error()); }

inline void *current_stream() {
  return static_cast<void *>(c10::hip::getCurrentHIPStream().stream());
}

inline void sync_current_stream() { c10::hip::getCurrentHIPStream().synchronize(); }

inline int id_bytes(const torch::Tensor &t, const char *name) {
  // the reference aborts with "ID can only be int32 or int64" (include/common.h:29-40)
  TORCH_CHECK(t.scalar_type() == torch::kInt32 || t.scalar_type() == torch::kInt64, name,
              ": ID can only be int32 or int64, got ", t.scalar_type());
  return static_cast<int>(t.element_size());
}

inline torch::Tensor cuda_ids(const torch::Tensor &t, const char *name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
  id_bytes(t, name);
  return t.contiguous();
}

// Address a kernel may dereference for tensor `t`: device tensors as they
// are, CPU tensors through the device alias of their pinned storage.
inline void *device_address(const torch::Tensor &t, const char *name) {
  if (t.numel() == 0) return t.data_ptr();
  if (t.is_cuda()) return t.data_ptr();
  void *dev = nullptr;
  int rc = shmt_host_devptr(t.data_ptr(), &dev);
  TORCH_CHECK(rc == SHMT_OK, name,
              " is a CPU tensor whose memory the GPU cannot address; call pin_memory() on it "
              "first (",
              shmt_last_error(), ")");
  return dev;
}

// Totals whose value only the GPU knows (nnz of a sample, number of unique
// ids) come back through int64 slots in pinned host memory. The host marks a
// slot pending before the launches and the kernel overwrites it with the
// total (always >= 0) in one store that bypasses the caches; the host then watches
// the slot instead of synchronising the stream, so it learns the total as
// soon as the kernel that computes it has run, while later kernels of the
// same operator are still queued or running. If the value does not show up
// within the spin budget (a failed launch, a hung device) the wait falls back
// to a stream synchronisation, which surfaces the error. One more pinned word
// mirrors the GPU's error word (shmt_async_error_mirror): a kernel that gave
// up a bounded wait sets it, and every wait here looks at it, so the failure
// surfaces as an exception at the next size read-back at no cost otherwise.
class Readback {
 public:
  static constexpr int kSlots = 4096;  // a ring: more than all operators together keep pending at once
  struct Slot {
    volatile int64_t *host;
    int64_t *dev;
  };

  Slot acquire() {
    std::lock_guard<std::mutex> lock(mutex_);
    if (!host_.defined()) {
      host_ = torch::zeros({kSlots + 1}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
      void *d = nullptr;
      check(shmt_host_devptr(host_.data_ptr(), &d));
      dev_ = static_cast<int64_t *>(d);
      gave_up_ = reinterpret_cast<volatile uint32_t *>(host_.data_ptr<int64_t>() + kSlots);
    }
    const int device = static_cast<int>(c10::hip::current_device());
    if (device >= 0 && device < 64 && !(mirrored_ >> device & 1)) {  // once per GPU this process launches on
      check(shmt_async_error_mirror(const_cast<uint32_t *>(gave_up_), dev_ + kSlots));
      mirrored_ |= 1ull << device;
    }
    const uint32_t i = next_;
    next_ = (next_ + 1) % kSlots;  // stays in [0, kSlots): nothing counts up without bound
    Slot s{host_.data_ptr<int64_t>() + i, dev_ + i};
    *s.host = kPending;
    std::atomic_thread_fence(std::memory_order_seq_cst);
    return s;
  }

  static int64_t wait(const Slot &s) {
    const auto t0 = std::chrono::steady_clock::now();
    for (uint64_t spins = 0;; ++spins) {
      const int64_t v = *s.host;
      if (v != kPending) {
        if (gave_up_ && *gave_up_ != 0) report_gave_up();
        return v;
      }
      if ((spins & 1023) == 1023 &&
          std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(kSpinBudgetMs))
        break;
      __builtin_ia32_pause();
    }
    sync_current_stream();
    const int64_t v = *s.host;
    if (v == kPending) {
      int gave_up = 0;  // a kernel that gave up a bounded wait says so in the GPU's error word
      const bool known = shmt_async_error(&gave_up) == SHMT_OK && gave_up != 0;
      TORCH_CHECK(false, known ? shmt_last_error() : "the GPU did not report a result size (kernel failed?)");
    }
    if (gave_up_ && *gave_up_ != 0) report_gave_up();
    return v;
  }

 private:
  // Reads and clears the GPU's error word (which also clears the mirror) and raises what it says.
  static void report_gave_up() {
    int code = 0;
    check(shmt_async_error(&code));
    TORCH_CHECK(code == 0, shmt_last_error());
  }

  static constexpr int64_t kPending = INT64_MIN;
  static constexpr int kSpinBudgetMs = 200;
  std::mutex mutex_;  // operators may run on several host threads (sample_blocks)
  torch::Tensor host_;
  int64_t *dev_ = nullptr;
  static inline volatile uint32_t *gave_up_ = nullptr;  // the mirror word, behind the slots
  uint64_t mirrored_ = 0;                 // bit d: the mirror is registered with GPU d
  uint32_t next_ = 0;
};

inline Readback &readback() {
  static Readback r;
  return r;
}

inline torch::Tensor device_bytes(int64_t nbytes) {
  return torch::empty({nbytes > 0 ? nbytes : 1},
                      torch::TensorOptions().dtype(torch::kUInt8).device(torch::kCUDA));
}

// ---- hashmap ---------------------------------------------------------------

class StaticHashmap {
 public:
  // `layout`: "auto" looks at the keys and builds the cheapest form that answers like the general table
  // (an id range, a rank bitmap, a direct table, narrow bucket slots); "buckets" builds the general bucket
  // table in the slot format the dtypes call for, whatever the keys look like (what cuco::static_map holds
  // in the reference, include/cuco_hashmap.cuh:57-77).
  StaticHashmap(torch::Tensor keys, torch::Tensor values, double load_factor, const std::string &layout_choice = "auto") {
    TORCH_CHECK(keys.is_cuda(), "keys must be a CUDA tensor");
    TORCH_CHECK(values.is_cuda(), "values must be a CUDA tensor");
    TORCH_CHECK(layout_choice == "auto" || layout_choice == "buckets", "layout must be \"auto\" or \"buckets\"");
    key_type_ = keys.scalar_type();
    value_type_ = values.scalar_type();
    const int kb = id_bytes(keys, "keys"), vb = id_bytes(values, "values");
    TORCH_CHECK(keys.numel() == values.numel(), "keys and values must have the same length");
    TORCH_CHECK(load_factor > 0.0 && load_factor <= 1.0, "load_factor must be in (0, 1]");
    keys = keys.contiguous();
    values = values.contiguous();
    const int64_t n = keys.numel();
    capacity_ = shmt_hashmap_capacity(n, load_factor);
    if (layout_choice == "buckets") {
      const int64_t bytes = shmt_hashmap_table_bytes(n, load_factor, kb, vb);
      table_ = device_bytes(bytes);
      memory_usage_ = bytes;
      kind_ = SHMT_MAP_BUCKETS;
      check(shmt_hashmap_create(&handle_, keys.data_ptr(), values.data_ptr(), n, kb, vb, load_factor,
                                table_.data_ptr(), bytes, current_stream()));
      return;
    }
    // the layout follows from the keys (dense id range, 32-bit ids ...): look first, then allocate what it needs
    shmt_hashmap_layout layout;
    {
      const int64_t scratch_bytes = shmt_hashmap_plan_scratch_bytes(n);
      torch::Tensor scratch = device_bytes(scratch_bytes);
      check(shmt_hashmap_plan(keys.data_ptr(), values.data_ptr(), n, kb, vb, load_factor, scratch.data_ptr(),
                              scratch_bytes, &layout, current_stream()));
    }
    table_ = device_bytes(layout.table_bytes);
    memory_usage_ = layout.kind == SHMT_MAP_RANGE ? 0 : layout.table_bytes;
    kind_ = layout.kind;
    check(shmt_hashmap_create_planned(&handle_, &layout, keys.data_ptr(), values.data_ptr(), n, kb, vb,
                                      load_factor, table_.data_ptr(), layout.table_bytes, current_stream()));
  }
  ~StaticHashmap() { shmt_hashmap_destroy(handle_); }
  StaticHashmap(const StaticHashmap &) = delete;
  StaticHashmap &operator=(const StaticHashmap &) = delete;

  torch::Tensor query(torch::Tensor requests) {
    TORCH_CHECK(requests.is_cuda(), "requests must be a CUDA tensor");
    if (requests.scalar_type() != torch::kInt32 && requests.scalar_type() != torch::kInt64)
      requests = requests.to(key_type_);  // src/cuco_hashmap.cu:29
    requests = requests.contiguous();
    torch::Tensor result = torch::empty_like(requests, requests.options().dtype(value_type_));
    check(shmt_hashmap_query(handle_, requests.data_ptr(), static_cast<int>(requests.element_size()),
                             requests.numel(), result.data_ptr(), current_stream()));
    return result;
  }
  int64_t capacity() const { return capacity_; }
  int64_t memory_usage() const { return memory_usage_; }
  // "buckets", "direct", "range" or "rank": the layout the constructor chose for these keys
  std::string layout() const {
    return kind_ == SHMT_MAP_RANGE ? "range" : kind_ == SHMT_MAP_DIRECT ? "direct" : kind_ == SHMT_MAP_RANK ? "rank" : "buckets";
  }
  const shmt_hashmap_t *handle() const { return handle_; }

 private:
  shmt_hashmap_t *handle_ = nullptr;
  torch::Tensor table_;
  torch::ScalarType key_type_, value_type_;
  int64_t capacity_ = 0, memory_usage_ = 0;
  int kind_ = SHMT_MAP_BUCKETS;
};

constexpr uint64_t kDefaultSeed = 7777;  // src/cache_graph_sampling.cu:204,407
// Buffers sized for a bound instead of the true, data-dependent size save a host wait but stay allocated
// as long as any result that views them lives. Budgets: the sampler's output is sized for S * num_picks up
// to kEagerOutputBytes (beyond it: plan, read the true size, allocate exactly); a hop is queued as one fused
// launch sequence while all its buffers (results, relabel input and table) stay within kHopBufferBytes
// (beyond it: the two operators one after the other, exact allocations).
constexpr int64_t kEagerOutputBytes = 256ll << 20;
constexpr int64_t kHopBufferBytes = 2ll << 30;

// Device memory a fused hop of S seeds with k picks holds: four results, the relabel input, plan and scratch.
inline int64_t hop_buffer_bytes(int64_t S, int64_t k, int ptr_bytes, int idx_bytes, int elem_bytes) {
  if (S <= 0 || k <= 0 || k > (int64_t{1} << 31) / S) return INT64_MAX;
  const int64_t bound = S * k, n_max = S + bound;
  return (S + 1) * ptr_bytes + bound * (idx_bytes + elem_bytes) + 3 * n_max * elem_bytes +
         shmt_sample_plan_bytes(S) + shmt_relabel_scratch_bytes(n_max);
}

// ---- operator surface (module.cc) used by the batch driver and the sampler ----
struct RowShape {
  int64_t row_bytes;
  std::vector<int64_t> out_sizes;
};
RowShape row_shape(const torch::Tensor &data, int64_t numel);
void check_tables(const torch::Tensor &uva_data, const torch::Tensor *gpu_data);
torch::Tensor fetch_impl(const torch::Tensor &uva_data, const torch::Tensor *gpu_data, torch::Tensor indices,
                         const StaticHashmap *hashmap, const torch::Tensor *mask);
std::tuple<torch::Tensor, torch::Tensor> sample_impl(const torch::Tensor &indptr, const torch::Tensor &indices,
                                                     const torch::Tensor *gpu_indptr,
                                                     const torch::Tensor *gpu_indices, const StaticHashmap *hashmap,
                                                     torch::Tensor seeds, int64_t num_picks, bool replace,
                                                     std::optional<int64_t> seed, int64_t stream_id);
std::tuple<torch::Tensor, std::vector<torch::Tensor>> tensor_relabel(std::vector<torch::Tensor> tensors);

// csr_[cache_]sampling followed by tensor_relabel([seeds, sub_indices]) returns,
// with relabel_indices = the labels of the sub_indices part.
// With coordinate output (create_block_from_coo, python/shmtensor/sampling.py:21-27) a fifth
// tensor follows: coo_dst[e] = position of the seed that sampled id e belongs to, so that
// (row, col) = (relabel_indices, coo_dst) are the source and destination of every edge of the block.
struct HopResult {
  torch::Tensor sub_indptr, sub_indices, unique, relabel_indices;
  torch::Tensor coo_dst;  // defined only when the coordinate form was asked for
};

struct CsrArgs {
  torch::Tensor indptr, indices;
  std::optional<torch::Tensor> gpu_indptr, gpu_indices;
  StaticHashmap *hashmap;
  bool coo = false;  // hops also return the destination position of every sampled id
  // what the kernels dereference for indptr / indices (translated once per call, not once per hop)
  void *indptr_dev = nullptr, *indices_dev = nullptr;
  bool cached() const { return hashmap != nullptr; }
};

inline void check_csr(CsrArgs &g) {
  TORCH_CHECK(!g.cached() || (g.gpu_indptr.has_value() && g.gpu_indices.has_value()),
              "sample_hop: a hashmap needs gpu_indptr and gpu_indices");
  id_bytes(g.indptr, "indptr");
  id_bytes(g.indices, "indices");
  TORCH_CHECK(g.indptr.is_contiguous() && g.indices.is_contiguous(), "CSR arrays must be contiguous");
  if (g.cached()) {
    TORCH_CHECK(g.gpu_indptr->is_cuda() && g.gpu_indices->is_cuda() && g.gpu_indptr->is_contiguous() &&
                    g.gpu_indices->is_contiguous(),
                "gpu_indptr and gpu_indices must be contiguous CUDA tensors");
    TORCH_CHECK(g.gpu_indptr->scalar_type() == g.indptr.scalar_type() &&
                    g.gpu_indices->scalar_type() == g.indices.scalar_type(),
                "cached CSR must have the dtypes of the full CSR");
  }
  g.indptr_dev = device_address(g.indptr, "indptr");
  g.indices_dev = device_address(g.indices, "indices");
}


// ---- batch driver (batch_driver.cc) ----
HopResult sample_hop(torch::Tensor indptr, torch::Tensor indices, std::optional<torch::Tensor> gpu_indptr,
                     std::optional<torch::Tensor> gpu_indices, StaticHashmap *hashmap, torch::Tensor seeds,
                     int64_t num_picks, bool replace, std::optional<int64_t> seed, int64_t stream_id, bool coo);
std::vector<std::vector<HopResult>> sample_blocks(
    torch::Tensor indptr, torch::Tensor indices, std::optional<torch::Tensor> gpu_indptr,
    std::optional<torch::Tensor> gpu_indices, StaticHashmap *hashmap, std::vector<torch::Tensor> seeds,
    std::vector<int64_t> num_picks, bool replace, std::optional<std::vector<int64_t>> seeds_rng,
    int64_t max_in_flight, bool coo);
std::vector<std::pair<std::vector<HopResult>, torch::Tensor>> sample_blocks_fetch(
    torch::Tensor indptr, torch::Tensor indices, std::optional<torch::Tensor> gpu_indptr,
    std::optional<torch::Tensor> gpu_indices, StaticHashmap *hashmap, std::vector<torch::Tensor> seeds,
    std::vector<int64_t> num_picks, bool replace, torch::Tensor uva_data, std::optional<torch::Tensor> gpu_data,
    StaticHashmap *data_hashmap, std::optional<std::vector<int64_t>> seeds_rng, int64_t max_in_flight,
    std::optional<int64_t> max_rows, bool coo);

// All hops of one batch on the current stream, chained on the device where their bounds allow
// (`g` already checked by check_csr).
std::vector<HopResult> sample_batch(const CsrArgs &g, torch::Tensor seeds, const std::vector<int64_t> &num_picks,
                                    bool replace, std::optional<int64_t> seed);

// ---- graph-replaying sampler (batch_sampler.cc) ----
void register_batch_sampler(py::module &m);

}  // namespace shim

// host tensor providers (host_tensors.cc)
void register_host_tensors(py::module &m);

namespace pybind11 {
namespace detail {
// A hop goes to Python as the tuple (sub_indptr, sub_indices, unique, relabel_indices), with the
// destination positions as a fifth member when the coordinate form was asked for.
template <>
struct type_caster<shim::HopResult> {
  PYBIND11_TYPE_CASTER(shim::HopResult, const_name("Tuple[Tensor, ...]"));
  bool load(handle, bool) { return false; }
  static handle cast(const shim::HopResult &h, return_value_policy, handle) {
    if (h.coo_dst.defined())
      return py::make_tuple(h.sub_indptr, h.sub_indices, h.unique, h.relabel_indices, h.coo_dst).release();
    return py::make_tuple(h.sub_indptr, h.sub_indices, h.unique, h.relabel_indices).release();
  }
};
}  // namespace detail
}  // namespace pybind11
