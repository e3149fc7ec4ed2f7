// ShmTensorLib: the Python operator surface of the GPU-cache hot path, with
// the names, argument names, defaults and return structure of the reference
// module (src/pybind.cc:16-65 in the ShmTensor tree). Host C++ only: every
// operator validates its tensors, allocates outputs and scratch from torch's
// caching allocator and calls the C ABI of libshmt.so (include/shmt.h) on
// torch's current HIP stream. Failures raise RuntimeError; nothing exits.
#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <cstdint>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
#include <exception>
#include <optional>
#include <thread>
#include <unordered_map>
#include <vector>

#include "shmt.h"

namespace py = pybind11;

namespace {

void check(int rc) { TORCH_CHECK(rc == SHMT_OK, shmt_last_error()); }

void *current_stream() {
  return static_cast<void *>(c10::hip::getCurrentHIPStream().stream());
}

void sync_current_stream() { c10::hip::getCurrentHIPStream().synchronize(); }

int id_bytes(const torch::Tensor &t, const char *name) {
  // the reference aborts with "ID can only be int32 or int64" (include/common.h:29-40)
  TORCH_CHECK(t.scalar_type() == torch::kInt32 || t.scalar_type() == torch::kInt64, name,
              ": ID can only be int32 or int64, got ", t.scalar_type());
  return static_cast<int>(t.element_size());
}

torch::Tensor cuda_ids(const torch::Tensor &t, const char *name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
  id_bytes(t, name);
  return t.contiguous();
}

// Address a kernel may dereference for tensor `t`: device tensors as they
// are, CPU tensors through the device alias of their pinned storage.
void *device_address(const torch::Tensor &t, const char *name) {
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
// to a stream synchronisation, which surfaces the error.
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
      host_ = torch::zeros({kSlots}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
      void *d = nullptr;
      check(shmt_host_devptr(host_.data_ptr(), &d));
      dev_ = static_cast<int64_t *>(d);
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
      if (v != kPending) return v;
      if ((spins & 1023) == 1023 &&
          std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(kSpinBudgetMs))
        break;
      __builtin_ia32_pause();
    }
    sync_current_stream();
    const int64_t v = *s.host;
    TORCH_CHECK(v != kPending, "the GPU did not report a result size (kernel failed?)");
    return v;
  }

 private:
  static constexpr int64_t kPending = INT64_MIN;
  static constexpr int kSpinBudgetMs = 200;
  std::mutex mutex_;  // operators may run on several host threads (sample_blocks)
  torch::Tensor host_;
  int64_t *dev_ = nullptr;
  uint32_t next_ = 0;
};

Readback &readback() {
  static Readback r;
  return r;
}

torch::Tensor device_bytes(int64_t nbytes) {
  return torch::empty({nbytes > 0 ? nbytes : 1},
                      torch::TensorOptions().dtype(torch::kUInt8).device(torch::kCUDA));
}

// ---- hashmap ---------------------------------------------------------------

class StaticHashmap {
 public:
  StaticHashmap(torch::Tensor keys, torch::Tensor values, double load_factor) {
    TORCH_CHECK(keys.is_cuda(), "keys must be a CUDA tensor");
    TORCH_CHECK(values.is_cuda(), "values must be a CUDA tensor");
    key_type_ = keys.scalar_type();
    value_type_ = values.scalar_type();
    const int kb = id_bytes(keys, "keys"), vb = id_bytes(values, "values");
    TORCH_CHECK(keys.numel() == values.numel(), "keys and values must have the same length");
    TORCH_CHECK(load_factor > 0.0 && load_factor <= 1.0, "load_factor must be in (0, 1]");
    keys = keys.contiguous();
    values = values.contiguous();
    const int64_t n = keys.numel();
    capacity_ = shmt_hashmap_capacity(n, load_factor);
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
  // "buckets", "direct" or "range": the layout the constructor chose for these keys
  std::string layout() const { return kind_ == SHMT_MAP_RANGE ? "range" : kind_ == SHMT_MAP_DIRECT ? "direct" : "buckets"; }
  const shmt_hashmap_t *handle() const { return handle_; }

 private:
  shmt_hashmap_t *handle_ = nullptr;
  torch::Tensor table_;
  torch::ScalarType key_type_, value_type_;
  int64_t capacity_ = 0, memory_usage_ = 0;
  int kind_ = SHMT_MAP_BUCKETS;
};

// ---- pin / unpin -----------------------------------------------------------

std::mutex g_pin_mutex;
std::unordered_map<void *, int64_t> g_registered;  // ranges registered in place by pin_memory

// Registering memory that already exists (hipHostRegister) is refused by some
// drivers, and a refused call can leave its error for the next HIP call to
// report. It is therefore only tried on request: set_host_register(true) or
// SHMT_HOST_REGISTER=1 in the environment.
std::atomic<int> g_host_register{-1};  // -1: not decided yet (read the environment)

bool host_register_enabled() {
  int v = g_host_register.load();
  if (v < 0) {
    const char *e = std::getenv("SHMT_HOST_REGISTER");
    v = (e != nullptr && e[0] != '\0' && e[0] != '0') ? 1 : 0;
    g_host_register.store(v);
  }
  return v == 1;
}

void set_host_register(bool on) { g_host_register.store(on ? 1 : 0); }

// PinMemory, src/cache_feature_fetch.cu:6-9: make a CPU tensor's memory
// addressable by kernels. With in-place registration enabled (see above) the
// memory is registered where it lies, as in the reference. Otherwise the
// tensor's STORAGE is re-homed: its bytes move into newly allocated pinned
// memory and the storage object points there afterwards, so the tensor and
// every other torch tensor that shares the storage (views, slices, aliases)
// keep seeing one memory, and later GPU writes (uva_set) reach all of them.
// What cannot follow is memory that torch does not own: a storage that wraps
// a numpy array, a shared-memory or file mapping. Re-homing such a storage
// cuts the tie to that memory, which is reported with a warning.
void pin_memory(torch::Tensor &data) {
  TORCH_CHECK(!data.is_cuda(), "data must be a CPU tensor");
  if (data.numel() == 0) return;
  TORCH_CHECK(data.is_contiguous(), "data must be contiguous");
  void *dev = nullptr;
  if (shmt_host_devptr(data.data_ptr(), &dev) == SHMT_OK) return;  // already addressable
  if (host_register_enabled() &&
      shmt_host_register(data.data_ptr(), static_cast<int64_t>(data.nbytes())) == SHMT_OK) {
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    g_registered[data.data_ptr()] = static_cast<int64_t>(data.nbytes());
    return;
  }
  c10::Storage storage = data.storage();
  const size_t nbytes = storage.nbytes();
  TORCH_CHECK(nbytes > 0 && storage.data() != nullptr, "pin_memory: tensor has no memory");
  if (!storage.resizable()) {
    // storages that wrap foreign memory (from_numpy, from_blob) are the non-resizable ones
    if (PyErr_WarnEx(PyExc_UserWarning,
                     "pin_memory: the tensor's memory is not owned by torch (a numpy array, a shared-memory or "
                     "file mapping) and existing memory is not registered in place with the current setting, so "
                     "its contents were copied into new pinned memory: the tensor now lives there and no longer "
                     "aliases the original buffer (GPU writes will not reach it). Allocate the data pinned in "
                     "the first place, or enable in-place registration with set_host_register(True).",
                     1) < 0)
      throw py::error_already_set();
  }
  at::Allocator *pinned = at::globalContext().getPinnedMemoryAllocator(c10::kCUDA);
  at::DataPtr fresh = pinned->allocate(nbytes);
  std::memcpy(fresh.get(), storage.data(), nbytes);
  // the old memory is released here (or, for foreign memory, handed back to its owner)
  storage.set_data_ptr_noswap(std::move(fresh));
}

// UnpinMemory, src/cache_feature_fetch.cu:11-13.
void unpin_memory(torch::Tensor &data) {
  if (data.numel() == 0) return;
  std::lock_guard<std::mutex> lock(g_pin_mutex);
  auto it = g_registered.find(data.data_ptr());
  if (it == g_registered.end()) return;  // pinned at allocation: released with the tensor
  g_registered.erase(it);
  check(shmt_host_unregister(data.data_ptr()));
}

// ---- fetch / set -----------------------------------------------------------

struct RowShape {
  int64_t row_bytes;
  std::vector<int64_t> out_sizes;
};

// Output shape rules of src/cache_feature_fetch.cu:137-163: 1-D data gives
// [numel]; otherwise [numel, *data.shape[1:]].
RowShape row_shape(const torch::Tensor &data, int64_t numel) {
  RowShape r;
  r.out_sizes.push_back(numel);
  int64_t dim = 1;
  for (int64_t i = 1; i < data.dim(); ++i) {
    dim *= data.size(i);
    r.out_sizes.push_back(data.size(i));
  }
  r.row_bytes = dim * static_cast<int64_t>(data.element_size());
  return r;
}

void check_tables(const torch::Tensor &uva_data, const torch::Tensor *gpu_data) {
  TORCH_CHECK(uva_data.dim() >= 1, "data must have at least one dimension");
  TORCH_CHECK(uva_data.is_contiguous(), "data must be contiguous");
  if (gpu_data) {
    TORCH_CHECK(gpu_data->is_cuda(), "gpu_data must be a CUDA tensor");
    TORCH_CHECK(gpu_data->is_contiguous(), "gpu_data must be contiguous");
    TORCH_CHECK(gpu_data->scalar_type() == uva_data.scalar_type(),
                "uva_data and gpu_data must have the same dtype");
    TORCH_CHECK(row_shape(*gpu_data, 0).row_bytes == row_shape(uva_data, 0).row_bytes,
                "uva_data and gpu_data must have the same row shape");
  }
}

torch::Tensor fetch_impl(const torch::Tensor &uva_data, const torch::Tensor *gpu_data,
                         torch::Tensor indices, const StaticHashmap *map,
                         const torch::Tensor *mask) {
  check_tables(uva_data, gpu_data);
  indices = cuda_ids(indices, "indices");
  const int64_t numel = indices.numel();
  const RowShape rs = row_shape(uva_data, numel);
  torch::Tensor output = torch::empty(rs.out_sizes, uva_data.options().device(torch::kCUDA));
  torch::Tensor m;
  if (mask) {
    m = cuda_ids(*mask, "mask");
    TORCH_CHECK(m.numel() == numel, "mask and indices must have the same length");
  }
  if (numel == 0 || rs.row_bytes == 0) return output;
  // an empty cache tensor has no storage; with a mask the C ABI wants a non-null table, and any
  // addressable pointer will do because no mask entry may point into an empty cache
  void *cache_ptr = nullptr;
  if (gpu_data) cache_ptr = gpu_data->numel() > 0 ? gpu_data->data_ptr() : output.data_ptr();
  check(shmt_fetch(device_address(uva_data, "uva_data"), cache_ptr,
                   indices.data_ptr(), static_cast<int>(indices.element_size()),
                   map ? map->handle() : nullptr, mask ? m.data_ptr() : nullptr,
                   mask ? static_cast<int>(m.element_size()) : 0, output.data_ptr(), numel,
                   rs.row_bytes, current_stream()));
  return output;
}

void set_impl(torch::Tensor &uva_data, torch::Tensor *gpu_data, torch::Tensor indices,
              torch::Tensor update, const StaticHashmap *map, const torch::Tensor *mask,
              bool write_through = false) {
  check_tables(uva_data, gpu_data);
  indices = cuda_ids(indices, "indices");
  const int64_t numel = indices.numel();
  const RowShape rs = row_shape(uva_data, numel);
  TORCH_CHECK(update.is_cuda(), "update must be a CUDA tensor");
  TORCH_CHECK(update.scalar_type() == uva_data.scalar_type(),
              "update must have the dtype of the data");
  update = update.contiguous();
  TORCH_CHECK(update.numel() * static_cast<int64_t>(update.element_size()) == numel * rs.row_bytes,
              "update must hold one row per index");
  torch::Tensor m;
  if (mask) {
    m = cuda_ids(*mask, "mask");
    TORCH_CHECK(m.numel() == numel, "mask and indices must have the same length");
  }
  if (numel == 0 || rs.row_bytes == 0) return;
  void *cache_ptr = nullptr;
  if (gpu_data) cache_ptr = gpu_data->numel() > 0 ? gpu_data->data_ptr() : update.data_ptr();
  const auto entry = write_through ? shmt_set_through : shmt_set;
  check(entry(device_address(uva_data, "uva_data"), cache_ptr, indices.data_ptr(),
              static_cast<int>(indices.element_size()), map ? map->handle() : nullptr,
              mask ? m.data_ptr() : nullptr, mask ? static_cast<int>(m.element_size()) : 0,
              update.data_ptr(), numel, rs.row_bytes, current_stream()));
}

torch::Tensor uva_fetch(torch::Tensor &data, torch::Tensor &indices) {
  return fetch_impl(data, nullptr, indices, nullptr, nullptr);
}
torch::Tensor cache_fetch(torch::Tensor uva_data, torch::Tensor gpu_data, torch::Tensor indices,
                          StaticHashmap &hashmap) {
  return fetch_impl(uva_data, &gpu_data, indices, &hashmap, nullptr);
}
torch::Tensor cache_fetch_with_mask(torch::Tensor uva_data, torch::Tensor gpu_data,
                                    torch::Tensor indices, torch::Tensor mask) {
  return fetch_impl(uva_data, &gpu_data, indices, nullptr, &mask);
}
void uva_set(torch::Tensor &data, torch::Tensor &indices, torch::Tensor &update) {
  set_impl(data, nullptr, indices, update, nullptr, nullptr);
}
void cache_set(torch::Tensor uva_data, torch::Tensor gpu_data, torch::Tensor indices,
               torch::Tensor update, StaticHashmap &hashmap, bool write_through) {
  set_impl(uva_data, &gpu_data, indices, update, &hashmap, nullptr, write_through);
}
void cache_set_with_mask(torch::Tensor uva_data, torch::Tensor gpu_data, torch::Tensor indices,
                         torch::Tensor update, torch::Tensor mask, bool write_through) {
  set_impl(uva_data, &gpu_data, indices, update, nullptr, &mask, write_through);
}

// ---- scan --------------------------------------------------------------------

// thrust_scan, src/thrust_scan.cu:9-18: in-place inclusive sum over int32.
void thrust_scan(torch::Tensor tensor) {
  TORCH_CHECK(tensor.scalar_type() == torch::kInt32, "thrust_scan expects an int32 tensor");
  TORCH_CHECK(tensor.is_contiguous(), "tensor must be contiguous");
  const int64_t n = tensor.numel();
  if (n == 0) return;
  const int64_t tmp_bytes = shmt_scan_tmp_bytes(n);
  torch::Tensor tmp = device_bytes(tmp_bytes);
  check(shmt_inclusive_scan_i32(device_address(tensor, "tensor"), n, tmp.data_ptr(), tmp_bytes,
                                current_stream()));
}

// ---- sampling ------------------------------------------------------------------

constexpr uint64_t kDefaultSeed = 7777;  // src/cache_graph_sampling.cu:204,407
constexpr int64_t kEagerOutputLimit = 1ll << 27;

std::tuple<torch::Tensor, torch::Tensor> sample_impl(const torch::Tensor &indptr,
                                                     const torch::Tensor &indices,
                                                     const torch::Tensor *gpu_indptr,
                                                     const torch::Tensor *gpu_indices,
                                                     const StaticHashmap *map, torch::Tensor seeds,
                                                     int64_t num_picks, bool replace,
                                                     std::optional<int64_t> seed,
                                                     int64_t stream_id) {
  const int pb = id_bytes(indptr, "indptr"), ib = id_bytes(indices, "indices");
  TORCH_CHECK(indptr.is_contiguous() && indices.is_contiguous(), "CSR arrays must be contiguous");
  TORCH_CHECK(num_picks >= 0, "num_picks must be >= 0");
  seeds = cuda_ids(seeds, "seeds");
  if (map) {
    TORCH_CHECK(gpu_indptr->is_cuda() && gpu_indices->is_cuda(),
                "gpu_indptr and gpu_indices must be CUDA tensors");
    TORCH_CHECK(gpu_indptr->scalar_type() == indptr.scalar_type() &&
                    gpu_indices->scalar_type() == indices.scalar_type(),
                "cached CSR must have the dtypes of the full CSR");
    TORCH_CHECK(gpu_indptr->is_contiguous() && gpu_indices->is_contiguous(),
                "cached CSR arrays must be contiguous");
  }
  const int64_t S = seeds.numel();
  const auto dev = torch::kCUDA;
  torch::Tensor sub_indptr = torch::empty({S + 1}, indptr.options().device(dev));
  const int64_t plan_bytes = shmt_sample_plan_bytes(S);
  torch::Tensor plan = device_bytes(plan_bytes);
  const Readback::Slot total = readback().acquire();
  void *stream = current_stream();
  void *const indptr_dev = device_address(indptr, "indptr");
  void *const indices_dev = device_address(indices, "indices");
  const int sb = static_cast<int>(seeds.element_size());
  const uint64_t rng_seed = static_cast<uint64_t>(seed.value_or(kDefaultSeed));
  // Output size is data dependent. When the bound S*k is modest, sample into a
  // buffer of that size and pick up the total afterwards (plan and pick are
  // queued back to back, two launches); otherwise plan, wait for the total,
  // allocate exactly, pick.
  const bool eager = S > 0 && num_picks > 0 && num_picks <= kEagerOutputLimit / S;
  torch::Tensor sub_indices;
  if (eager) {
    sub_indices = torch::empty({S * num_picks}, indices.options().device(dev));
    check(shmt_sample(indptr_dev, pb, indices_dev, ib, map ? gpu_indptr->data_ptr() : nullptr,
                      map ? gpu_indices->data_ptr() : nullptr, map ? map->handle() : nullptr, seeds.data_ptr(),
                      sb, S, num_picks, replace, rng_seed, static_cast<uint32_t>(stream_id),
                      sub_indptr.data_ptr(), sub_indices.data_ptr(), plan.data_ptr(), plan_bytes, total.dev,
                      stream));
    sub_indices = sub_indices.narrow(0, 0, Readback::wait(total));
  } else {
    check(shmt_sample_plan(indptr_dev, pb, map ? gpu_indptr->data_ptr() : nullptr,
                           map ? map->handle() : nullptr, seeds.data_ptr(), sb, S, num_picks, replace,
                           sub_indptr.data_ptr(), plan.data_ptr(), plan_bytes, total.dev, stream));
    sub_indices = torch::empty({Readback::wait(total)}, indices.options().device(dev));
    check(shmt_sample_pick(indices_dev, map ? gpu_indices->data_ptr() : nullptr, ib, seeds.data_ptr(), sb, S,
                           num_picks, replace, sub_indptr.data_ptr(), pb, plan.data_ptr(),
                           sub_indices.data_ptr(), rng_seed, static_cast<uint32_t>(stream_id), stream));
  }
  return std::make_tuple(sub_indptr, sub_indices);
}

std::tuple<torch::Tensor, torch::Tensor> csr_sampling(torch::Tensor indptr, torch::Tensor indices,
                                                      torch::Tensor seeds, int64_t num_picks,
                                                      bool replace, std::optional<int64_t> seed,
                                                      int64_t stream_id) {
  return sample_impl(indptr, indices, nullptr, nullptr, nullptr, seeds, num_picks, replace, seed,
                     stream_id);
}

std::tuple<torch::Tensor, torch::Tensor> csr_cache_sampling(
    torch::Tensor uva_indptr, torch::Tensor uva_indices, torch::Tensor gpu_indptr,
    torch::Tensor gpu_indices, StaticHashmap &hashmap, torch::Tensor seeds, int64_t num_picks,
    bool replace, std::optional<int64_t> seed, int64_t stream_id) {
  return sample_impl(uva_indptr, uva_indices, &gpu_indptr, &gpu_indices, &hashmap, seeds, num_picks,
                     replace, seed, stream_id);
}

// CreateCacheCSR, src/cache_graph_sampling.cu:455-492.
std::tuple<torch::Tensor, torch::Tensor> create_subcsr(torch::Tensor uva_indptr,
                                                       torch::Tensor uva_indices,
                                                       torch::Tensor seeds) {
  const int pb = id_bytes(uva_indptr, "uva_indptr"), ib = id_bytes(uva_indices, "uva_indices");
  TORCH_CHECK(uva_indptr.is_contiguous() && uva_indices.is_contiguous(),
              "CSR arrays must be contiguous");
  seeds = cuda_ids(seeds, "seeds");
  const int64_t C = seeds.numel();
  torch::Tensor gpu_indptr = torch::empty({C + 1}, uva_indptr.options().device(torch::kCUDA));
  const int64_t tmp_bytes = shmt_scan_tmp_bytes(C + 1);
  torch::Tensor tmp = device_bytes(tmp_bytes);
  const Readback::Slot total = readback().acquire();
  void *stream = current_stream();
  void *indptr_dev = device_address(uva_indptr, "uva_indptr");
  check(shmt_subcsr_plan(indptr_dev, pb, seeds.data_ptr(), static_cast<int>(seeds.element_size()), C,
                         gpu_indptr.data_ptr(), tmp.data_ptr(), tmp_bytes, total.dev, stream));
  const int64_t nnz = Readback::wait(total);
  torch::Tensor gpu_indices = torch::empty({nnz}, uva_indices.options().device(torch::kCUDA));
  check(shmt_subcsr_copy(indptr_dev, device_address(uva_indices, "uva_indices"), pb, ib,
                         seeds.data_ptr(), static_cast<int>(seeds.element_size()), C,
                         gpu_indptr.data_ptr(), nnz, gpu_indices.data_ptr(), stream));
  return std::make_tuple(gpu_indptr, gpu_indices);
}

// ---- relabel ---------------------------------------------------------------------

// TensorRelabel, src/tensor_relabel.cu:125-209.
std::tuple<torch::Tensor, std::vector<torch::Tensor>> tensor_relabel(
    std::vector<torch::Tensor> tensors) {
  TORCH_CHECK(!tensors.empty(), "tensor_relabel needs at least one tensor");
  std::vector<int64_t> split_sizes;
  for (auto &t : tensors) {
    TORCH_CHECK(t.is_cuda(), "tensor_relabel expects CUDA tensors");
    split_sizes.push_back(t.numel());
  }
  // dtype of torch::cat(tensors): int64 as soon as one input is int64
  int eb = 4;
  for (auto &t : tensors) eb = std::max(eb, id_bytes(t, "tensors"));
  const auto options = tensors[0].options().dtype(eb == 8 ? torch::kInt64 : torch::kInt32);
  int64_t N = 0;
  for (int64_t n : split_sizes) N += n;
  torch::Tensor unique = torch::empty({N}, options);
  torch::Tensor labels = torch::empty({N}, options);
  if (N == 0) return std::make_tuple(unique, labels.split_with_sizes(split_sizes, 0));
  const int64_t scratch_bytes = shmt_relabel_scratch_bytes(N);
  torch::Tensor scratch = device_bytes(scratch_bytes);
  const Readback::Slot count = readback().acquire();
  if (tensors.size() <= SHMT_RELABEL_MAX_SEGMENTS) {
    // concatenation fused into the first relabel pass
    std::vector<torch::Tensor> keep;
    const void *ptrs[SHMT_RELABEL_MAX_SEGMENTS];
    int64_t lens[SHMT_RELABEL_MAX_SEGMENTS];
    int widths[SHMT_RELABEL_MAX_SEGMENTS];
    for (size_t i = 0; i < tensors.size(); ++i) {
      keep.push_back(tensors[i].contiguous());
      ptrs[i] = keep[i].data_ptr();
      lens[i] = keep[i].numel();
      widths[i] = static_cast<int>(keep[i].element_size());
    }
    torch::Tensor total = torch::empty({N}, options);
    check(shmt_relabel_segments(ptrs, lens, widths, static_cast<int>(tensors.size()), nullptr, 0, eb,
                                total.data_ptr(), scratch.data_ptr(), scratch_bytes,
                                unique.data_ptr(), labels.data_ptr(), count.dev, current_stream()));
  } else {
    torch::Tensor total = torch::cat(tensors, 0).contiguous();
    check(shmt_relabel(total.data_ptr(), N, eb, scratch.data_ptr(), scratch_bytes, unique.data_ptr(),
                       labels.data_ptr(), count.dev, current_stream()));
  }
  const int64_t U = Readback::wait(count);
  return std::make_tuple(unique.narrow(0, 0, U), labels.split_with_sizes(split_sizes, 0));
}

// One hop of mini-batch sampling as the dataloader runs it
// (python/shmtensor/sampling.py:128-143): sample the seeds, then relabel
// [seeds, sub_indices]. No counterpart as a single operator in the reference.
// All kernels of the hop are queued without the host learning nnz in between
// (the relabel kernels read it from sub_indptr[S] on the device); nnz and the
// number of unique ids are picked up together at the end. The result is
// (sub_indptr, sub_indices, unique, relabel_indices): exactly what
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

void check_csr(CsrArgs &g) {
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

// A hop whose kernels are queued on the stream that was current when it was
// issued and whose two data-dependent sizes have not been read yet.
struct PendingHop {
  bool finished = false;
  HopResult result;                       // valid when finished
  int64_t S = 0;                          // number of seeds the buffers are sized for
  bool counted_seeds = false;             // the kernels took the true number of seeds from device memory
  torch::Tensor sub_indptr, sub_indices, unique, labels, coo_dst;
  torch::Tensor workspace;                // plan + relabel input + relabel scratch, kept until the sizes are in
  Readback::Slot nnz_slot{}, count_slot{};
  int64_t *count_dev = nullptr;           // fused hops: the number of unique ids in device memory as well
};

// Queues one hop. `seeds_len` (device memory) makes it a chained hop: `seeds`
// then holds an unknown number of ids, at most seeds.numel(), and the kernels
// read the true number there (the count_dev of the hop before, whose unique
// buffer is `seeds`); every buffer is sized for the bound.
PendingHop hop_issue(const CsrArgs &g, torch::Tensor seeds, const int64_t *seeds_len, int64_t num_picks,
                     bool replace, std::optional<int64_t> seed, int64_t stream_id) {
  PendingHop h;
  seeds = cuda_ids(seeds, "seeds");
  TORCH_CHECK(num_picks >= 0, "num_picks must be >= 0");
  const int64_t S = seeds.numel();
  const bool fused = S > 0 && num_picks > 0 && num_picks <= kEagerOutputLimit / S;
  if (!fused) {  // degenerate or very large bound: the two operators one after the other
    TORCH_CHECK(seeds_len == nullptr, "internal: a chained hop must be a fused one");
    auto sampled = sample_impl(g.indptr, g.indices, g.cached() ? &*g.gpu_indptr : nullptr,
                               g.cached() ? &*g.gpu_indices : nullptr, g.hashmap, seeds, num_picks,
                               replace, seed, stream_id);
    auto relabeled = tensor_relabel({seeds, std::get<1>(sampled)});
    h.result = HopResult{std::get<0>(sampled), std::get<1>(sampled), std::get<0>(relabeled),
                         std::get<1>(relabeled)[1], torch::Tensor()};
    if (g.coo) {
      const torch::Tensor &sp = h.result.sub_indptr, &labels = h.result.relabel_indices;
      h.result.coo_dst = torch::empty_like(labels);
      check(shmt_csr_rows(sp.data_ptr(), static_cast<int>(sp.element_size()), seeds.numel(), labels.numel(),
                          h.result.coo_dst.data_ptr(), static_cast<int>(labels.element_size()),
                          current_stream()));
    }
    h.finished = true;
    return h;
  }
  const int pb = static_cast<int>(g.indptr.element_size());
  const int ib = static_cast<int>(g.indices.element_size());
  const int sb = static_cast<int>(seeds.element_size());
  void *stream = current_stream();
  const int64_t bound = S * num_picks;
  h.S = S;
  h.counted_seeds = seeds_len != nullptr;
  const int eb = std::max(sb, ib);
  const auto id_type = eb == 8 ? torch::kInt64 : torch::kInt32;
  const int64_t n_max = S + bound;
  auto aligned = [](int64_t bytes) { return (bytes + 255) & ~int64_t{255}; };
  // Two allocations per hop (the allocator is shared by all host threads that drive
  // batches): one for the four results, which are typed views of it, and the count ...
  torch::Tensor results = device_bytes(aligned((S + 1) * pb) + aligned(bound * ib) + 2 * aligned(n_max * eb) +
                                       (g.coo ? aligned(bound * eb) : 0) + 256);
  int64_t offset = 0;
  auto carve = [&](int64_t count, int elem, torch::ScalarType type) {
    torch::Tensor t = results.narrow(0, offset, count * elem).view(type);
    offset += aligned(count * elem);
    return t;
  };
  h.sub_indptr = carve(S + 1, pb, g.indptr.scalar_type());
  h.sub_indices = carve(bound, ib, g.indices.scalar_type());
  h.unique = carve(n_max, eb, id_type);
  h.labels = carve(n_max, eb, id_type);
  if (g.coo) h.coo_dst = carve(bound, eb, id_type);
  h.count_dev = reinterpret_cast<int64_t *>(static_cast<char *>(results.data_ptr()) + offset);
  // ... and one for everything that does not outlive the hop
  const int64_t plan_bytes = shmt_sample_plan_bytes(S);
  const int64_t total_bytes = n_max * eb;
  const int64_t scratch_bytes = shmt_relabel_scratch_bytes(n_max);
  h.workspace = device_bytes(aligned(plan_bytes) + aligned(total_bytes) + scratch_bytes);
  char *const plan_ptr = static_cast<char *>(h.workspace.data_ptr());
  char *const total_ptr = plan_ptr + aligned(plan_bytes);
  char *const scratch_ptr = total_ptr + aligned(total_bytes);
  h.nnz_slot = readback().acquire();
  h.count_slot = readback().acquire();
  shmt_hop_job j{};
  j.indptr = g.indptr_dev;
  j.ptr_bytes = pb;
  j.indices = g.indices_dev;
  j.idx_bytes = ib;
  j.cache_indptr = g.cached() ? g.gpu_indptr->data_ptr() : nullptr;
  j.cache_indices = g.cached() ? g.gpu_indices->data_ptr() : nullptr;
  j.map = g.cached() ? g.hashmap->handle() : nullptr;
  j.seeds = seeds.data_ptr();
  j.seed_bytes = sb;
  j.max_seeds = S;
  j.seeds_len = seeds_len;
  j.k = num_picks;
  j.replace = replace;
  j.rng_seed = static_cast<uint64_t>(seed.value_or(kDefaultSeed));
  j.rng_seed_dev = nullptr;
  j.rng_stream = static_cast<uint32_t>(stream_id);
  j.sub_indptr = h.sub_indptr.data_ptr();
  j.sub_indices = h.sub_indices.data_ptr();
  j.plan = plan_ptr;
  j.plan_bytes = plan_bytes;
  j.elem_bytes = eb;
  j.total_out = total_ptr;
  j.scratch = scratch_ptr;
  j.scratch_bytes = scratch_bytes;
  j.unique_out = h.unique.data_ptr();
  j.labels_out = h.labels.data_ptr();
  j.nnz_out = h.nnz_slot.dev;
  j.count_out = h.count_slot.dev;
  j.count_dev_out = h.count_dev;
  j.coo_dst = g.coo ? h.coo_dst.data_ptr() : nullptr;
  j.coo_bytes = eb;
  check(shmt_sample_hops_chained(&j, 1, stream));
  return h;
}

// Must run with the stream of hop_issue current (the wait falls back to
// synchronising the current stream). `true_seeds`: the number of seeds of a
// chained hop, i.e. the number of unique ids of the hop before it.
HopResult hop_finish(PendingHop &h, int64_t true_seeds = -1) {
  if (!h.finished) {
    const int64_t S = h.counted_seeds ? true_seeds : h.S;
    TORCH_CHECK(S >= 0 && S <= h.S, "internal: chained hop finished without its seed count");
    const int64_t nnz = Readback::wait(h.nnz_slot);
    const int64_t U = Readback::wait(h.count_slot);
    h.result = HopResult{h.sub_indptr.narrow(0, 0, S + 1), h.sub_indices.narrow(0, 0, nnz),
                         h.unique.narrow(0, 0, U), h.labels.narrow(0, S, nnz),
                         h.coo_dst.defined() ? h.coo_dst.narrow(0, 0, nnz) : torch::Tensor()};
    h.finished = true;
    // scratch goes back to the allocator of its stream; work queued later on
    // that stream is ordered after the kernels that still read it
    h.workspace = torch::Tensor();
  }
  return h.result;
}

// Feature table of the fused "last relabel -> fetch" (sample_blocks_fetch).
struct FeatureArgs {
  torch::Tensor uva_data;
  std::optional<torch::Tensor> gpu_data;
  StaticHashmap *hashmap;   // null: every row comes from uva_data
  int64_t max_rows;         // rows of the speculative output; < 0: the hop's bound; 0: do not speculate
  void *uva_dev = nullptr;
  bool cached() const { return hashmap != nullptr; }
};

void check_features(FeatureArgs &f) {
  TORCH_CHECK(!f.cached() || f.gpu_data.has_value(), "a feature hashmap needs gpu_data");
  check_tables(f.uva_data, f.cached() ? &*f.gpu_data : nullptr);
  f.uva_dev = device_address(f.uva_data, "uva_data");
}

torch::Tensor fetch_rows(const FeatureArgs &f, const torch::Tensor &ids) {
  return fetch_impl(f.uva_data, f.cached() ? &*f.gpu_data : nullptr, ids, f.hashmap, nullptr);
}

// Queues the fetch of the rows of the hop's unique ids behind the hop, before
// the host knows how many there are: the kernel takes the count from device
// memory. Returns the output sized for `rows` ids (the caller narrows it once
// the count is in).
torch::Tensor issue_counted_fetch(const PendingHop &h, const FeatureArgs &f, int64_t rows) {
  const RowShape rs = row_shape(f.uva_data, rows);
  torch::Tensor out = torch::empty(rs.out_sizes, f.uva_data.options().device(torch::kCUDA));
  void *cache_ptr = nullptr;
  if (f.cached()) cache_ptr = f.gpu_data->numel() > 0 ? f.gpu_data->data_ptr() : out.data_ptr();
  check(shmt_fetch_counted(f.uva_dev, cache_ptr, h.unique.data_ptr(),
                           static_cast<int>(h.unique.element_size()),
                           f.cached() ? f.hashmap->handle() : nullptr, nullptr, 0, out.data_ptr(), rows,
                           h.count_dev, nullptr, rs.row_bytes, current_stream()));
  return out;
}

HopResult sample_hop(torch::Tensor indptr, torch::Tensor indices,
                     std::optional<torch::Tensor> gpu_indptr, std::optional<torch::Tensor> gpu_indices,
                     StaticHashmap *hashmap, torch::Tensor seeds, int64_t num_picks, bool replace,
                     std::optional<int64_t> seed, int64_t stream_id, bool coo) {
  CsrArgs g{indptr, indices, gpu_indptr, gpu_indices, hashmap, coo};
  check_csr(g);
  PendingHop h = hop_issue(g, seeds, nullptr, num_picks, replace, seed, stream_id);
  return hop_finish(h);
}

// RAII: make `s` torch's current stream, restore the previous one on exit.
class CurrentStreamScope {
 public:
  explicit CurrentStreamScope(c10::hip::HIPStreamMasqueradingAsCUDA s)
      : prev_(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA()) {
    c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(s);
  }
  ~CurrentStreamScope() { c10::hip::setCurrentHIPStreamMasqueradingAsCUDA(prev_); }
  CurrentStreamScope(const CurrentStreamScope &) = delete;
  CurrentStreamScope &operator=(const CurrentStreamScope &) = delete;

 private:
  c10::hip::HIPStreamMasqueradingAsCUDA prev_;
};

constexpr int64_t kMaxBatchesInFlight = 32;

struct BatchResult {
  std::vector<HopResult> hops;
  torch::Tensor features;  // defined only when features were asked for
};

// Ids a chained hop's buffers may be sized for: hop h + 1 is queued behind hop
// h without waiting for h's sizes as long as its bound (every seed of the
// bound-sized unique list of h with all its picks) stays below this.
constexpr int64_t kChainLimit = 1ll << 21;

// All hops of one batch on the current stream: hop h samples `num_picks[h]`
// neighbours of the previous hop's unique ids (RNG stream h when a seed is
// given), as the dataloader's loop does (python/shmtensor/sampling.py:128-143; `num_picks` is
// already in call order, i.e. the reversed fanout list). Consecutive hops are
// chained on the device while their bounds allow: the next hop takes its seeds
// and their number from the buffers of the one before and is queued at once,
// and the host reads all sizes of the chain afterwards. With `features` the
// rows of the last hop's unique ids (the input nodes of the mini-batch) are
// fetched as well, queued directly behind that hop.
BatchResult run_hops(const CsrArgs &g, torch::Tensor seeds, const std::vector<int64_t> &num_picks,
                     bool replace, std::optional<int64_t> seed, const FeatureArgs *features) {
  BatchResult batch;
  batch.hops.reserve(num_picks.size());
  std::vector<PendingHop> chain;  // queued hops whose sizes have not been read yet
  auto finish_chain = [&]() {
    for (PendingHop &h : chain) {
      const int64_t true_seeds = batch.hops.empty() ? -1 : batch.hops.back().unique.numel();
      batch.hops.push_back(hop_finish(h, true_seeds));
    }
    chain.clear();
  };
  for (size_t hop = 0; hop < num_picks.size(); ++hop) {
    // without an RNG seed every call draws from the fixed default seed, stream 0,
    // as every call of the reference does (src/cache_graph_sampling.cu:204,407)
    const int64_t rng_stream = seed.has_value() ? static_cast<int64_t>(hop) : 0;
    const int64_t k = num_picks[hop];
    const int64_t *seeds_len = nullptr;
    if (!chain.empty()) {
      const PendingHop &prev = chain.back();
      if (k > 0 && prev.unique.numel() <= kChainLimit / (k + 1)) {
        seeds = prev.unique;
        seeds_len = prev.count_dev;
      } else {
        finish_chain();
      }
    }
    if (chain.empty() && !batch.hops.empty()) seeds = batch.hops.back().unique;
    PendingHop h = hop_issue(g, seeds, seeds_len, k, replace, seed, rng_stream);
    if (h.finished)
      batch.hops.push_back(h.result);  // ran as two separate operators (never a chained hop)
    else
      chain.push_back(std::move(h));
  }
  if (!features) {
    finish_chain();
    return batch;
  }
  const FeatureArgs &f = *features;
  const bool speculate = f.max_rows != 0 && row_shape(f.uva_data, 0).row_bytes > 0;
  if (chain.empty() || !speculate) {
    finish_chain();
    batch.features = fetch_rows(f, batch.hops.empty() ? cuda_ids(seeds, "seeds") : batch.hops.back().unique);
    return batch;
  }
  // the rows of the last hop's unique ids, fetched before the host knows how many there are
  const PendingHop &last = chain.back();
  const int64_t bound = last.unique.numel();
  const int64_t rows = f.max_rows < 0 ? bound : std::min(bound, f.max_rows);
  torch::Tensor out = issue_counted_fetch(last, f, rows);
  finish_chain();
  const torch::Tensor &nodes = batch.hops.back().unique;
  batch.features = nodes.numel() <= rows ? out.narrow(0, 0, nodes.numel()) : fetch_rows(f, nodes);
  return batch;
}

// True when every hop of a batch of S seeds can be queued without a host wait
// (all hops fused, every hop after the first within the chaining bound).
bool chains_entirely(int64_t S, const std::vector<int64_t> &num_picks) {
  if (S <= 0 || num_picks.empty()) return false;
  int64_t bound = S;
  for (size_t hop = 0; hop < num_picks.size(); ++hop) {
    const int64_t k = num_picks[hop];
    if (k <= 0 || k > kEagerOutputLimit / bound) return false;
    if (hop > 0 && bound > kChainLimit / (k + 1)) return false;
    bound += bound * k;
  }
  return true;
}

// The hops of several batches in lockstep on the current stream: hop h of all
// batches goes out in ONE call whose launches are shared between the batches
// (shmt_sample_hops_chained), then hop h + 1, chained on the device; the sizes
// of all of them are read at the end. Every batch must chain entirely, so all
// bounds are known up front: a batch gets one allocation for the results of
// all its hops and one for their scratch, and result tensors are made once,
// when the sizes are in (with several batches per launch the host's own
// bookkeeping, not the GPU, is what bounds the rate).
struct TogetherHop {
  int64_t s_max, n_max;
  int64_t off_sp, off_si, off_unique, off_labels, off_coo, off_count;  // bytes into the batch's results
  Readback::Slot nnz, count;
};
struct TogetherBatch {
  torch::Tensor seeds, results, workspace;
  std::vector<TogetherHop> hops;
  int sb, eb;
};

// Queue all hops of the group; finish_together() reads the sizes and makes the results.
std::vector<TogetherBatch> issue_together(const CsrArgs &g, const std::vector<torch::Tensor> &seeds,
                                          const std::vector<int64_t> &num_picks, bool replace,
                                          const std::vector<std::optional<int64_t>> &rng) {
  using Hop = TogetherHop;
  using Batch = TogetherBatch;
  const size_t B = seeds.size(), H = num_picks.size();
  const int pb = static_cast<int>(g.indptr.element_size());
  const int ib = static_cast<int>(g.indices.element_size());
  auto aligned = [](int64_t bytes) { return (bytes + 255) & ~int64_t{255}; };
  void *stream = current_stream();
  std::vector<Batch> batches(B);
  std::vector<std::vector<shmt_hop_job>> jobs(H, std::vector<shmt_hop_job>(B));
  for (size_t b = 0; b < B; ++b) {
    Batch &bt = batches[b];
    bt.seeds = cuda_ids(seeds[b], "seeds");
    bt.sb = static_cast<int>(bt.seeds.element_size());
    bt.eb = std::max(bt.sb, ib);
    bt.hops.resize(H);
    int64_t results_bytes = 0, work_bytes = 0, s_max = bt.seeds.numel();
    std::vector<int64_t> off_plan(H), off_total(H), off_scratch(H), plan_bytes(H), scratch_bytes(H);
    for (size_t h = 0; h < H; ++h) {
      Hop &hp = bt.hops[h];
      const int64_t k = num_picks[h];
      hp.s_max = s_max;
      hp.n_max = s_max + s_max * k;
      hp.off_sp = results_bytes;
      results_bytes += aligned((s_max + 1) * pb);
      hp.off_si = results_bytes;
      results_bytes += aligned(s_max * k * ib);
      hp.off_unique = results_bytes;
      results_bytes += aligned(hp.n_max * bt.eb);
      hp.off_labels = results_bytes;
      results_bytes += aligned(hp.n_max * bt.eb);
      hp.off_coo = results_bytes;
      if (g.coo) results_bytes += aligned(s_max * k * bt.eb);
      hp.off_count = results_bytes;
      results_bytes += 256;
      plan_bytes[h] = shmt_sample_plan_bytes(s_max);
      scratch_bytes[h] = shmt_relabel_scratch_bytes(hp.n_max);
      off_plan[h] = work_bytes;
      work_bytes += aligned(plan_bytes[h]);
      off_total[h] = work_bytes;
      work_bytes += aligned(hp.n_max * bt.eb);
      off_scratch[h] = work_bytes;
      work_bytes += aligned(scratch_bytes[h]);
      s_max = hp.n_max;
    }
    bt.results = device_bytes(results_bytes);
    bt.workspace = device_bytes(work_bytes);
    char *const r = static_cast<char *>(bt.results.data_ptr());
    char *const w = static_cast<char *>(bt.workspace.data_ptr());
    for (size_t h = 0; h < H; ++h) {
      Hop &hp = bt.hops[h];
      hp.nnz = readback().acquire();
      hp.count = readback().acquire();
      shmt_hop_job &j = jobs[h][b];
      j = shmt_hop_job{};
      j.indptr = g.indptr_dev;
      j.ptr_bytes = pb;
      j.indices = g.indices_dev;
      j.idx_bytes = ib;
      j.cache_indptr = g.cached() ? g.gpu_indptr->data_ptr() : nullptr;
      j.cache_indices = g.cached() ? g.gpu_indices->data_ptr() : nullptr;
      j.map = g.cached() ? g.hashmap->handle() : nullptr;
      j.seeds = h == 0 ? bt.seeds.data_ptr() : static_cast<void *>(r + bt.hops[h - 1].off_unique);
      j.seed_bytes = h == 0 ? bt.sb : bt.eb;
      j.max_seeds = hp.s_max;
      j.seeds_len = h == 0 ? nullptr : reinterpret_cast<const int64_t *>(r + bt.hops[h - 1].off_count);
      j.k = num_picks[h];
      j.replace = replace;
      j.rng_seed = static_cast<uint64_t>(rng[b].value_or(kDefaultSeed));
      j.rng_seed_dev = nullptr;
      j.rng_stream = static_cast<uint32_t>(rng[b].has_value() ? h : 0);
      j.sub_indptr = r + hp.off_sp;
      j.sub_indices = r + hp.off_si;
      j.plan = w + off_plan[h];
      j.plan_bytes = plan_bytes[h];
      j.elem_bytes = bt.eb;
      j.total_out = w + off_total[h];
      j.scratch = w + off_scratch[h];
      j.scratch_bytes = scratch_bytes[h];
      j.unique_out = r + hp.off_unique;
      j.labels_out = r + hp.off_labels;
      j.nnz_out = hp.nnz.dev;
      j.count_out = hp.count.dev;
      j.count_dev_out = reinterpret_cast<int64_t *>(r + hp.off_count);
      j.coo_dst = g.coo ? r + hp.off_coo : nullptr;
      j.coo_bytes = bt.eb;
    }
  }
  for (size_t h = 0; h < H; ++h)
    check(shmt_sample_hops_chained(jobs[h].data(), static_cast<int>(B), stream));
  return batches;
}

// Must run with the stream of issue_together current.
std::vector<BatchResult> finish_together(const CsrArgs &g, std::vector<TogetherBatch> &batches) {
  const size_t B = batches.size();
  const int pb = static_cast<int>(g.indptr.element_size());
  const int ib = static_cast<int>(g.indices.element_size());
  // sizes in, batch by batch; typed views of the results buffer are made from two typed aliases of it
  std::vector<BatchResult> out(B);
  for (size_t b = 0; b < B; ++b) {
    TogetherBatch &bt = batches[b];
    const size_t H = bt.hops.size();
    const torch::Tensor as32 = bt.results.view(torch::kInt32), as64 = bt.results.view(torch::kInt64);
    auto typed = [&](int64_t off, int64_t first, int64_t count, int elem) {
      return (elem == 8 ? as64 : as32).narrow(0, off / elem + first, count);
    };
    int64_t s_now = bt.seeds.numel();
    out[b].hops.reserve(H);
    for (size_t h = 0; h < H; ++h) {
      const TogetherHop &hp = bt.hops[h];
      const int64_t nnz = Readback::wait(hp.nnz);
      const int64_t U = Readback::wait(hp.count);
      out[b].hops.push_back(HopResult{typed(hp.off_sp, 0, s_now + 1, pb), typed(hp.off_si, 0, nnz, ib),
                                      typed(hp.off_unique, 0, U, bt.eb), typed(hp.off_labels, s_now, nnz, bt.eb),
                                      g.coo ? typed(hp.off_coo, 0, nnz, bt.eb) : torch::Tensor()});
      s_now = U;
    }
  }
  return out;
}

// Multi-hop sampling of several independent seed batches. Every batch is a
// chain of short, latency-bound kernels with a host read of the sizes at its end,
// so one batch alone leaves most of the GPU idle. Batches whose hops all chain
// on the device advance in lockstep, `min(max_in_flight, 8)` at a time, and
// share their kernel launches (issue_together). Otherwise (a hop too large to
// chain, or features to fetch) up to `max_in_flight` batches advance at the
// same time, each driven by its own host thread on its own stream (default
// priority, the same streams every call), so that both the launches and the
// kernels of different batches overlap. Results are those of
// sample_hop called hop by hop, batch by batch (`seeds_rng[b]` is the RNG seed
// of batch b, RNG stream = hop number; without seeds_rng every hop uses the
// default seed and stream 0); they are ordered after the calling
// stream's earlier work and before its later work, and their memory is
// registered with the calling stream.
std::vector<BatchResult> drive_batches(const CsrArgs &g, const std::vector<torch::Tensor> &seeds,
                                       const std::vector<int64_t> &num_picks, bool replace,
                                       const std::optional<std::vector<int64_t>> &seeds_rng,
                                       int64_t max_in_flight, const FeatureArgs *features) {
  const int64_t B = static_cast<int64_t>(seeds.size());
  TORCH_CHECK(!seeds_rng.has_value() || static_cast<int64_t>(seeds_rng->size()) == B,
              "seeds_rng must have one entry per batch");
  TORCH_CHECK(max_in_flight >= 1, "max_in_flight must be >= 1");
  for (const torch::Tensor &t : seeds) cuda_ids(t, "seeds");
  for (int64_t k : num_picks) TORCH_CHECK(k >= 0, "num_picks must be >= 0");
  auto rng_of = [&](int64_t b) {
    return seeds_rng ? std::optional<int64_t>((*seeds_rng)[b]) : std::nullopt;
  };
  std::vector<BatchResult> out(B);
  const int64_t K = std::min<int64_t>({max_in_flight, kMaxBatchesInFlight, B});
  if (K <= 1) {
    py::gil_scoped_release no_gil;  // lets a Python thread that prefetches batches run beside the caller
    for (int64_t b = 0; b < B; ++b) {
      if (!features && chains_entirely(seeds[b].numel(), num_picks)) {
        // all bounds known up front: two allocations and one set of result tensors for the batch
        std::vector<TogetherBatch> one = issue_together(g, {seeds[b]}, num_picks, replace, {rng_of(b)});
        out[b] = std::move(finish_together(g, one)[0]);
      } else {
        out[b] = run_hops(g, seeds[b], num_picks, replace, rng_of(b), features);
      }
    }
    return out;
  }
  if (!features) {
    // Batches whose hops all chain on the device advance in lockstep and share their launches:
    // up to 8 of them per kernel launch, on the caller's stream, without helper threads.
    bool any = false;
    for (int64_t b = 0; b < B; ++b) any = any || chains_entirely(seeds[b].numel(), num_picks);
    if (any) {
      py::gil_scoped_release no_gil;
      // (two groups are queued at a time, each holding two size slots per hop and batch)
      const int64_t by_slots = Readback::kSlots / 8 / static_cast<int64_t>(std::max<size_t>(num_picks.size(), 1));
      const size_t group_size = static_cast<size_t>(std::max<int64_t>(1, std::min<int64_t>({K, 8, by_slots})));
      std::vector<int64_t> group;
      // one group is queued ahead of the one whose sizes are being read, so the GPU never waits
      // for the host's bookkeeping
      std::deque<std::pair<std::vector<int64_t>, std::vector<TogetherBatch>>> queued;
      auto finish_oldest = [&]() {
        std::vector<BatchResult> done = finish_together(g, queued.front().second);
        for (size_t i = 0; i < done.size(); ++i) out[queued.front().first[i]] = std::move(done[i]);
        queued.pop_front();
      };
      auto flush = [&]() {
        if (group.empty()) return;
        std::vector<torch::Tensor> group_seeds;
        std::vector<std::optional<int64_t>> group_rng;
        for (int64_t b : group) {
          group_seeds.push_back(seeds[b]);
          group_rng.push_back(rng_of(b));
        }
        queued.emplace_back(group, issue_together(g, group_seeds, num_picks, replace, group_rng));
        group.clear();
        if (queued.size() > 1) finish_oldest();
      };
      for (int64_t b = 0; b < B; ++b) {
        if (chains_entirely(seeds[b].numel(), num_picks)) {
          group.push_back(b);
          if (group.size() == group_size) flush();
        } else {
          out[b] = run_hops(g, seeds[b], num_picks, replace, rng_of(b), nullptr);
        }
      }
      flush();
      while (!queued.empty()) finish_oldest();
      return out;
    }
  }
  const auto caller = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const c10::DeviceIndex device = caller.device_index();
  at::cuda::CUDAEvent inputs_ready;
  inputs_ready.record(caller);
  // the same lanes every call: torch's allocator caches blocks per stream
  static std::vector<c10::hip::HIPStreamMasqueradingAsCUDA> lane_pool;
  while (static_cast<int64_t>(lane_pool.size()) < K)
    lane_pool.push_back(c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, device));
  const std::vector<c10::hip::HIPStreamMasqueradingAsCUDA> lanes(lane_pool.begin(), lane_pool.begin() + K);
  for (auto &lane : lanes) inputs_ready.block(lane);

  std::atomic<int64_t> next_batch{0};
  std::vector<std::exception_ptr> failures(K);
  {
    py::gil_scoped_release no_gil;  // the workers touch tensors, never Python objects
    std::vector<std::thread> workers;
    workers.reserve(K);
    for (int64_t j = 0; j < K; ++j) {
      workers.emplace_back([&, j] {
        try {
          c10::hip::set_device(device);
          CurrentStreamScope scope(lanes[j]);  // torch's current stream is per thread
          for (int64_t b = next_batch++; b < B; b = next_batch++)
            out[b] = run_hops(g, seeds[b], num_picks, replace, rng_of(b), features);
        } catch (...) {
          failures[j] = std::current_exception();
          next_batch = B;  // the call will fail: the other workers stop after their current batch
        }
      });
    }
    for (auto &w : workers) w.join();
  }
  // later work of the caller's stream sees the results; their memory must not be
  // reused by the lanes while the caller's stream may still read it
  for (auto &lane : lanes) {
    at::cuda::CUDAEvent done;
    done.record(lane);
    done.block(caller);
  }
  for (auto &f : failures)
    if (f) std::rethrow_exception(f);
  auto hand_over = [&](const torch::Tensor &t) {
    if (t.defined() && t.is_cuda() && t.numel() > 0) t.record_stream(caller.unwrap());
  };
  for (auto &batch : out) {
    for (auto &r : batch.hops)
      for (const torch::Tensor &t : {r.sub_indptr, r.sub_indices, r.unique, r.relabel_indices, r.coo_dst})
        hand_over(t);
    hand_over(batch.features);
  }
  return out;
}

std::vector<std::vector<HopResult>> sample_blocks(
    torch::Tensor indptr, torch::Tensor indices, std::optional<torch::Tensor> gpu_indptr,
    std::optional<torch::Tensor> gpu_indices, StaticHashmap *hashmap, std::vector<torch::Tensor> seeds,
    std::vector<int64_t> num_picks, bool replace, std::optional<std::vector<int64_t>> seeds_rng,
    int64_t max_in_flight, bool coo) {
  CsrArgs g{indptr, indices, gpu_indptr, gpu_indices, hashmap, coo};
  check_csr(g);
  std::vector<std::vector<HopResult>> out;
  for (BatchResult &b : drive_batches(g, seeds, num_picks, replace, seeds_rng, max_in_flight, nullptr))
    out.push_back(std::move(b.hops));
  return out;
}

// sample_blocks plus, per batch, the feature rows of its input nodes (the
// unique ids of the last hop): `features[b][i, :]` = row of `unique[i]`, as
// cache_fetch(uva_data, gpu_data, unique, data_hashmap) returns it (uva_fetch
// without a data_hashmap). The fetch is queued behind the last relabel before
// the host knows the number of unique ids, into an output of `max_rows` rows
// (None: the bound S * (k + 1) of the last hop; 0: never speculate); a batch
// with more unique ids than that is fetched after its count is known.
std::vector<std::pair<std::vector<HopResult>, torch::Tensor>> sample_blocks_fetch(
    torch::Tensor indptr, torch::Tensor indices, std::optional<torch::Tensor> gpu_indptr,
    std::optional<torch::Tensor> gpu_indices, StaticHashmap *hashmap, std::vector<torch::Tensor> seeds,
    std::vector<int64_t> num_picks, bool replace, torch::Tensor uva_data,
    std::optional<torch::Tensor> gpu_data, StaticHashmap *data_hashmap,
    std::optional<std::vector<int64_t>> seeds_rng, int64_t max_in_flight,
    std::optional<int64_t> max_rows, bool coo) {
  CsrArgs g{indptr, indices, gpu_indptr, gpu_indices, hashmap, coo};
  check_csr(g);
  TORCH_CHECK(!max_rows.has_value() || *max_rows >= 0, "max_rows must be >= 0");
  FeatureArgs f{uva_data, gpu_data, data_hashmap, max_rows.value_or(-1)};
  check_features(f);
  std::vector<std::pair<std::vector<HopResult>, torch::Tensor>> out;
  for (BatchResult &b : drive_batches(g, seeds, num_picks, replace, seeds_rng, max_in_flight, &f))
    out.emplace_back(std::move(b.hops), std::move(b.features));
  return out;
}


// ---- a mini-batch captured once, replayed per batch ---------------------------
//
// Sampling a mini-batch is a chain of ~20 short kernels; issuing them costs the
// host more than running them costs the GPU once several batches are in flight.
// BatchSampler queues the chained hops of one batch once, on fixed buffers,
// records that as a HIP graph and from then on spends one staging kernel and one
// graph launch per batch: the seeds, their number and the RNG seed are copied
// to where the recorded kernels read them. Several such "lanes" (graph, buffers,
// stream) exist so that batches overlap; a lane's output memory is handed to
// the caller as tensors and the lane is reused only after those tensors have
// all been released. Results are those of sample_blocks.
constexpr int64_t kSamplerLimit = 1ll << 23;  // ids the last hop's buffers may be sized for

class SamplerState : public std::enable_shared_from_this<SamplerState> {
 public:
  struct HopBuffers {
    int64_t s_max, k, n_max;
    int64_t off_sp, off_si, off_unique, off_labels;  // into the lane's results
    int64_t *count_dev;
    char *plan, *total, *scratch;
    int64_t plan_bytes, scratch_bytes;
    volatile int64_t *nnz_host, *count_host;
    int64_t *nnz_dev, *count_slot_dev;
  };
  struct Lane {
    bool seeded = false;
    torch::Tensor results, workspace, slots;
    std::vector<HopBuffers> hops;
    char *staged = nullptr;
    int64_t *len_dev = nullptr;
    uint64_t *rng_dev = nullptr;
    void *graph = nullptr;
    std::optional<c10::hip::HIPStreamMasqueradingAsCUDA> stream, consumer;
    // events live as long as the lane: creating one costs more than a short kernel runs
    at::cuda::CUDAEvent inputs_ready;   // caller's stream position when the batch was handed in
    at::cuda::CUDAEvent done;           // lane's stream position after the replay
    at::cuda::CUDAEvent released;       // consumer's stream position when the results were dropped
    bool wait_released = false;
    bool release_unordered = false;     // the drop could not be ordered: synchronise before reuse
  };

  SamplerState(CsrArgs g, int64_t batch_size, std::vector<int64_t> picks, bool replace, int seed_bytes)
      : g_(std::move(g)), batch_size_(batch_size), picks_(std::move(picks)), replace_(replace), sb_(seed_bytes) {
    pb_ = static_cast<int>(g_.indptr.element_size());
    ib_ = static_cast<int>(g_.indices.element_size());
    eb_ = std::max(sb_, ib_);
  }
  ~SamplerState() {
    for (auto &lane : lanes_) shmt_graph_destroy(lane->graph);
  }

  int64_t lanes() {
    std::lock_guard<std::mutex> lock(mutex_);
    return static_cast<int64_t>(lanes_.size());
  }

  Lane *acquire(bool seeded) {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      for (size_t i = 0; i < free_.size(); ++i) {
        if (free_[i]->seeded == seeded) {
          Lane *lane = free_[i];
          free_.erase(free_.begin() + static_cast<std::ptrdiff_t>(i));
          return lane;
        }
      }
    }
    std::unique_ptr<Lane> lane = make_lane(seeded);
    std::lock_guard<std::mutex> lock(mutex_);
    lanes_.push_back(std::move(lane));
    return lanes_.back().get();
  }

  // Called when the last tensor that views a lane's results is gone, from
  // whichever thread dropped it.
  void release(Lane *lane) noexcept {
    try {
      lane->released.record(*lane->consumer);
      lane->wait_released = true;
      lane->release_unordered = false;
    } catch (...) {
      lane->wait_released = false;
      lane->release_unordered = true;
    }
    try {
      std::lock_guard<std::mutex> lock(mutex_);
      free_.push_back(lane);
    } catch (...) {
    }
  }

  // A lane that was acquired but whose batch could not be queued.
  void give_back(Lane *lane) {
    lane->release_unordered = true;  // whatever did get queued is waited for before the next use
    std::lock_guard<std::mutex> lock(mutex_);
    free_.push_back(lane);
  }

  // Stage the batch and replay the lane's graph on the lane's stream.
  void launch(Lane *lane, const torch::Tensor &seeds, uint64_t rng_seed,
              c10::hip::HIPStreamMasqueradingAsCUDA caller) {
    auto &stream = *lane->stream;
    lane->inputs_ready.record(caller);
    lane->inputs_ready.block(stream);
    if (lane->release_unordered) c10::hip::device_synchronize();
    if (lane->wait_released) lane->released.block(stream);
    lane->wait_released = false;
    lane->release_unordered = false;
    for (HopBuffers &b : lane->hops) {
      *b.nnz_host = kSlotPending;
      *b.count_host = kSlotPending;
    }
    std::atomic_thread_fence(std::memory_order_seq_cst);
    void *raw = static_cast<void *>(stream.stream());
    check(shmt_stage_seeds(seeds.data_ptr(), sb_, seeds.numel(), lane->staged, sb_, lane->len_dev, rng_seed,
                           lane->rng_dev, raw));
    check(shmt_graph_launch(lane->graph, raw));
  }

  // Wait for the sizes of every hop and hand the lane's results out as tensors.
  std::vector<HopResult> collect(Lane *lane, int64_t n_seeds, c10::hip::HIPStreamMasqueradingAsCUDA caller) {
    std::vector<int64_t> nnz, uniq;
    for (HopBuffers &b : lane->hops) {
      nnz.push_back(wait_slot(b.nnz_host, *lane->stream));
      uniq.push_back(wait_slot(b.count_host, *lane->stream));
    }
    lane->done.record(*lane->stream);
    lane->done.block(caller);
    lane->consumer = caller;
    auto self = shared_from_this();
    torch::Tensor blob = torch::from_blob(
        lane->results.data_ptr(), {lane->results.numel()}, [self, lane](void *) { self->release(lane); },
        lane->results.options());
    std::vector<HopResult> out;
    int64_t s_now = n_seeds;
    const auto id_type = eb_ == 8 ? torch::kInt64 : torch::kInt32;
    for (size_t h = 0; h < lane->hops.size(); ++h) {
      const HopBuffers &b = lane->hops[h];
      auto view = [&](int64_t off, int64_t first, int64_t count, int elem, torch::ScalarType type) {
        return blob.narrow(0, off + first * elem, count * elem).view(type);
      };
      out.push_back(HopResult{view(b.off_sp, 0, s_now + 1, pb_, g_.indptr.scalar_type()),
                              view(b.off_si, 0, nnz[h], ib_, g_.indices.scalar_type()),
                              view(b.off_unique, 0, uniq[h], eb_, id_type),
                              view(b.off_labels, s_now, nnz[h], eb_, id_type), torch::Tensor()});
      s_now = uniq[h];
    }
    return out;
  }

  const CsrArgs &graph() const { return g_; }
  int64_t batch_size() const { return batch_size_; }
  const std::vector<int64_t> &picks() const { return picks_; }
  bool replace() const { return replace_; }
  int seed_bytes() const { return sb_; }

 private:
  static constexpr int64_t kSlotPending = INT64_MIN;

  static int64_t wait_slot(volatile int64_t *slot, c10::hip::HIPStreamMasqueradingAsCUDA stream) {
    const auto t0 = std::chrono::steady_clock::now();
    for (uint64_t spins = 0;; ++spins) {
      const int64_t v = *slot;
      if (v != kSlotPending) return v;
      if ((spins & 1023) == 1023 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(200)) break;
      __builtin_ia32_pause();
    }
    stream.synchronize();  // surfaces a failed replay
    const int64_t v = *slot;
    TORCH_CHECK(v != kSlotPending, "the GPU did not report a result size (kernel failed?)");
    return v;
  }

  std::unique_ptr<Lane> make_lane(bool seeded) {
    auto lane = std::make_unique<Lane>();
    lane->seeded = seeded;
    auto aligned = [](int64_t bytes) { return (bytes + 255) & ~int64_t{255}; };
    // sizes: every hop is sized for the bound the hop before it allows
    int64_t results_bytes = 0, work_bytes = aligned(batch_size_ * sb_) + 512;
    int64_t s_max = batch_size_;
    std::vector<HopBuffers> hops;
    for (int64_t k : picks_) {
      HopBuffers b{};
      b.s_max = s_max;
      b.k = k;
      b.n_max = s_max + s_max * k;
      b.off_sp = results_bytes;
      results_bytes += aligned((s_max + 1) * pb_);
      b.off_si = results_bytes;
      results_bytes += aligned(s_max * k * ib_);
      b.off_unique = results_bytes;
      results_bytes += aligned(b.n_max * eb_);
      b.off_labels = results_bytes;
      results_bytes += aligned(b.n_max * eb_);
      b.plan_bytes = shmt_sample_plan_bytes(s_max);
      b.scratch_bytes = shmt_relabel_scratch_bytes(b.n_max);
      work_bytes += aligned(b.plan_bytes) + aligned(b.n_max * eb_) + aligned(b.scratch_bytes) + 256;
      hops.push_back(b);
      s_max = b.n_max;
    }
    lane->results = device_bytes(results_bytes);
    lane->workspace = device_bytes(work_bytes);
    lane->slots = torch::zeros({static_cast<int64_t>(2 * hops.size())},
                               torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    void *slots_dev = nullptr;
    check(shmt_host_devptr(lane->slots.data_ptr(), &slots_dev));
    char *w = static_cast<char *>(lane->workspace.data_ptr());
    lane->staged = w;
    w += aligned(batch_size_ * sb_);
    lane->len_dev = reinterpret_cast<int64_t *>(w);
    lane->rng_dev = reinterpret_cast<uint64_t *>(w + 256);
    w += 512;
    for (size_t h = 0; h < hops.size(); ++h) {
      HopBuffers &b = hops[h];
      b.plan = w;
      w += aligned(b.plan_bytes);
      b.total = w;
      w += aligned(b.n_max * eb_);
      b.scratch = w;
      w += aligned(b.scratch_bytes);
      b.count_dev = reinterpret_cast<int64_t *>(w);
      w += 256;
      b.nnz_host = lane->slots.data_ptr<int64_t>() + 2 * h;
      b.count_host = lane->slots.data_ptr<int64_t>() + 2 * h + 1;
      b.nnz_dev = static_cast<int64_t *>(slots_dev) + 2 * h;
      b.count_slot_dev = static_cast<int64_t *>(slots_dev) + 2 * h + 1;
    }
    lane->hops = std::move(hops);
    const c10::DeviceIndex device = lane->results.device().index();
    lane->stream = c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, device);
    // record the chained hops once
    void *raw = static_cast<void *>(lane->stream->stream());
    char *r = static_cast<char *>(lane->results.data_ptr());
    check(shmt_capture_begin(raw));
    int rc = SHMT_OK;
    const void *src = lane->staged;
    const int64_t *src_len = lane->len_dev;
    int src_bytes = sb_;
    for (size_t h = 0; h < lane->hops.size() && rc == SHMT_OK; ++h) {
      const HopBuffers &b = lane->hops[h];
      rc = shmt_sample_hop_chained(
          g_.indptr_dev, pb_, g_.indices_dev, ib_, g_.cached() ? g_.gpu_indptr->data_ptr() : nullptr,
          g_.cached() ? g_.gpu_indices->data_ptr() : nullptr, g_.cached() ? g_.hashmap->handle() : nullptr, src,
          src_bytes, b.s_max, src_len, b.k, replace_, kDefaultSeed, lane->rng_dev,
          static_cast<uint32_t>(seeded ? h : 0), r + b.off_sp, r + b.off_si, b.plan, b.plan_bytes, eb_, b.total,
          b.scratch, b.scratch_bytes, r + b.off_unique, r + b.off_labels, b.nnz_dev, b.count_slot_dev, b.count_dev,
          raw);
      src = r + b.off_unique;
      src_len = b.count_dev;
      src_bytes = eb_;
    }
    const std::string failure = rc == SHMT_OK ? std::string() : std::string(shmt_last_error());
    const int end_rc = shmt_capture_end(raw, &lane->graph);  // always: leaves the stream usable
    TORCH_CHECK(rc == SHMT_OK, failure);
    check(end_rc);
    return lane;
  }

  CsrArgs g_;
  int64_t batch_size_;
  std::vector<int64_t> picks_;
  bool replace_;
  int sb_, pb_ = 8, ib_ = 8, eb_ = 8;
  std::mutex mutex_;
  std::vector<std::unique_ptr<Lane>> lanes_;
  std::vector<Lane *> free_;
};

class BatchSampler {
 public:
  BatchSampler(torch::Tensor indptr, torch::Tensor indices, std::optional<torch::Tensor> gpu_indptr,
               std::optional<torch::Tensor> gpu_indices, StaticHashmap *hashmap, int64_t batch_size,
               std::vector<int64_t> num_picks, bool replace, int64_t seed_bytes) {
    CsrArgs g{indptr, indices, gpu_indptr, gpu_indices, hashmap};
    check_csr(g);
    TORCH_CHECK(seed_bytes == 4 || seed_bytes == 8, "seed_bytes must be 4 or 8");
    TORCH_CHECK(batch_size >= 1, "batch_size must be >= 1");
    TORCH_CHECK(!num_picks.empty(), "num_picks must name at least one hop");
    int64_t s_max = batch_size;
    for (int64_t k : num_picks) {
      TORCH_CHECK(k >= 1, "num_picks must be >= 1 for a recorded batch");
      TORCH_CHECK(s_max <= kSamplerLimit / (k + 1),
                  "the recorded batch would need buffers for more than ", kSamplerLimit,
                  " ids per hop (batch_size * prod(num_picks + 1)): use sample_blocks for this configuration");
      s_max += s_max * k;
    }
    state_ = std::make_shared<SamplerState>(std::move(g), batch_size, std::move(num_picks), replace,
                                            static_cast<int>(seed_bytes));
  }

  // Queue one batch (at most batch_size seeds; `seed_rng` as one entry of
  // sample_blocks' seeds_rng) and return at once with a ticket for collect().
  // Submitting further batches before collecting keeps several in flight.
  int64_t submit(torch::Tensor seeds, std::optional<int64_t> seed_rng) {
    SamplerState &st = *state_;
    seeds = checked(seeds);
    Pending p;
    p.n_seeds = seeds.numel();
    p.caller = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    if (p.n_seeds == 0) {  // nothing to replay a graph for: the plain operators give the empty results
      p.ready = run_hops(st.graph(), seeds, st.picks(), st.replace(), seed_rng, nullptr).hops;
    } else {
      p.lane = st.acquire(seed_rng.has_value());
      try {
        st.launch(p.lane, seeds, seed_rng ? static_cast<uint64_t>(*seed_rng) : kDefaultSeed, *p.caller);
      } catch (...) {
        st.give_back(p.lane);
        throw;
      }
    }
    std::lock_guard<std::mutex> lock(mutex_);
    const int64_t ticket = next_ticket_++;
    pending_.emplace(ticket, std::move(p));
    return ticket;
  }

  // The hop results of a submitted batch, as sample_blocks returns them for
  // it. The tensors view memory of the sampler that is reused once all of them
  // are gone; they are ready on the stream that was current at submit() and
  // must be consumed on it (or on streams ordered after it).
  std::vector<HopResult> collect(int64_t ticket) {
    Pending p;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      auto it = pending_.find(ticket);
      TORCH_CHECK(it != pending_.end(), "unknown or already collected ticket ", ticket);
      p = std::move(it->second);
      pending_.erase(it);
    }
    if (!p.lane) return p.ready;
    return state_->collect(p.lane, p.n_seeds, *p.caller);
  }

  // submit + collect for a list of batches, at most max_in_flight of them
  // queued at a time: the equivalent of sample_blocks.
  std::vector<std::vector<HopResult>> sample(std::vector<torch::Tensor> seeds,
                                             std::optional<std::vector<int64_t>> seeds_rng,
                                             int64_t max_in_flight) {
    const int64_t B = static_cast<int64_t>(seeds.size());
    TORCH_CHECK(!seeds_rng.has_value() || static_cast<int64_t>(seeds_rng->size()) == B,
                "seeds_rng must have one entry per batch");
    TORCH_CHECK(max_in_flight >= 1, "max_in_flight must be >= 1");
    for (const torch::Tensor &t : seeds) checked(t);
    std::vector<std::vector<HopResult>> out(B);
    std::deque<std::pair<int64_t, int64_t>> in_flight;  // (batch, ticket)
    for (int64_t b = 0; b < B; ++b) {
      if (static_cast<int64_t>(in_flight.size()) >= max_in_flight) {
        out[in_flight.front().first] = collect(in_flight.front().second);
        in_flight.pop_front();
      }
      in_flight.emplace_back(b, submit(seeds[b], seeds_rng ? std::optional<int64_t>((*seeds_rng)[b]) : std::nullopt));
    }
    for (auto &f : in_flight) out[f.first] = collect(f.second);
    return out;
  }

  int64_t lanes() const { return state_->lanes(); }

 private:
  struct Pending {
    SamplerState::Lane *lane = nullptr;
    int64_t n_seeds = 0;
    std::optional<c10::hip::HIPStreamMasqueradingAsCUDA> caller;
    std::vector<HopResult> ready;  // batches that needed no replay
  };

  torch::Tensor checked(const torch::Tensor &seeds) const {
    torch::Tensor t = cuda_ids(seeds, "seeds");
    TORCH_CHECK(static_cast<int>(t.element_size()) == state_->seed_bytes(), "seeds must be ",
                state_->seed_bytes(), "-byte ids, as the sampler was built for");
    TORCH_CHECK(t.numel() <= state_->batch_size(), "a batch holds at most ", state_->batch_size(), " seeds");
    return t;
  }

  std::shared_ptr<SamplerState> state_;
  std::mutex mutex_;
  int64_t next_ticket_ = 0;
  std::unordered_map<int64_t, Pending> pending_;
};

}  // namespace

void register_host_tensors(py::module &m);  // host_tensors.cc

namespace pybind11 {
namespace detail {
// A hop goes to Python as the tuple (sub_indptr, sub_indices, unique, relabel_indices), with the
// destination positions as a fifth member when the coordinate form was asked for.
template <>
struct type_caster<HopResult> {
  PYBIND11_TYPE_CASTER(HopResult, const_name("Tuple[Tensor, ...]"));
  bool load(handle, bool) { return false; }
  static handle cast(const HopResult &h, return_value_policy, handle) {
    if (h.coo_dst.defined())
      return py::make_tuple(h.sub_indptr, h.sub_indices, h.unique, h.relabel_indices, h.coo_dst).release();
    return py::make_tuple(h.sub_indptr, h.sub_indices, h.unique, h.relabel_indices).release();
  }
};
}  // namespace detail
}  // namespace pybind11

PYBIND11_MODULE(ShmTensorLib, m) {
  m.doc() = "MI355X-native ShmTensor GPU-cache operators (HIP, gfx950)";
  register_host_tensors(m);

  m.def("thrust_scan", &thrust_scan, py::arg("tensor"));

  m.def("set_host_register", &set_host_register, py::arg("enabled"),
        "Let pin_memory() try to register existing memory in place (hipHostRegister) before it falls "
        "back to re-homing the tensor's storage in new pinned memory. Off by default; also switched on "
        "by SHMT_HOST_REGISTER=1 in the environment.");
  m.def("pin_memory", &pin_memory, py::arg("data"))
      .def("unpin_memory", &unpin_memory, py::arg("data"))
      .def("uva_fetch", &uva_fetch, py::arg("data"), py::arg("indices"))
      .def("cache_fetch", &cache_fetch, py::arg("uva_data"), py::arg("gpu_data"),
           py::arg("indices"), py::arg("hashmap"))
      .def("cache_fetch_with_mask", &cache_fetch_with_mask, py::arg("uva_data"),
           py::arg("gpu_data"), py::arg("indices"), py::arg("mask"))
      .def("uva_set", &uva_set, py::arg("data"), py::arg("indices"), py::arg("update"))
      .def("cache_set", &cache_set, py::arg("uva_data"), py::arg("gpu_data"), py::arg("indices"),
           py::arg("update"), py::arg("hashmap"), py::arg("write_through") = false)
      .def("cache_set_with_mask", &cache_set_with_mask, py::arg("uva_data"), py::arg("gpu_data"),
           py::arg("indices"), py::arg("update"), py::arg("mask"), py::arg("write_through") = false)
      .def("csr_sampling", &csr_sampling, py::arg("indptr"), py::arg("indices"), py::arg("seeds"),
           py::arg("num_picks"), py::arg("replace"), py::arg("seed") = py::none(),
           py::arg("stream_id") = 0)
      .def("csr_cache_sampling", &csr_cache_sampling, py::arg("uva_indptr"),
           py::arg("uva_indices"), py::arg("gpu_indptr"), py::arg("gpu_indices"),
           py::arg("hashmap"), py::arg("seeds"), py::arg("num_picks"), py::arg("replace"),
           py::arg("seed") = py::none(), py::arg("stream_id") = 0)
      .def("create_subcsr", &create_subcsr, py::arg("uva_indptr"), py::arg("uva_indices"),
           py::arg("seeds"))
      .def("tensor_relabel", &tensor_relabel, py::arg("tensors"))
      .def("sample_hop", &sample_hop, py::arg("indptr"), py::arg("indices"), py::arg("gpu_indptr"),
           py::arg("gpu_indices"), py::arg("hashmap"), py::arg("seeds"), py::arg("num_picks"),
           py::arg("replace"), py::arg("seed") = py::none(), py::arg("stream_id") = 0, py::arg("coo") = false)
      .def("sample_blocks", &sample_blocks, py::arg("indptr"), py::arg("indices"), py::arg("gpu_indptr"),
           py::arg("gpu_indices"), py::arg("hashmap"), py::arg("seeds"), py::arg("num_picks"),
           py::arg("replace"), py::arg("seeds_rng") = py::none(), py::arg("max_in_flight") = 4,
           py::arg("coo") = false)
      .def("sample_blocks_fetch", &sample_blocks_fetch, py::arg("indptr"), py::arg("indices"),
           py::arg("gpu_indptr"), py::arg("gpu_indices"), py::arg("hashmap"), py::arg("seeds"),
           py::arg("num_picks"), py::arg("replace"), py::arg("uva_data"), py::arg("gpu_data"),
           py::arg("data_hashmap"), py::arg("seeds_rng") = py::none(), py::arg("max_in_flight") = 4,
           py::arg("max_rows") = py::none(), py::arg("coo") = false);

  py::class_<BatchSampler>(m, "BatchSampler")
      .def(py::init<torch::Tensor, torch::Tensor, std::optional<torch::Tensor>, std::optional<torch::Tensor>,
                    StaticHashmap *, int64_t, std::vector<int64_t>, bool, int64_t>(),
           py::arg("indptr"), py::arg("indices"), py::arg("gpu_indptr"), py::arg("gpu_indices"), py::arg("hashmap"),
           py::arg("batch_size"), py::arg("num_picks"), py::arg("replace"), py::arg("seed_bytes") = 8,
           py::keep_alive<1, 6>())
      .def("sample", &BatchSampler::sample, py::arg("seeds"), py::arg("seeds_rng") = py::none(),
           py::arg("max_in_flight") = 4, py::call_guard<py::gil_scoped_release>())
      .def("submit", &BatchSampler::submit, py::arg("seeds"), py::arg("seed_rng") = py::none(),
           py::call_guard<py::gil_scoped_release>())
      .def("collect", &BatchSampler::collect, py::arg("ticket"), py::call_guard<py::gil_scoped_release>())
      .def("lanes", &BatchSampler::lanes);

  py::class_<StaticHashmap>(m, "CUCOStaticHashmap")
      .def(py::init<torch::Tensor, torch::Tensor, double>())
      .def("query", &StaticHashmap::query)
      .def("capacity", &StaticHashmap::capacity)
      .def("memory_usage", &StaticHashmap::memory_usage)
      .def("layout", &StaticHashmap::layout);
}
