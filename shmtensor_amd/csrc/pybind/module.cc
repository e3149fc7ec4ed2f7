// ShmTensorLib: the Python operator surface of the GPU-cache hot path, with
// the names, argument names, defaults and return structure of the reference
// module (src/pybind.cc:16-65 in the ShmTensor tree). Host C++ only: every
// operator validates its tensors, allocates outputs and scratch from torch's
// caching allocator and calls the C ABI of libshmt.so (include/shmt.h) on
// torch's current HIP stream. Failures raise RuntimeError; nothing exits.
// This file holds the reference's operators and the module definition; the
// multi-batch driver is in batch_driver.cc, the graph-replaying sampler in
// batch_sampler.cc, the host tensor providers in host_tensors.cc.
#include "shim.h"

namespace shim {

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

// Scan workspace that is kept clean: one per device and stream, all zero when it is made; every scan
// leaves it all zero again, so no scan has to clear it first (shmt_*_scan_kept). Scans of one stream run
// one after the other, which is all the sharing such a workspace allows.
torch::Tensor kept_scan_workspace(int64_t bytes) {
  static std::mutex mutex;
  static std::unordered_map<uint64_t, torch::Tensor> kept;
  const auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const uint64_t key = (static_cast<uint64_t>(stream.device_index()) << 48) ^ static_cast<uint64_t>(stream.id());
  std::lock_guard<std::mutex> lock(mutex);
  torch::Tensor &w = kept[key];
  if (!w.defined() || w.numel() < bytes)
    w = torch::zeros({std::max<int64_t>(bytes, 1 << 16)}, torch::TensorOptions().dtype(torch::kUInt8).device(torch::kCUDA));
  return w;
}

// thrust_scan, src/thrust_scan.cu:9-18: in-place inclusive sum over int32.
void thrust_scan(torch::Tensor tensor) {
  TORCH_CHECK(tensor.scalar_type() == torch::kInt32, "thrust_scan expects an int32 tensor");
  TORCH_CHECK(tensor.is_contiguous(), "tensor must be contiguous");
  const int64_t n = tensor.numel();
  if (n == 0) return;
  const int64_t tmp_bytes = shmt_scan_tmp_bytes(n);
  torch::Tensor tmp = tmp_bytes > 0 ? kept_scan_workspace(tmp_bytes) : torch::Tensor();
  check(shmt_inclusive_scan_i32_kept(device_address(tensor, "tensor"), n, tmp_bytes > 0 ? tmp.data_ptr() : nullptr,
                                     tmp_bytes, current_stream()));
}

// What shmt_async_error reports as an exception (nothing when no kernel gave up a bounded wait).
// Synchronises the device; meant for the end of a job, for tests, and for the slow path of a size
// read-back that did not arrive.
void raise_async_error() {
  int code = 0;
  check(shmt_async_error(&code));
  TORCH_CHECK(code == 0, shmt_last_error());
}

// ---- sampling ------------------------------------------------------------------


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
  const bool eager = S > 0 && num_picks > 0 && num_picks <= kEagerOutputBytes / ib / S;
  torch::Tensor sub_indices;
  if (eager) {
    sub_indices = torch::empty({S * num_picks}, indices.options().device(dev));
    check(shmt_sample(indptr_dev, pb, indices_dev, ib, map ? gpu_indptr->data_ptr() : nullptr,
                      map ? gpu_indices->data_ptr() : nullptr, map ? map->handle() : nullptr, seeds.data_ptr(),
                      sb, S, num_picks, replace, rng_seed, static_cast<uint32_t>(stream_id),
                      sub_indptr.data_ptr(), sub_indices.data_ptr(), plan.data_ptr(), plan_bytes, total.dev,
                      stream));
    const int64_t nnz = Readback::wait(total);
    // a view keeps the whole bound-sized buffer alive: hand back a copy when most of a large one is unused
    const bool mostly_unused = nnz < S * num_picks / 4 && S * num_picks * ib > (16ll << 20);
    sub_indices = mostly_unused ? sub_indices.narrow(0, 0, nnz).clone() : sub_indices.narrow(0, 0, nnz);
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
// 2^31 ids or more: concatenated as int64 and relabelled with 64-bit positions (shmt_relabel switches to
// its wide form); the reference cannot represent such inputs (int numel, src/tensor_relabel.cu:136).
static std::tuple<torch::Tensor, std::vector<torch::Tensor>> relabel_huge(const std::vector<torch::Tensor> &tensors,
                                                                          const std::vector<int64_t> &split_sizes,
                                                                          int64_t N) {
  std::vector<torch::Tensor> wide;
  for (const auto &t : tensors) wide.push_back(t.to(torch::kInt64));
  torch::Tensor total = torch::cat(wide, 0).contiguous();
  wide.clear();
  torch::Tensor unique = torch::empty({N}, total.options());
  torch::Tensor labels = torch::empty({N}, total.options());
  const int64_t scratch_bytes = shmt_relabel_scratch_bytes(N);
  torch::Tensor scratch = device_bytes(scratch_bytes);
  const Readback::Slot count = readback().acquire();
  check(shmt_relabel(total.data_ptr(), N, 8, scratch.data_ptr(), scratch_bytes, unique.data_ptr(),
                     labels.data_ptr(), count.dev, current_stream()));
  const int64_t U = Readback::wait(count);
  return std::make_tuple(unique.narrow(0, 0, U), labels.split_with_sizes(split_sizes, 0));
}

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
  // 2^31 ids and more: positions need 64 bits, so the results are int64 whatever the inputs are
  if (N >= (int64_t{1} << 31)) return relabel_huge(tensors, split_sizes, N);
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
}  // namespace shim

using namespace shim;

PYBIND11_MODULE(ShmTensorLib, m) {
  m.doc() = "MI355X-native ShmTensor GPU-cache operators (HIP, gfx950)";
  register_host_tensors(m);

  m.def("thrust_scan", &thrust_scan, py::arg("tensor"));

  m.def("raise_async_error", &raise_async_error,
        "Raises RuntimeError if a kernel of this library gave up a bounded wait for another workgroup since the "
        "last call (a device-wide scan whose look-back starved); synchronises the device.");
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

  register_batch_sampler(m);

  py::class_<StaticHashmap>(m, "CUCOStaticHashmap")
      .def(py::init<torch::Tensor, torch::Tensor, double, const std::string &>(), py::arg("keys"), py::arg("values"),
           py::arg("load_factor"), py::arg("layout") = "auto")
      .def("query", &StaticHashmap::query)
      .def("capacity", &StaticHashmap::capacity)
      .def("memory_usage", &StaticHashmap::memory_usage)
      .def("layout", &StaticHashmap::layout);
}
