// Multi-hop, multi-batch sampling on top of the C ABI's fused hop: one hop as
// one launch sequence (sample_hop), the hops of a batch chained on the device,
// several batches advancing at once (merged launches, or one host thread and
// stream per batch), and the feature fetch queued behind the last relabel.
// The body of the dataloader's loop (python/shmtensor/sampling.py:128-143 in
// the ShmTensor tree) as operators; results are those of csr_[cache_]sampling
// + tensor_relabel called hop by hop.
#include "shim.h"

namespace shim {

namespace {

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
  const bool fused =
      S > 0 && num_picks > 0 &&
      hop_buffer_bytes(S, num_picks, static_cast<int>(g.indptr.element_size()),
                       static_cast<int>(g.indices.element_size()),
                       static_cast<int>(std::max(seeds.element_size(), g.indices.element_size()))) <= kHopBufferBytes;
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
  // Set when several batches are driven and the id-addressed table lives in host memory: the rows
  // that miss the cache are moved by a second, small launch on this stream (one per device, shared
  // by all batches), so that the host-link part of batch b runs beside the sampling of batch b + 1
  // instead of holding the whole GPU while it waits for the link.
  std::optional<c10::hip::HIPStreamMasqueradingAsCUDA> link, link2;
  std::atomic<uint32_t> *turn = nullptr;  // batches take the two link streams in turn
  // ... and the rows that hit by a launch on this one, so that the HBM-bound copy of batch b runs beside
  // the latency-bound sampling kernels of batch b + 1 as well
  std::optional<c10::hip::HIPStreamMasqueradingAsCUDA> hits;
  int link_blocks = 0;      // workgroups of the launch on the link stream (0: the library's default)
  bool cached() const { return hashmap != nullptr; }
};

void check_features(FeatureArgs &f) {
  TORCH_CHECK(!f.cached() || f.gpu_data.has_value(), "a feature hashmap needs gpu_data");
  check_tables(f.uva_data, f.cached() ? &*f.gpu_data : nullptr);
  f.uva_dev = device_address(f.uva_data, "uva_data");
}

// True when the fetch of `ids` can go out as hits now + listed misses on the link stream.
bool splits(const FeatureArgs &f, int64_t rows, int64_t row_bytes) {
  if (rows >= (int64_t{1} << 32) || !f.link.has_value() || !f.cached() || f.uva_data.is_cuda() || f.gpu_data->numel() == 0) return false;
  const uintptr_t bits = static_cast<uintptr_t>(row_bytes) | reinterpret_cast<uintptr_t>(f.uva_dev) |
                         reinterpret_cast<uintptr_t>(f.gpu_data->data_ptr());
  return row_bytes > 0 && (bits & 15) == 0;
}

// out[i, :] for the first min(rows, *count) ids (count: device memory, or null for exactly `rows`):
// the rows that hit the cache on the current stream, the others on the link stream behind them.
// Everything the link stream touches is registered with it; the caller makes its own stream wait
// for the link stream before it hands results on (drive_batches).
void fetch_split(const FeatureArgs &f, const torch::Tensor &ids, const int64_t *count, int64_t rows,
                 int64_t row_bytes, torch::Tensor &out) {
  const auto lane = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const auto &link = (f.turn->fetch_add(1) & 1) ? *f.link2 : *f.link;
  const auto &hits = *f.hits;
  torch::Tensor marks = device_bytes((rows + 31) / 32 * 4);  // one bit per row: it missed the cache
  uint32_t *const bits = reinterpret_cast<uint32_t *>(marks.data_ptr());
  const int ib = static_cast<int>(ids.element_size());
  at::cuda::CUDAEvent ids_ready;
  ids_ready.record(lane);
  ids_ready.block(hits);
  check(shmt_fetch_cached_part(f.uva_dev, f.gpu_data->data_ptr(), ids.data_ptr(), ib, f.hashmap->handle(), nullptr,
                               0, out.data_ptr(), rows, count, row_bytes, bits, hits.stream()));
  at::cuda::CUDAEvent hits_done;
  hits_done.record(hits);
  hits_done.block(link);
  check(shmt_fetch_missed_part(f.uva_dev, ids.data_ptr(), ib, bits, out.data_ptr(), rows, count, row_bytes,
                               f.link_blocks, link.stream()));
  for (const torch::Tensor &t : {out, marks, ids}) {
    t.record_stream(hits.unwrap());
    t.record_stream(link.unwrap());
  }
}

torch::Tensor fetch_rows(const FeatureArgs &f, const torch::Tensor &ids) {
  const RowShape rs = row_shape(f.uva_data, ids.numel());
  if (ids.numel() > 0 && splits(f, ids.numel(), rs.row_bytes)) {
    torch::Tensor out = torch::empty(rs.out_sizes, f.uva_data.options().device(torch::kCUDA));
    fetch_split(f, ids, nullptr, ids.numel(), rs.row_bytes, out);
    return out;
  }
  return fetch_impl(f.uva_data, f.cached() ? &*f.gpu_data : nullptr, ids, f.hashmap, nullptr);
}

// Queues the fetch of the rows of the hop's unique ids behind the hop, before
// the host knows how many there are: the kernel takes the count from device
// memory. Returns the output sized for `rows` ids (the caller narrows it once
// the count is in).
torch::Tensor issue_counted_fetch(const PendingHop &h, const FeatureArgs &f, int64_t rows) {
  const RowShape rs = row_shape(f.uva_data, rows);
  torch::Tensor out = torch::empty(rs.out_sizes, f.uva_data.options().device(torch::kCUDA));
  if (rows > 0 && splits(f, rows, rs.row_bytes)) {
    fetch_split(f, h.unique, h.count_dev, rows, rs.row_bytes, out);
    return out;
  }
  void *cache_ptr = nullptr;
  if (f.cached()) cache_ptr = f.gpu_data->numel() > 0 ? f.gpu_data->data_ptr() : out.data_ptr();
  check(shmt_fetch_counted(f.uva_dev, cache_ptr, h.unique.data_ptr(),
                           static_cast<int>(h.unique.element_size()),
                           f.cached() ? f.hashmap->handle() : nullptr, nullptr, 0, out.data_ptr(), rows,
                           h.count_dev, nullptr, rs.row_bytes, current_stream()));
  return out;
}

}  // namespace

HopResult sample_hop(torch::Tensor indptr, torch::Tensor indices,
                     std::optional<torch::Tensor> gpu_indptr, std::optional<torch::Tensor> gpu_indices,
                     StaticHashmap *hashmap, torch::Tensor seeds, int64_t num_picks, bool replace,
                     std::optional<int64_t> seed, int64_t stream_id, bool coo) {
  CsrArgs g{indptr, indices, gpu_indptr, gpu_indices, hashmap, coo};
  check_csr(g);
  PendingHop h = hop_issue(g, seeds, nullptr, num_picks, replace, seed, stream_id);
  return hop_finish(h);
}

namespace {

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
    if (k <= 0 || hop_buffer_bytes(bound, k, 8, 8, 8) > kHopBufferBytes) return false;
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

// Side streams of the pipelined fetch: two for the host-link launches, taken in turn, and one for the
// launch that moves the cached rows. Streams share a few hardware queues (four per process by default),
// work of two streams on one queue runs one after the other, and the runtime does not tell which stream
// sits on which queue: so the three are chosen, once per calling stream, by trying pool streams until
// three are found that make progress while the calling stream and the ones chosen before are kept busy
// (a 300 us wait on each; a stream that shares a queue with any of them cannot finish a kernel before
// that wait ends). When fewer than three such streams exist the remaining roles take what is left: the
// results do not depend on the choice, only the overlap does.
struct SideStreams {
  c10::hip::HIPStreamMasqueradingAsCUDA link, link2, hits;
};

bool runs_beside(const c10::hip::HIPStreamMasqueradingAsCUDA &candidate,
                 const std::vector<c10::hip::HIPStreamMasqueradingAsCUDA> &busy) {
  std::vector<at::cuda::CUDAEvent> waits(busy.size());
  for (size_t i = 0; i < busy.size(); ++i) {
    check(shmt_busy_wait(busy[i].stream(), 300));
    waits[i].record(busy[i]);
  }
  check(shmt_busy_wait(candidate.stream(), 0));
  at::cuda::CUDAEvent done;
  done.record(candidate);
  done.synchronize();
  bool beside = true;
  for (auto &w : waits) beside = beside && !w.query();
  for (auto &w : waits) w.synchronize();
  return beside;
}

SideStreams side_streams_for(const c10::hip::HIPStreamMasqueradingAsCUDA &caller) {
  static std::mutex mutex;
  static std::unordered_map<uint64_t, SideStreams> chosen;  // by device and calling stream
  const c10::DeviceIndex device = caller.device_index();
  const uint64_t key = (static_cast<uint64_t>(device) << 48) ^ static_cast<uint64_t>(caller.id());
  std::lock_guard<std::mutex> lock(mutex);
  auto it = chosen.find(key);
  if (it != chosen.end()) return it->second;
  std::vector<c10::hip::HIPStreamMasqueradingAsCUDA> pool, busy{caller}, picked;
  for (int i = 0; i < 12; ++i) pool.push_back(c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, device));
  for (const auto &s : pool) {
    if (picked.size() == 3) break;
    if (s == caller || std::find(picked.begin(), picked.end(), s) != picked.end()) continue;
    if (runs_beside(s, busy)) {
      picked.push_back(s);
      busy.push_back(s);
    }
  }
  for (const auto &s : pool)  // not enough independent queues: any other stream will do
    if (picked.size() < 3 && !(s == caller) && std::find(picked.begin(), picked.end(), s) == picked.end())
      picked.push_back(s);
  const SideStreams side{picked[0], picked[1], picked[2]};
  chosen.emplace(key, side);
  return side;
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
  const auto caller = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const c10::DeviceIndex device = caller.device_index();
  // With several batches to drive and the feature table in host memory, the rows that miss the cache
  // are fetched on the device's link stream (see FeatureArgs::link): batch b's host-link reads then
  // run beside batch b + 1's sampling, whatever the number of host threads.
  std::atomic<uint32_t> turn{0};
  FeatureArgs with_link;
  if (features && B > 1 && features->cached() && !features->uva_data.is_cuda()) {
    with_link.uva_data = features->uva_data;
    with_link.gpu_data = features->gpu_data;
    with_link.hashmap = features->hashmap;
    with_link.max_rows = features->max_rows;
    with_link.uva_dev = features->uva_dev;
    const SideStreams side = side_streams_for(caller);
    with_link.link = side.link;
    with_link.link2 = side.link2;
    with_link.hits = side.hits;
    with_link.turn = &turn;
    features = &with_link;
  }
  // what the link stream still has queued must be done before the caller's stream reads results
  auto join_link = [&]() {
    if (!features || !features->link.has_value()) return;
    for (const auto &side : {*features->link, *features->link2}) {  // ordered behind the hits stream's launches
      at::cuda::CUDAEvent done;
      done.record(side);
      done.block(caller);
    }
  };
  // With the side streams one host thread is the better driver: it queues batch b + 1's sampling while the
  // side streams still move batch b's rows (measured on 4,096-seed batches with 1 KiB feature rows: 1.17 ms
  // per batch from one thread, 1.30 - 1.45 from two, which contend for the allocator and the launch path).
  if (K <= 1 || (features && features->link.has_value())) {
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
    join_link();
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
  at::cuda::CUDAEvent inputs_ready;
  inputs_ready.record(caller);
  // the same lanes every call (torch's allocator caches blocks per stream), one pool per device;
  // calls may come from several Python threads (the dataloader's background producer among them)
  static std::mutex lane_pool_mutex;
  static std::unordered_map<int, std::vector<c10::hip::HIPStreamMasqueradingAsCUDA>> lane_pools;
  std::vector<c10::hip::HIPStreamMasqueradingAsCUDA> lanes;
  {
    std::lock_guard<std::mutex> lock(lane_pool_mutex);
    auto &pool = lane_pools[static_cast<int>(device)];
    while (static_cast<int64_t>(pool.size()) < K)
      pool.push_back(c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, device));
    lanes.assign(pool.begin(), pool.begin() + K);
  }
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
  join_link();
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

}  // namespace

std::vector<HopResult> sample_batch(const CsrArgs &g, torch::Tensor seeds, const std::vector<int64_t> &num_picks,
                                    bool replace, std::optional<int64_t> seed) {
  return run_hops(g, seeds, num_picks, replace, seed, nullptr).hops;
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


}  // namespace shim
