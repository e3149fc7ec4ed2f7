// BatchSampler: the chained hops of one mini-batch recorded once as a HIP graph
// and replayed per batch (no counterpart in the reference, whose loader issues
// every kernel of every hop from the host: python/shmtensor/sampling.py:128-143
// in the ShmTensor tree).
#include "shim.h"

namespace shim {

namespace {

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
      p.ready = sample_batch(st.graph(), seeds, st.picks(), st.replace(), seed_rng);
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

void register_batch_sampler(py::module &m) {
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
}

}  // namespace shim
