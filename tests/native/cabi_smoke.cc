// Stand-alone check of the C ABI: no Python, no torch. Links libshmt.so and the
// HIP runtime only, allocates with hipMalloc / hipHostMalloc, and compares the
// hashmap (dtype-chosen and key-chosen layouts), fetch, set, scan (with and
// without a workspace), relabel, sampling, the fused hop and the coordinate
// form of a block with plain C++ loops on the host. Exit status 0 = every check passed.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <numeric>
#include <unordered_map>
#include <vector>

#include "shmt.h"

#define HIP_OK(x)                                                                 \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      return 2;                                                                   \
    }                                                                             \
  } while (0)
#define SHMT_OK_(x)                                                          \
  do {                                                                       \
    int rc_ = (x);                                                           \
    if (rc_ != 0) {                                                          \
      fprintf(stderr, "%s:%d %s -> %d: %s\n", __FILE__, __LINE__, #x, rc_, shmt_last_error()); \
      return 3;                                                              \
    }                                                                        \
  } while (0)
#define EXPECT(c)                                                  \
  do {                                                             \
    if (!(c)) {                                                    \
      fprintf(stderr, "%s:%d check failed: %s\n", __FILE__, __LINE__, #c); \
      return 1;                                                    \
    }                                                              \
  } while (0)

template <typename T>
static T *to_device(const std::vector<T> &v) {
  T *d = nullptr;
  if (hipMalloc(&d, std::max<size_t>(v.size(), 1) * sizeof(T)) != hipSuccess) return nullptr;
  if (!v.empty()) (void)hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice);
  return d;
}
template <typename T>
static std::vector<T> to_host(const T *d, size_t n) {
  std::vector<T> v(n);
  if (n) (void)hipMemcpy(v.data(), d, n * sizeof(T), hipMemcpyDeviceToHost);
  return v;
}

static uint64_t rng_state = 88172645463325252ull;
static uint64_t rnd() {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return rng_state;
}

int main() {
  EXPECT(shmt_abi_version() == SHMT_ABI_VERSION);
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // ---- hashmap: 100,000 distinct int64 keys -> int32 values ----
  const int64_t n = 100000, nq = 300001;
  std::vector<int64_t> keys(n);
  std::vector<int32_t> vals(n);
  std::unordered_map<int64_t, int32_t> truth;
  for (int64_t i = 0; i < n; ++i) {
    int64_t k;
    do k = static_cast<int64_t>(rnd() % (1ull << 40)); while (truth.count(k));
    keys[i] = k;
    vals[i] = static_cast<int32_t>(i);
    truth[k] = vals[i];
  }
  int64_t *d_keys = to_device(keys);
  int32_t *d_vals = to_device(vals);
  const int64_t table_bytes = shmt_hashmap_table_bytes(n, 0.8, 8, 4);
  EXPECT(table_bytes > 0 && shmt_hashmap_capacity(n, 0.8) == 125000);
  void *d_table = nullptr;
  HIP_OK(hipMalloc(&d_table, table_bytes));
  shmt_hashmap_t *map = nullptr;
  SHMT_OK_(shmt_hashmap_create(&map, d_keys, d_vals, n, 8, 4, 0.8, d_table, table_bytes, stream));
  std::vector<int64_t> req(nq);
  for (int64_t i = 0; i < nq; ++i) req[i] = (i % 2) ? keys[rnd() % n] : static_cast<int64_t>(rnd() % (1ull << 40));
  int64_t *d_req = to_device(req);
  int32_t *d_res = nullptr;
  HIP_OK(hipMalloc(&d_res, nq * sizeof(int32_t)));
  SHMT_OK_(shmt_hashmap_query(map, d_req, 8, nq, d_res, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<int32_t> res = to_host(d_res, nq);
  for (int64_t i = 0; i < nq; ++i) {
    auto it = truth.find(req[i]);
    EXPECT(res[i] == (it == truth.end() ? -1 : it->second));
  }

  // ---- fetch / set: 20,000 x 96-byte rows in pinned host memory, 5,000 cached ----
  const int64_t rows = 20000, row_bytes = 96, cached = 5000, Q = 70001;
  char *h_table = nullptr;
  HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&h_table), rows * row_bytes, hipHostMallocDefault));
  for (int64_t i = 0; i < rows * row_bytes; ++i) h_table[i] = static_cast<char>(rnd());
  void *table_alias = nullptr;
  SHMT_OK_(shmt_host_devptr(h_table, &table_alias));
  std::vector<int64_t> cache_ids(rows);
  std::iota(cache_ids.begin(), cache_ids.end(), 0);
  for (int64_t i = rows - 1; i > 0; --i) std::swap(cache_ids[i], cache_ids[rnd() % (i + 1)]);
  cache_ids.resize(cached);
  std::vector<int64_t> slots(cached);
  std::iota(slots.begin(), slots.end(), 0);
  std::vector<char> cache_rows(cached * row_bytes);
  for (int64_t s = 0; s < cached; ++s)
    for (int64_t b = 0; b < row_bytes; ++b)
      cache_rows[s * row_bytes + b] = static_cast<char>(h_table[cache_ids[s] * row_bytes + b] ^ 0x5a);  // differs from host
  char *d_cache = to_device(cache_rows);
  int64_t *d_cids = to_device(cache_ids), *d_slots = to_device(slots);
  const int64_t fbytes = shmt_hashmap_table_bytes(cached, 0.5, 8, 8);
  void *d_ftable = nullptr;
  HIP_OK(hipMalloc(&d_ftable, fbytes));
  shmt_hashmap_t *fmap = nullptr;
  SHMT_OK_(shmt_hashmap_create(&fmap, d_cids, d_slots, cached, 8, 8, 0.5, d_ftable, fbytes, stream));
  std::vector<int32_t> q(Q);
  for (auto &x : q) x = static_cast<int32_t>(rnd() % rows);
  int32_t *d_q = to_device(q);
  char *d_out = nullptr;
  HIP_OK(hipMalloc(&d_out, Q * row_bytes));
  SHMT_OK_(shmt_fetch(table_alias, d_cache, d_q, 4, fmap, nullptr, 0, d_out, Q, row_bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<char> out = to_host(d_out, Q * row_bytes);
  std::unordered_map<int64_t, int64_t> slot_of;
  for (int64_t s = 0; s < cached; ++s) slot_of[cache_ids[s]] = s;
  for (int64_t i = 0; i < Q; ++i) {
    auto it = slot_of.find(q[i]);
    const char *expect = it == slot_of.end() ? h_table + q[i] * row_bytes : cache_rows.data() + it->second * row_bytes;
    EXPECT(std::equal(expect, expect + row_bytes, out.begin() + i * row_bytes));
  }
  // the same fetch told on the device how many rows there are: the first `counted`
  // rows arrive, the rest of the output is left alone
  const int64_t counted = Q / 3;
  int64_t *d_count = to_device(std::vector<int64_t>{counted});
  HIP_OK(hipMemsetAsync(d_out, 0x5A, Q * row_bytes, stream));
  SHMT_OK_(shmt_fetch_counted(table_alias, d_cache, d_q, 4, fmap, nullptr, 0, d_out, Q, d_count, nullptr,
                              row_bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<char> part = to_host(d_out, Q * row_bytes);
  EXPECT(std::equal(part.begin(), part.begin() + counted * row_bytes, out.begin()));
  for (int64_t i = counted * row_bytes; i < Q * row_bytes; ++i) EXPECT(part[i] == 0x5A);
  EXPECT(shmt_fetch_counted(table_alias, d_cache, d_q, 4, fmap, nullptr, 0, d_out, Q, nullptr, nullptr,
                            row_bytes, stream) == SHMT_EINVAL);
  HIP_OK(hipFree(d_count));
  // the same fetch in two launches: the rows that hit on this stream, the rows that missed from a few
  // workgroups on a second stream once an event says the first part is done; the bitmap is never cleared
  {
    hipStream_t side = nullptr;
    hipEvent_t hits_done = nullptr, misses_done = nullptr;
    HIP_OK(hipStreamCreateWithFlags(&side, hipStreamNonBlocking));
    HIP_OK(hipEventCreateWithFlags(&hits_done, hipEventDisableTiming));
    HIP_OK(hipEventCreateWithFlags(&misses_done, hipEventDisableTiming));
    uint32_t *d_bits = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_bits), ((Q + 31) / 32) * 4));
    HIP_OK(hipMemsetAsync(d_bits, 0xA5, ((Q + 31) / 32) * 4, stream));   // stale content must not matter
    HIP_OK(hipMemsetAsync(d_out, 0x5A, Q * row_bytes, stream));
    SHMT_OK_(shmt_fetch_cached_part(table_alias, d_cache, d_q, 4, fmap, nullptr, 0, d_out, Q, nullptr, row_bytes,
                                    d_bits, stream));
    HIP_OK(hipEventRecord(hits_done, stream));
    HIP_OK(hipStreamWaitEvent(side, hits_done, 0));
    SHMT_OK_(shmt_fetch_missed_part(table_alias, d_q, 4, d_bits, d_out, Q, nullptr, row_bytes, 8, side));
    HIP_OK(hipEventRecord(misses_done, side));
    HIP_OK(hipStreamWaitEvent(stream, misses_done, 0));
    HIP_OK(hipStreamSynchronize(stream));
    EXPECT(to_host(d_out, Q * row_bytes) == out);
    std::vector<uint32_t> bits = to_host(d_bits, (Q + 31) / 32);
    for (int64_t i = 0; i < Q; ++i) EXPECT(((bits[i / 32] >> (i % 32)) & 1u) == (slot_of.count(q[i]) ? 0u : 1u));
    // rows that do not allow 16-byte accesses are refused
    EXPECT(shmt_fetch_cached_part(table_alias, d_cache, d_q, 4, fmap, nullptr, 0, d_out, Q, nullptr, 24, d_bits,
                                  stream) == SHMT_EINVAL);
    HIP_OK(hipFree(d_bits));
    HIP_OK(hipEventDestroy(hits_done));
    HIP_OK(hipEventDestroy(misses_done));
    HIP_OK(hipStreamDestroy(side));
  }
  // pageable host memory is refused instead of faulting
  std::vector<char> pageable(4096);
  void *alias = nullptr;
  EXPECT(shmt_host_devptr(pageable.data(), &alias) == SHMT_ENOTPINNED);

  // ---- exclusive scan, int32, 1,000,001 elements ----
  const int64_t len = 1000001;
  std::vector<int32_t> a(len);
  for (auto &x : a) x = static_cast<int32_t>(rnd() % 1000);
  int32_t *d_a = to_device(a);
  const int64_t tmp_bytes = shmt_scan_tmp_bytes(len);
  void *d_tmp = nullptr;
  HIP_OK(hipMalloc(&d_tmp, std::max<int64_t>(tmp_bytes, 1)));
  SHMT_OK_(shmt_exclusive_scan(d_a, len, 4, d_tmp, tmp_bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<int32_t> scanned = to_host(d_a, len);
  uint32_t run = 0;
  for (int64_t i = 0; i < len; ++i) {
    EXPECT(static_cast<uint32_t>(scanned[i]) == run);
    run += static_cast<uint32_t>(a[i]);
  }

  // ---- relabel: 200,000 int64 ids, first-occurrence order ----
  const int64_t N = 200000;
  std::vector<int64_t> ids(N);
  for (auto &x : ids) x = static_cast<int64_t>(rnd() % 50000);
  int64_t *d_ids = to_device(ids), *d_unique = nullptr, *d_labels = nullptr, *h_count = nullptr;
  HIP_OK(hipMalloc(&d_unique, N * 8));
  HIP_OK(hipMalloc(&d_labels, N * 8));
  HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&h_count), 8, hipHostMallocDefault));
  const int64_t sbytes = shmt_relabel_scratch_bytes(N);
  void *d_scratch = nullptr;
  HIP_OK(hipMalloc(&d_scratch, sbytes));
  SHMT_OK_(shmt_relabel(d_ids, N, 8, d_scratch, sbytes, d_unique, d_labels, h_count, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::unordered_map<int64_t, int64_t> first;
  std::vector<int64_t> uniq;
  for (int64_t x : ids)
    if (first.emplace(x, static_cast<int64_t>(uniq.size())).second) uniq.push_back(x);
  EXPECT(*h_count == static_cast<int64_t>(uniq.size()));
  EXPECT(to_host(d_unique, uniq.size()) == uniq);
  std::vector<int64_t> labels = to_host(d_labels, N);
  for (int64_t i = 0; i < N; ++i) EXPECT(labels[i] == first[ids[i]]);

  // ---- sampling: 7-row CSR of the reference's unit test, k = 5, no replacement ----
  std::vector<int64_t> indptr = {0, 0, 4, 9, 15, 100, 101, 107}, indices(107), seeds = {5, 0, 1, 2, 3, 4, 6};
  std::iota(indices.begin(), indices.end(), 0);
  int64_t *d_indptr = to_device(indptr), *d_indices = to_device(indices), *d_seeds = to_device(seeds);
  int64_t *d_sub_indptr = nullptr, *d_sub = nullptr;
  HIP_OK(hipMalloc(&d_sub_indptr, 8 * 8));
  HIP_OK(hipMalloc(&d_sub, 7 * 5 * 8));
  const int64_t pbytes = shmt_sample_plan_bytes(7);
  void *d_plan = nullptr;
  HIP_OK(hipMalloc(&d_plan, pbytes));
  SHMT_OK_(shmt_sample_plan(d_indptr, 8, nullptr, nullptr, d_seeds, 8, 7, 5, 0, d_sub_indptr, d_plan, pbytes,
                            h_count, stream));
  SHMT_OK_(shmt_sample_pick(d_indices, nullptr, 8, d_seeds, 8, 7, 5, 0, d_sub_indptr, 8, d_plan, d_sub, 7777, 0,
                            stream));
  HIP_OK(hipStreamSynchronize(stream));
  EXPECT(*h_count == 25);
  EXPECT((to_host(d_sub_indptr, 8) == std::vector<int64_t>{0, 1, 1, 5, 10, 15, 20, 25}));
  std::vector<int64_t> sub = to_host(d_sub, 25);
  EXPECT((std::vector<int64_t>(sub.begin(), sub.begin() + 10) == std::vector<int64_t>{100, 0, 1, 2, 3, 4, 5, 6, 7, 8}));
  for (int seg = 0; seg < 3; ++seg) {      // rows of degree 6, 85, 6: five distinct neighbours each
    const int64_t lo[3] = {9, 15, 101}, hi[3] = {15, 100, 107};
    std::vector<int64_t> s(sub.begin() + 10 + 5 * seg, sub.begin() + 15 + 5 * seg);
    std::sort(s.begin(), s.end());
    EXPECT(std::adjacent_find(s.begin(), s.end()) == s.end() && s.front() >= lo[seg] && s.back() < hi[seg]);
  }

  // ---- the same hop as one launch sequence: sample + relabel([seeds, sampled]) ----
  {
    const int64_t S = 7, k = 5, n_max = S + S * k;
    int64_t *d_sp2 = nullptr, *d_sub2 = nullptr, *d_total = nullptr, *d_uniq2 = nullptr, *d_lab2 = nullptr;
    int64_t *h_nnz = nullptr, *h_uniq_count = nullptr;
    void *d_plan2 = nullptr, *d_scratch2 = nullptr;
    HIP_OK(hipMalloc(&d_sp2, (S + 1) * 8));
    HIP_OK(hipMalloc(&d_sub2, S * k * 8));
    HIP_OK(hipMalloc(&d_total, n_max * 8));
    HIP_OK(hipMalloc(&d_uniq2, n_max * 8));
    HIP_OK(hipMalloc(&d_lab2, n_max * 8));
    HIP_OK(hipMalloc(&d_plan2, pbytes));
    const int64_t sbytes2 = shmt_relabel_scratch_bytes(n_max);
    HIP_OK(hipMalloc(&d_scratch2, sbytes2));
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&h_nnz), 8, hipHostMallocDefault));
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&h_uniq_count), 8, hipHostMallocDefault));
    SHMT_OK_(shmt_sample_hop(d_indptr, 8, d_indices, 8, nullptr, nullptr, nullptr, d_seeds, 8, S, k, 0, 7777, 0,
                             d_sp2, d_sub2, d_plan2, pbytes, 8, d_total, d_scratch2, sbytes2, d_uniq2, d_lab2,
                             h_nnz, h_uniq_count, stream));
    HIP_OK(hipStreamSynchronize(stream));
    EXPECT(*h_nnz == 25);
    EXPECT(to_host(d_sp2, 8) == to_host(d_sub_indptr, 8));
    EXPECT(to_host(d_sub2, 25) == sub);                      // same seed and stream: same sample
    std::vector<int64_t> all(seeds);
    all.insert(all.end(), sub.begin(), sub.end());
    std::unordered_map<int64_t, int64_t> first2;
    std::vector<int64_t> uniq2;
    for (int64_t x : all)
      if (first2.emplace(x, static_cast<int64_t>(uniq2.size())).second) uniq2.push_back(x);
    EXPECT(*h_uniq_count == static_cast<int64_t>(uniq2.size()));
    EXPECT(to_host(d_uniq2, uniq2.size()) == uniq2);
    EXPECT(to_host(d_total, all.size()) == all);
    std::vector<int64_t> lab2 = to_host(d_lab2, all.size());
    for (size_t i = 0; i < all.size(); ++i) EXPECT(lab2[i] == first2[all[i]]);
  }

  // ---- map layouts chosen from the keys: id range, direct table, rank bitmap ----
  {
    const int64_t m = 50000;
    std::vector<int64_t> rk(m), rv(m), dk(m), dv(m), bk(m), bv(m);
    for (int64_t i = 0; i < m; ++i) {
      rk[i] = 700 + i;       // ids 700 .. 50,699 -> slot id - 700: a range
      rv[i] = i;
      dk[i] = 3 * i + 5;     // every third id: a direct table over the id universe
      dv[i] = m - 1 - i;
      bk[i] = 7 * i + 3 + (i % 5);  // ascending ids with consecutive slots from 11 on: ranks
      bv[i] = 11 + i;
    }
    struct Case { std::vector<int64_t> *k, *v; int kind; } cases[3] = {{&rk, &rv, SHMT_MAP_RANGE}, {&dk, &dv, SHMT_MAP_DIRECT}, {&bk, &bv, SHMT_MAP_RANK}};
    const int64_t sbytes = shmt_hashmap_plan_scratch_bytes(m);
    void *d_ps = nullptr;
    HIP_OK(hipMalloc(&d_ps, sbytes));
    for (const Case &c : cases) {
      int64_t *dk_ = to_device(*c.k), *dv_ = to_device(*c.v);
      shmt_hashmap_layout lay;
      SHMT_OK_(shmt_hashmap_plan(dk_, dv_, m, 8, 8, 0.8, d_ps, sbytes, &lay, stream));
      EXPECT(lay.kind == c.kind);
      void *d_t = nullptr;
      HIP_OK(hipMalloc(&d_t, lay.table_bytes));
      shmt_hashmap_t *pm = nullptr;
      SHMT_OK_(shmt_hashmap_create_planned(&pm, &lay, dk_, dv_, m, 8, 8, 0.8, d_t, lay.table_bytes, stream));
      EXPECT(shmt_hashmap_kind(pm) == c.kind);
      std::vector<int64_t> rq(100001);
      for (auto &x : rq) x = static_cast<int64_t>(rnd() % 400000) - 100;
      int64_t *d_rq = to_device(rq), *d_rr = nullptr;
      HIP_OK(hipMalloc(&d_rr, rq.size() * 8));
      SHMT_OK_(shmt_hashmap_query(pm, d_rq, 8, static_cast<int64_t>(rq.size()), d_rr, stream));
      HIP_OK(hipStreamSynchronize(stream));
      std::unordered_map<int64_t, int64_t> t;
      for (int64_t i = 0; i < m; ++i) t[(*c.k)[i]] = (*c.v)[i];
      std::vector<int64_t> rr = to_host(d_rr, rq.size());
      for (size_t i = 0; i < rq.size(); ++i) {
        auto it = t.find(rq[i]);
        EXPECT(rr[i] == (it == t.end() ? -1 : it->second));
      }
      shmt_hashmap_destroy(pm);
      HIP_OK(hipFree(d_t));
      HIP_OK(hipFree(d_rq));
      HIP_OK(hipFree(d_rr));
      HIP_OK(hipFree(dk_));
      HIP_OK(hipFree(dv_));
    }
    HIP_OK(hipFree(d_ps));
  }

  // ---- scan without a workspace argument: 3,000,001 int64, then a shorter int32 array ----
  {
    const int64_t l1 = 3000001, l2 = 70001;
    std::vector<int64_t> b1(l1);
    for (auto &x : b1) x = static_cast<int64_t>(rnd() >> 8);
    std::vector<int32_t> b2(l2);
    for (auto &x : b2) x = static_cast<int32_t>(rnd() % 77);
    int64_t *d_b1 = to_device(b1);
    int32_t *d_b2 = to_device(b2);
    SHMT_OK_(shmt_exclusive_scan_noalloc(nullptr, 0, 8, stream));     // set-up call
    SHMT_OK_(shmt_exclusive_scan_noalloc(d_b1, l1, 8, stream));
    SHMT_OK_(shmt_exclusive_scan_noalloc(d_b2, l2, 4, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int64_t> s1 = to_host(d_b1, l1);
    uint64_t r1 = 0;
    for (int64_t i = 0; i < l1; ++i) {
      EXPECT(static_cast<uint64_t>(s1[i]) == r1);
      r1 += static_cast<uint64_t>(b1[i]);
    }
    std::vector<int32_t> s2 = to_host(d_b2, l2);
    uint32_t r2 = 0;
    for (int64_t i = 0; i < l2; ++i) {
      EXPECT(static_cast<uint32_t>(s2[i]) == r2);
      r2 += static_cast<uint32_t>(b2[i]);
    }
    EXPECT(shmt_exclusive_scan_noalloc(d_b1, SHMT_SCAN_NOALLOC_MAX_LEN + 1, 8, stream) == SHMT_EINVAL);
  }

  // ---- scans on a workspace that is cleared once and then kept: no clearing launch, left all zero ----
  {
    const int64_t l1 = 2500003, l2 = 900001;
    std::vector<int64_t> b1(l1);
    for (auto &x : b1) x = static_cast<int64_t>(rnd() >> 8);
    std::vector<uint32_t> b2(l2);
    for (auto &x : b2) x = static_cast<uint32_t>(rnd() % 1000);
    int64_t *d_b1 = to_device(b1);
    uint32_t *d_b2 = to_device(b2);
    const int64_t wbytes = std::max(shmt_scan_tmp_bytes(l1), shmt_scan_tmp_bytes(l2));
    char *d_ws = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_ws), wbytes));
    HIP_OK(hipMemsetAsync(d_ws, 0xEE, wbytes, stream));
    SHMT_OK_(shmt_scan_workspace_clear(d_ws, wbytes, stream));
    SHMT_OK_(shmt_exclusive_scan_kept(d_b1, l1, 8, d_ws, wbytes, stream));
    SHMT_OK_(shmt_inclusive_scan_i32_kept(d_b2, l2, d_ws, wbytes, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int64_t> s1 = to_host(d_b1, l1);
    uint64_t r1 = 0;
    for (int64_t i = 0; i < l1; ++i) {
      EXPECT(static_cast<uint64_t>(s1[i]) == r1);
      r1 += static_cast<uint64_t>(b1[i]);
    }
    std::vector<uint32_t> s2 = to_host(d_b2, l2);
    uint32_t r2 = 0;
    for (int64_t i = 0; i < l2; ++i) {
      r2 += b2[i];
      EXPECT(s2[i] == r2);
    }
    for (char c : to_host(d_ws, wbytes)) EXPECT(c == 0);
    HIP_OK(hipFree(d_ws));
    HIP_OK(hipFree(d_b1));
    HIP_OK(hipFree(d_b2));
  }

  // ---- the error word of bounded waits, set from the host: read-and-clear, and its pinned mirror ----
  {
    int code = -1;
    SHMT_OK_(shmt_async_error(&code));
    EXPECT(code == 0);
    uint32_t *h_word = nullptr;
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&h_word), 4, hipHostMallocDefault));
    void *word_alias = nullptr;
    SHMT_OK_(shmt_host_devptr(h_word, &word_alias));
    *h_word = 0xFFFFFFFFu;
    SHMT_OK_(shmt_async_error_mirror(h_word, word_alias));
    EXPECT(*h_word == 0);
    EXPECT(shmt_async_error_mirror(h_word, nullptr) == SHMT_EINVAL);
    SHMT_OK_(shmt_async_error_inject(1));
    EXPECT(*static_cast<volatile uint32_t *>(h_word) != 0);
    SHMT_OK_(shmt_async_error(&code));
    EXPECT(code == 1 && strstr(shmt_last_error(), "look-back of a device-wide scan") != nullptr);
    EXPECT(*static_cast<volatile uint32_t *>(h_word) == 0);
    SHMT_OK_(shmt_async_error(&code));
    EXPECT(code == 0);
    SHMT_OK_(shmt_async_error_mirror(nullptr, nullptr));   // withdrawn before the word is freed
    HIP_OK(hipHostFree(h_word));
    // a kernel that only passes time (the probe for streams that run side by side)
    SHMT_OK_(shmt_busy_wait(stream, 50));
    HIP_OK(hipStreamSynchronize(stream));
  }

  // ---- coordinate form: destination position of every sampled id, from a hop job and from sub_indptr ----
  {
    const int64_t S = 7, k = 5, n_max = S + S * k;
    int64_t *d_sp = nullptr, *d_sub3 = nullptr, *d_total = nullptr, *d_uniq = nullptr, *d_lab = nullptr;
    int64_t *d_coo = nullptr, *d_rows = nullptr, *h_sizes = nullptr;
    void *d_plan3 = nullptr, *d_scr = nullptr;
    HIP_OK(hipMalloc(&d_sp, (S + 1) * 8));
    HIP_OK(hipMalloc(&d_sub3, S * k * 8));
    HIP_OK(hipMalloc(&d_total, n_max * 8));
    HIP_OK(hipMalloc(&d_uniq, n_max * 8));
    HIP_OK(hipMalloc(&d_lab, n_max * 8));
    HIP_OK(hipMalloc(&d_coo, S * k * 8));
    HIP_OK(hipMalloc(&d_rows, S * k * 8));
    HIP_OK(hipMalloc(&d_plan3, pbytes));
    const int64_t sb3 = shmt_relabel_scratch_bytes(n_max);
    HIP_OK(hipMalloc(&d_scr, sb3));
    HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&h_sizes), 16, hipHostMallocDefault));
    shmt_hop_job job = {};
    job.indptr = d_indptr; job.ptr_bytes = 8; job.indices = d_indices; job.idx_bytes = 8;
    job.seeds = d_seeds; job.seed_bytes = 8; job.max_seeds = S; job.k = k; job.replace = 0;
    job.rng_seed = 7777; job.rng_stream = 0;
    job.sub_indptr = d_sp; job.sub_indices = d_sub3; job.plan = d_plan3; job.plan_bytes = pbytes;
    job.elem_bytes = 8; job.total_out = d_total; job.scratch = d_scr; job.scratch_bytes = sb3;
    job.unique_out = d_uniq; job.labels_out = d_lab; job.nnz_out = h_sizes; job.count_out = h_sizes + 1;
    job.coo_dst = d_coo; job.coo_bytes = 8;
    SHMT_OK_(shmt_sample_hops_chained(&job, 1, stream));
    HIP_OK(hipStreamSynchronize(stream));
    EXPECT(h_sizes[0] == 25);
    SHMT_OK_(shmt_csr_rows(d_sp, 8, S, h_sizes[0], d_rows, 8, stream));
    HIP_OK(hipStreamSynchronize(stream));
    const std::vector<int64_t> want = {0, 2, 2, 2, 2, 3, 3, 3, 3, 3, 4, 4, 4, 4, 4, 5, 5, 5, 5, 5, 6, 6, 6, 6, 6};
    EXPECT(to_host(d_coo, 25) == want);
    EXPECT(to_host(d_rows, 25) == want);
  }

  shmt_hashmap_destroy(map);
  shmt_hashmap_destroy(fmap);
  printf("cabi_smoke: all checks passed\n");
  return 0;
}
