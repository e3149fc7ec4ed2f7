/*
 * oracle.c — CPU restatement of the ShmTensor GPU-cache hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the product (shmtensor_amd/, libshmt.so,
 * ShmTensorLib) links, imports or calls this file. It is used by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, as the
 * checker and as the timed CPU baseline, never as the thing shipped.
 *
 * Each function restates, sequentially (or with OpenMP threads standing in for
 * CUDA threads), what the cited reference code computes. file:line citations
 * are relative to the ShmTensor source tree.
 *
 * Third-party algorithm not present in the reference tree: the static hashmap
 * is NVIDIA/cuCollections `cuco::static_map` (fetched at configure time,
 * GIT_TAG dev, i.e. no pinned version: CMakeLists.txt:46-54), instantiated
 * with linear_probing<1, default_hash_function<Key>>, storage<1>, empty key
 * -1, empty value -1 (include/cuco_hashmap.cuh:52-67). Its published
 * algorithm is open addressing with linear probing: insert claims the first
 * empty slot on the probe sequence with a compare-and-swap, find walks the
 * same sequence until it meets the key or an empty slot. That is what
 * orc_map_* does. cuco's hash function and capacity rounding cannot be
 * observed through the reference API (results depend only on the key set),
 * so a 64-bit mixer is used here.
 *
 * Pinning status (see tests/test_oracle.py):
 *   hashmap query        pinned by brute force / Python dict
 *   fetch / set          pinned by numpy fancy indexing and sequential loops
 *   exclusive scan       pinned by numpy cumsum incl. wraparound
 *   relabel              pinned by the reference KAT and dict.setdefault
 *   sub-CSR              pinned by the reference KAT and numpy concat
 *   sample counts/copy   pinned by the reference KAT (sub_indptr, deg <= k)
 *   sample deg > k       distribution only (chi-square vs the uniform law);
 *                        the reference's exact cuRAND stream is unpinned
 *   philox4x32-10        pinned by the Random123 known-answer vectors
 *   thrust_scan          parity unpinned: the reference body is a data race
 *                        (src/thrust_scan.cu:13-16); program order is used
 *   memory_usage()       parity unpinned (cuco-internal allocation sizes)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* helpers                                                              */

static inline int64_t ld(const void *p, int64_t i, int bytes) {
  return bytes == 8 ? ((const int64_t *)p)[i] : (int64_t)((const int32_t *)p)[i];
}
static inline void st(void *p, int64_t i, int bytes, int64_t v) {
  if (bytes == 8)
    ((int64_t *)p)[i] = v;
  else
    ((int32_t *)p)[i] = (int32_t)v;
}

static inline uint64_t mix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

ORC_EXPORT int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORC_EXPORT void orc_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ------------------------------------------------------------------ */
/* Static hashmap: include/cuco_hashmap.cuh:57-87, src/cuco_hashmap.cu:24-34 */

typedef struct {
  int64_t *keys;
  int64_t *vals;
  int64_t cap;       /* slots actually allocated                        */
  int64_t capacity;  /* what capacity() reports: ceil(n / load_factor)   */
  int key_bytes, val_bytes;
} orc_map;

/* capacity_ = std::ceil(numel / load_factor), include/cuco_hashmap.cuh:62,75 */
ORC_EXPORT int64_t orc_map_capacity(int64_t n, double lf) { return (int64_t)ceil((double)n / lf); }

/* Narrow a request to the key dtype: requests.to(key_type_), src/cuco_hashmap.cu:29 */
static inline int64_t to_key(int64_t r, int key_bytes) {
  return key_bytes == 4 ? (int64_t)(int32_t)r : r;
}

ORC_EXPORT orc_map *orc_map_build(const void *keys, const void *vals, int64_t n, int key_bytes,
                                  int val_bytes, double lf) {
  orc_map *m = (orc_map *)calloc(1, sizeof(orc_map));
  m->capacity = orc_map_capacity(n, lf);
  m->cap = m->capacity > n ? m->capacity : n + 1; /* keep one empty slot so find terminates */
  if (m->cap < 1) m->cap = 1;
  m->key_bytes = key_bytes;
  m->val_bytes = val_bytes;
  m->keys = (int64_t *)malloc(sizeof(int64_t) * (size_t)m->cap);
  m->vals = (int64_t *)malloc(sizeof(int64_t) * (size_t)m->cap);
  for (int64_t i = 0; i < m->cap; ++i) { /* empty_key{-1}, empty_value{-1}: cuco_hashmap.cuh:58-59 */
    m->keys[i] = -1;
    m->vals[i] = -1;
  }
  for (int64_t i = 0; i < n; ++i) { /* map_->insert(zipped, zipped + numel): cuco_hashmap.cuh:68-70 */
    int64_t k = ld(keys, i, key_bytes);
    if (k == -1) continue; /* sentinel cannot be stored */
    int64_t pos = (int64_t)(mix64((uint64_t)k) % (uint64_t)m->cap);
    for (;;) {
      if (m->keys[pos] == -1) {
        m->keys[pos] = k;
        m->vals[pos] = ld(vals, i, val_bytes);
        break;
      }
      if (m->keys[pos] == k) break; /* duplicate key: first insert wins */
      pos = pos + 1 == m->cap ? 0 : pos + 1;
    }
  }
  return m;
}

static inline int64_t map_find(const orc_map *m, int64_t k) {
  if (k == -1) return -1;
  int64_t pos = (int64_t)(mix64((uint64_t)k) % (uint64_t)m->cap);
  for (int64_t probes = 0; probes < m->cap; ++probes) {
    if (m->keys[pos] == k) return m->vals[pos];
    if (m->keys[pos] == -1) return -1;
    pos = pos + 1 == m->cap ? 0 : pos + 1;
  }
  return -1;
}

/* result = full_like(requests, -1); map_->find(...): cuco_hashmap.cuh:81-87 */
ORC_EXPORT void orc_map_query(const orc_map *m, const void *req, int req_bytes, int64_t n, void *out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i)
    st(out, i, m->val_bytes, map_find(m, to_key(ld(req, i, req_bytes), m->key_bytes)));
}

ORC_EXPORT int64_t orc_map_reported_capacity(const orc_map *m) { return m->capacity; }

ORC_EXPORT void orc_map_free(orc_map *m) {
  if (!m) return;
  free(m->keys);
  free(m->vals);
  free(m);
}

/* ------------------------------------------------------------------ */
/* Feature fetch / set.
 * Routing rule: src/cache_feature_fetch.cu:117-127 (hashmap), :213-222 (mask),
 * :37-44 (uva); src/cache_feature_set.cu:104-114, :196-205, :28-35.
 * mode 0: no cache (slot = -1); mode 1: slot = map.find(idx); mode 2: slot = mask[i]. */

static inline int64_t route(int mode, const orc_map *m, const void *mask, int mask_bytes, int64_t i,
                            int64_t idx) {
  if (mode == 1) return map_find(m, to_key(idx, m->key_bytes));
  if (mode == 2) return ld(mask, i, mask_bytes);
  return -1;
}

ORC_EXPORT void orc_fetch(const char *host, const char *gpu, const void *indices, int idx_bytes,
                          int mode, const orc_map *m, const void *mask, int mask_bytes, char *out,
                          int64_t Q, int64_t row_bytes) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < Q; ++i) {
    int64_t idx = ld(indices, i, idx_bytes);
    int64_t slot = route(mode, m, mask, mask_bytes, i, idx);
    const char *src = slot >= 0 ? gpu + slot * row_bytes : host + idx * row_bytes;
    memcpy(out + i * row_bytes, src, (size_t)row_bytes);
  }
}

/* Sequential on purpose: duplicate indices then have the defined outcome
 * "last writer wins", a superset of what the (racy) reference guarantees. */
ORC_EXPORT void orc_set(char *host, char *gpu, const void *indices, int idx_bytes, int mode,
                        const orc_map *m, const void *mask, int mask_bytes, const char *update,
                        int64_t Q, int64_t row_bytes) {
  for (int64_t i = 0; i < Q; ++i) {
    int64_t idx = ld(indices, i, idx_bytes);
    int64_t slot = route(mode, m, mask, mask_bytes, i, idx);
    char *dst = slot >= 0 ? gpu + slot * row_bytes : host + idx * row_bytes;
    memcpy(dst, update + i * row_bytes, (size_t)row_bytes); /* a hit leaves the host row stale */
  }
}

/* ------------------------------------------------------------------ */
/* Scans. cub_exclusiveSum: src/tensor_relabel.cu:11-26 (in place, len = n+1,
 * last input ignored). thrust_scan: src/thrust_scan.cu:9-18 in program order. */

ORC_EXPORT void orc_exclusive_scan(void *data, int64_t len, int bytes) {
  if (bytes == 8) {
    uint64_t run = 0, *p = (uint64_t *)data;
    for (int64_t i = 0; i < len; ++i) {
      uint64_t v = p[i];
      p[i] = run;
      run += v;
    }
  } else {
    uint32_t run = 0, *p = (uint32_t *)data;
    for (int64_t i = 0; i < len; ++i) {
      uint32_t v = p[i];
      p[i] = run;
      run += v;
    }
  }
}

ORC_EXPORT void orc_inclusive_scan_i32(int32_t *p, int64_t n) {
  for (int64_t i = 1; i < n; ++i) p[i] = (int32_t)((uint32_t)p[i] + (uint32_t)p[i - 1]);
}

/* ------------------------------------------------------------------ */
/* Relabel: src/tensor_relabel.cu:125-209, OpenMP threads in the role of the
 * CUDA threads, same four passes, same table (RelabelHashmap :68-123):
 * capacity 1 << (floor(log2 N) + 1) (:139), hash = key & (cap-1) (:111-117),
 * probe pos = hash(pos + delta), delta++ (:80-81), CAS on the key, atomicMin
 * on the first index.                                                   */

static inline uint32_t rl_hash(int64_t key, uint32_t cap) { return (uint32_t)((uint64_t)key & (cap - 1)); }

static uint32_t rl_search(const int64_t *kt, uint32_t cap, int64_t key) {
  uint32_t delta = 1, pos = rl_hash(key, cap);
  for (;;) {
    if (kt[pos] == key) return pos;
    pos = rl_hash((int64_t)(pos + delta), cap);
    delta += 1;
  }
}

/* total: N int64 values; unique: room for N; labels: N. Returns the number of
 * distinct values. */
ORC_EXPORT int64_t orc_relabel(const int64_t *total, int64_t N, int64_t *unique, int64_t *labels) {
  if (N == 0) return 0;
  uint32_t cap = 1u << ((uint32_t)floor(log2((double)N)) + 1);
  int64_t *kt = (int64_t *)malloc(sizeof(int64_t) * cap);
  int64_t *it = (int64_t *)malloc(sizeof(int64_t) * cap);
  int64_t *vt = (int64_t *)malloc(sizeof(int64_t) * cap);
  int64_t *prefix = (int64_t *)malloc(sizeof(int64_t) * (size_t)(N + 1));
  for (uint32_t i = 0; i < cap; ++i) { /* torch::full(-1) / torch::full(MAX): :141-144 */
    kt[i] = -1;
    it[i] = INT64_MAX;
  }
  /* pass 1, Update(in[i], i): :147-154 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    int64_t key = total[i];
    uint32_t delta = 1, pos = rl_hash(key, cap);
    for (;;) {
      int64_t expected = -1;
      if (__atomic_compare_exchange_n(&kt[pos], &expected, key, 0, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST) ||
          expected == key)
        break;
      pos = rl_hash((int64_t)(pos + delta), cap);
      delta += 1;
    }
    int64_t cur = __atomic_load_n(&it[pos], __ATOMIC_SEQ_CST);
    while (i < cur && !__atomic_compare_exchange_n(&it[pos], &cur, i, 0, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {
    }
  }
  /* pass 2, count[i] = SearchForValue(in[i]) == i: :161-169, then exclusive sum :170 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) prefix[i] = it[rl_search(kt, cap, total[i])] == i ? 1 : 0;
  prefix[N] = 0;
  orc_exclusive_scan(prefix, N + 1, 8);
  int64_t tot = prefix[N]; /* :173 */
  /* pass 3, unique[prefix[i]] = in[i]; value[pos] = prefix[i]: :178-192 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    uint32_t pos = rl_search(kt, cap, total[i]);
    if (it[pos] == i) {
      unique[prefix[i]] = total[i];
      vt[pos] = prefix[i];
    }
  }
  /* pass 4, out[i] = SearchForValue(in[i]) on the value table: :196-203 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) labels[i] = vt[rl_search(kt, cap, total[i])];
  free(kt);
  free(it);
  free(vt);
  free(prefix);
  return tot;
}

/* The same contract as a CPU programmer would write it (not a restatement of
 * the reference's kernel structure; used as the faster of the two CPU
 * baselines): one sequential sweep, open addressing with a mixed hash, a new
 * id is appended to `unique` the first time it is met. First-occurrence order
 * falls out of the sweep order, so no index table, no counting pass and no
 * scan are needed (src/tensor_relabel.cu:127-130, 206-208 for the contract).
 * The table is kept between calls and emptied by the slots a call used. Not
 * re-entrant. */
static int64_t *g_sw_key = NULL, *g_sw_val = NULL; /* kept between calls, emptied by the slots a call used */
static uint64_t *g_sw_used = NULL;
static uint64_t g_sw_cap = 0;

ORC_EXPORT int64_t orc_relabel_sweep(const int64_t *total, int64_t N, int64_t *unique, int64_t *labels) {
  if (N == 0) return 0;
  uint64_t cap = 16;
  while (cap < (uint64_t)N * 2) cap <<= 1;
  if (cap > g_sw_cap) {
    free(g_sw_key);
    free(g_sw_val);
    free(g_sw_used);
    g_sw_key = (int64_t *)malloc(sizeof(int64_t) * cap);
    g_sw_val = (int64_t *)malloc(sizeof(int64_t) * cap);
    g_sw_used = (uint64_t *)malloc(sizeof(uint64_t) * (cap / 2));
    g_sw_cap = cap;
    memset(g_sw_key, 0xff, sizeof(int64_t) * cap); /* -1: empty */
  }
  int64_t *const kt = g_sw_key, *const vt = g_sw_val;
  const uint64_t mask = g_sw_cap - 1;
  int64_t count = 0;
  for (int64_t i = 0; i < N; ++i) {
    const int64_t key = total[i];
    uint64_t pos = mix64((uint64_t)key) & mask;
    while (kt[pos] != -1 && kt[pos] != key) pos = (pos + 1) & mask;
    if (kt[pos] == -1) {
      kt[pos] = key;
      vt[pos] = count;
      g_sw_used[count] = pos;
      unique[count++] = key;
    }
    labels[i] = vt[pos];
  }
  for (int64_t u = 0; u < count; ++u) kt[g_sw_used[u]] = -1;
  return count;
}

/* The same contract on all host cores (the tuned CPU baseline of bench.py, not
 * a restatement of the reference's kernel structure), without atomics: ids are dealt to one
 * partition per thread by the top bits of their mixed hash, each partition in
 * index order (a counting pass and a scatter pass over the threads' chunks),
 * every thread then sweeps ITS partition with a private table exactly as
 * orc_relabel_sweep does (first occurrences fall out of the index order), the
 * first-occurrence flags are ranked by a two-level prefix sum, and a last pass
 * maps every element's first index to its rank. All tables and buffers are
 * kept between calls. Small inputs take the sequential sweep, which wins there.
 * Not re-entrant. Contract: src/tensor_relabel.cu:127-130, 206-208. */
typedef struct {
  uint32_t *items;  /* indices dealt to the partitions, partition after partition */
  uint32_t *first;  /* per element: index of the first occurrence of its id */
  uint32_t *rank;   /* per index: number of first occurrences before it */
  int64_t items_cap;
  uint64_t *key;    /* private tables, one region per thread */
  uint32_t *val;
  uint64_t table_cap; /* slots per thread */
  int threads;
} RlPartState;
static RlPartState g_part = {0};

ORC_EXPORT int64_t orc_relabel_parallel(const int64_t *total, int64_t N, int64_t *unique, int64_t *labels) {
  if (N < 16384 || N >= ((int64_t)1 << 31)) return orc_relabel_sweep(total, N, unique, labels);
  const int T = omp_get_max_threads();
  int shift = 64;
  int parts = 1;
  while (parts < T) { parts <<= 1; --shift; } /* partitions: power of two >= threads, dealt round-robin */
  RlPartState *g = &g_part;
  if (N > g->items_cap) {
    free(g->items); free(g->first); free(g->rank);
    g->items = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)N);
    g->first = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)N);
    g->rank = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)(N + 1));
    g->items_cap = N;
  }
  /* a partition holds N / parts ids on average; tables sized for four times that (load <= 0.5 at twice the mean) */
  uint64_t want = 1024;
  while (want < (uint64_t)(N / parts + 1) * 4) want <<= 1;
  if (want > g->table_cap || parts != g->threads) {
    free(g->key); free(g->val);
    g->key = (uint64_t *)malloc(sizeof(uint64_t) * want * (size_t)parts);
    g->val = (uint32_t *)malloc(sizeof(uint32_t) * want * (size_t)parts);
    g->table_cap = want;
    g->threads = parts;
    memset(g->key, 0xff, sizeof(uint64_t) * want * (size_t)parts);
  }
  int64_t *counts = (int64_t *)calloc((size_t)T * parts + 1, sizeof(int64_t)); /* [thread][partition] */
  int64_t *starts = (int64_t *)calloc((size_t)parts + 1, sizeof(int64_t));
  int64_t *firsts = (int64_t *)calloc((size_t)T + 1, sizeof(int64_t));
  int overflow = 0;
  int64_t tot = 0;
#pragma omp parallel num_threads(T)
  {
    const int t = omp_get_thread_num();
    const int64_t lo = N * t / T, hi = N * (t + 1) / T;
    int64_t *mine = counts + (size_t)t * parts;
    for (int64_t i = lo; i < hi; ++i) mine[parts == 1 ? 0 : (mix64((uint64_t)total[i]) >> shift)]++;
#pragma omp barrier
#pragma omp single
    {
      /* partition p holds the ids of thread 0's chunk first, then thread 1's, ...: index order */
      int64_t run = 0;
      for (int p = 0; p < parts; ++p) {
        starts[p] = run;
        for (int k = 0; k < T; ++k) {
          const int64_t c = counts[(size_t)k * parts + p];
          counts[(size_t)k * parts + p] = run;
          run += c;
        }
      }
      starts[parts] = run;
      for (int p = 0; p < parts; ++p)
        if ((uint64_t)(starts[p + 1] - starts[p]) * 2 > g->table_cap) overflow = 1; /* a very uneven deal */
    }
    if (!overflow) {
      for (int64_t i = lo; i < hi; ++i)
        g->items[mine[parts == 1 ? 0 : (mix64((uint64_t)total[i]) >> shift)]++] = (uint32_t)i;
#pragma omp barrier
      /* sweep the partitions (round-robin over the threads), each with its own table */
      int64_t nfirst = 0;
      for (int p = t; p < parts; p += T) {
        uint64_t *kt = g->key + (size_t)p * g->table_cap;
        uint32_t *vt = g->val + (size_t)p * g->table_cap;
        const uint64_t mask = g->table_cap - 1;
        for (int64_t e = starts[p]; e < starts[p + 1]; ++e) {
          const uint32_t i = g->items[e];
          const uint64_t key = (uint64_t)total[i];
          uint64_t pos = (mix64(key) * 0x9E3779B97F4A7C15ull >> 20) & mask; /* independent of the partition bits */
          while (kt[pos] != ~0ull && kt[pos] != key) pos = (pos + 1) & mask;
          if (kt[pos] == ~0ull && key != ~0ull) {
            kt[pos] = key;
            vt[pos] = i;
          }
          g->first[i] = kt[pos] == key ? vt[pos] : i;
          g->rank[e] = (uint32_t)pos; /* scratch until the ranks are written: the slot this element used */
        }
        /* leave the table empty: only the slots used (by remembered position: emptying while probing
         * would cut the chains of the ids still to be found) */
        for (int64_t e = starts[p]; e < starts[p + 1]; ++e) kt[g->rank[e]] = ~0ull;
      }
#pragma omp barrier
      for (int64_t i = lo; i < hi; ++i) nfirst += g->first[i] == (uint32_t)i;
      firsts[t + 1] = nfirst;
#pragma omp barrier
#pragma omp single
      {
        for (int k = 0; k < T; ++k) firsts[k + 1] += firsts[k];
        tot = firsts[T];
      }
      int64_t r = firsts[t];
      for (int64_t i = lo; i < hi; ++i) {
        g->rank[i] = (uint32_t)r;
        if (g->first[i] == (uint32_t)i) unique[r++] = total[i];
      }
#pragma omp barrier
      for (int64_t i = lo; i < hi; ++i) labels[i] = (int64_t)g->rank[g->first[i]];
    }
  }
  free(counts);
  free(starts);
  free(firsts);
  if (overflow) return orc_relabel_sweep(total, N, unique, labels);
  return tot;
}

/* ------------------------------------------------------------------ */
/* Philox4x32-10 (Random123), the generator of the new sampler. The reference
 * uses cuRAND's Philox4_32_10 state (src/cache_graph_sampling.cu:105-107),
 * whose stream (seed 7777 + lane, subsequence thread id) is not reproduced. */

ORC_EXPORT void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0;
  out[1] = c1;
  out[2] = c2;
  out[3] = c3;
}

static inline uint64_t draw(uint64_t seed, uint32_t stream, int64_t node, uint32_t j, uint64_t range) {
  uint32_t ctr[4] = {(uint32_t)(uint64_t)node, (uint32_t)((uint64_t)node >> 32), j, stream};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t o[4];
  orc_philox4x32_10(ctr, key, o);
  uint64_t bits = ((uint64_t)o[1] << 32) | o[0];
  return (uint64_t)(((unsigned __int128)bits * range) >> 64);
}

/* ------------------------------------------------------------------ */
/* Neighbour sampling: src/cache_graph_sampling.cu.
 * Sizes: GetSubIndptr :47-89 / GetSubIndptrWithCache :222-289.
 * Selection: CSRWiseSampleUniformKernel :91-146 (Algorithm R; the kernel's
 * atomicMax reproduces "the replacement order the serial algorithm would
 * have", :131-135, so the serial algorithm is what is written here),
 * CSRWiseSampleUniformReplaceKernel :148-177.
 * All arrays int64 here; cache may be NULL (m == NULL).                  */

static inline void adjacency(const int64_t *indptr, const int64_t *indices, const int64_t *gpu_indptr,
                             const int64_t *gpu_indices, const orc_map *m, int64_t v,
                             const int64_t **adj, int64_t *deg) {
  int64_t slot = m ? map_find(m, to_key(v, m->key_bytes)) : -1; /* :258-268 */
  if (slot >= 0) {
    *adj = gpu_indices + gpu_indptr[slot];
    *deg = gpu_indptr[slot + 1] - gpu_indptr[slot];
  } else {
    *adj = indices + indptr[v];
    *deg = indptr[v + 1] - indptr[v];
  }
}

ORC_EXPORT int64_t orc_sample_counts(const int64_t *indptr, const int64_t *indices,
                                     const int64_t *gpu_indptr, const int64_t *gpu_indices,
                                     const orc_map *m, const int64_t *seeds, int64_t S, int64_t k,
                                     int replace, int64_t *sub_indptr) {
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    const int64_t *adj;
    int64_t deg;
    adjacency(indptr, indices, gpu_indptr, gpu_indices, m, seeds[s], &adj, &deg);
    sub_indptr[s] = replace ? (deg == 0 ? 0 : k) : (deg < k ? deg : k); /* :76-80 */
  }
  sub_indptr[S] = 0;
  orc_exclusive_scan(sub_indptr, S + 1, 8); /* :83-84 */
  return sub_indptr[S];
}

/* algo 0: Algorithm R as in the reference (own RNG stream);
 * algo 1: Floyd's subset algorithm with the draw schedule of the HIP kernel
 *         (mirrors the device selection rule bit for bit; pins the
 *         implementation, not the reference).                            */
ORC_EXPORT void orc_sample_fill(const int64_t *indptr, const int64_t *indices,
                                const int64_t *gpu_indptr, const int64_t *gpu_indices,
                                const orc_map *m, const int64_t *seeds, int64_t S, int64_t k,
                                int replace, const int64_t *sub_indptr, int64_t *out, uint64_t seed,
                                uint32_t stream, int algo) {
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t s = 0; s < S; ++s) {
    const int64_t *adj;
    int64_t deg;
    const int64_t v = seeds[s];
    adjacency(indptr, indices, gpu_indptr, gpu_indices, m, v, &adj, &deg);
    int64_t *o = out + sub_indptr[s];
    if (replace) { /* :168-175 */
      if (deg > 0)
        for (int64_t j = 0; j < k; ++j) o[j] = adj[draw(seed, stream, v, (uint32_t)j, (uint64_t)deg)];
    } else if (deg <= k) { /* just copy: :116-120 */
      for (int64_t j = 0; j < deg; ++j) o[j] = adj[j];
    } else if (algo == 0) { /* reservoir: :122-143 */
      for (int64_t j = 0; j < k; ++j) o[j] = j;
      for (int64_t i = k; i < deg; ++i) {
        int64_t num = (int64_t)draw(seed, stream ^ 0x5bd1e995u, v * 1315423911ll + s, (uint32_t)i, (uint64_t)(i + 1));
        if (num < k) o[num] = i;
      }
      for (int64_t j = 0; j < k; ++j) o[j] = adj[o[j]];
    } else { /* Floyd */
      for (int64_t step = 0; step < k; ++step) {
        int64_t J = deg - k + step;
        int64_t t = (int64_t)draw(seed, stream, v, (uint32_t)step, (uint64_t)(J + 1));
        int taken = 0;
        for (int64_t q = 0; q < step; ++q) taken |= (o[q] == t);
        o[step] = taken ? J : t;
      }
      for (int64_t j = 0; j < k; ++j) o[j] = adj[o[j]];
    }
  }
}

/* CreateCacheCSR: src/cache_graph_sampling.cu:455-492 */
ORC_EXPORT int64_t orc_subcsr_counts(const int64_t *indptr, const int64_t *seeds, int64_t C,
                                     int64_t *gpu_indptr) {
  for (int64_t i = 0; i < C; ++i) gpu_indptr[i] = indptr[seeds[i] + 1] - indptr[seeds[i]]; /* :470-477 */
  gpu_indptr[C] = 0;
  orc_exclusive_scan(gpu_indptr, C + 1, 8);
  return gpu_indptr[C];
}

ORC_EXPORT void orc_subcsr_copy(const int64_t *indptr, const int64_t *indices, const int64_t *seeds,
                                int64_t C, const int64_t *gpu_indptr, int64_t *gpu_indices) {
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < C; ++i) { /* CSRIndicesCopyKernel: :440-451 */
    int64_t begin = indptr[seeds[i]], deg = indptr[seeds[i] + 1] - begin;
    memcpy(gpu_indices + gpu_indptr[i], indices + begin, sizeof(int64_t) * (size_t)deg);
  }
}
