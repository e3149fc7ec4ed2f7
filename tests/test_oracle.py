"""Pins the CPU oracle (oracle/oracle.c) before anything is compared with it:
the reference's own known-answer vectors, closed forms from numpy / Python
containers, brute force on small inputs, and the uniform law for sampling."""
import numpy as np
import pytest

from conftest import load_golden

RNG = np.random.default_rng(1234)
DTYPES = [np.int32, np.int64]


# ---- hashmap ---------------------------------------------------------------

@pytest.mark.parametrize("kd", DTYPES)
@pytest.mark.parametrize("vd", DTYPES)
@pytest.mark.parametrize("lf", [0.1, 0.5, 0.8, 0.99, 1.0])
def test_hashmap_matches_dict(oracle, kd, vd, lf):
    keys = RNG.choice(100000, size=3000, replace=False).astype(kd)
    vals = RNG.integers(0, 2**31 - 1, size=keys.size).astype(vd)
    h = oracle.Hashmap(keys, vals, lf)
    table = dict(zip(keys.tolist(), vals.tolist()))
    req = np.concatenate([keys[:500], RNG.integers(0, 100000, size=2000), [-1, -1]]).astype(np.int64)
    got = h.query(req)
    assert got.dtype == vd
    assert got.tolist() == [table.get(int(r), -1) for r in req]
    assert h.capacity() == int(np.ceil(keys.size / lf))


def test_hashmap_request_narrowing(oracle):
    # requests.to(key dtype): an int64 request whose low 32 bits equal a key of an
    # int32-keyed map hits (two's-complement narrowing), as torch's cast does
    keys = np.array([7, 123456], dtype=np.int32)
    h = oracle.Hashmap(keys, np.array([10, 20], dtype=np.int64), 0.5)
    req = np.array([7, 7 + (1 << 32), 123456 - (1 << 32), 8], dtype=np.int64)
    assert h.query(req).tolist() == [10, 10, 20, -1]
    # int32 requests against int64 keys are sign-extended
    h2 = oracle.Hashmap(np.array([5, 2, 1], dtype=np.int64), np.arange(3), 0.8)
    assert h2.query(np.array([5, 0, 1, 2, 3], dtype=np.int32)).tolist() == [0, -1, 2, 1, -1]


def test_hashmap_single_and_empty(oracle):
    h = oracle.Hashmap(np.array([42]), np.array([0]), 1.0)
    assert h.query(np.array([42, 41])).tolist() == [0, -1]
    h0 = oracle.Hashmap(np.zeros(0, np.int64), np.zeros(0, np.int64), 0.5)
    assert h0.query(np.array([1, 2])).tolist() == [-1, -1]


# ---- fetch / set -----------------------------------------------------------

@pytest.mark.parametrize("shape", [(100,), (100, 7), (50, 4, 5), (64, 128)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8, np.int64])
def test_fetch_is_fancy_indexing(oracle, shape, dtype):
    n = shape[0]
    host = RNG.integers(-100, 100, size=shape).astype(dtype)
    ids = RNG.choice(n, size=n // 3, replace=False)
    # cache rows deliberately differ from the host rows: routing itself is checked
    gpu = (host[ids] + 1).astype(dtype)
    h = oracle.Hashmap(ids, np.arange(ids.size), 0.8)
    q = RNG.integers(0, n, size=300)
    slot = h.query(q)
    expect = np.where((slot >= 0).reshape((-1,) + (1,) * (len(shape) - 1)), gpu[np.maximum(slot, 0)], host[q])
    assert np.array_equal(oracle.fetch(host, gpu, q, hashmap=h), expect)
    assert np.array_equal(oracle.fetch(host, gpu, q.astype(np.int32), mask=slot.astype(np.int32)), expect)
    assert np.array_equal(oracle.fetch(host, None, q), host[q])


def test_set_is_sequential_loop(oracle):
    host = RNG.standard_normal((200, 6)).astype(np.float32)
    ids = RNG.choice(200, size=80, replace=False)
    gpu = host[ids].copy()
    h = oracle.Hashmap(ids, np.arange(ids.size), 0.8)
    q = np.unique(RNG.integers(0, 200, size=120))
    upd = RNG.standard_normal((q.size, 6)).astype(np.float32)
    eh, eg = host.copy(), gpu.copy()
    pos = {int(k): i for i, k in enumerate(ids)}
    for i, v in enumerate(q.tolist()):
        if v in pos:
            eg[pos[v]] = upd[i]      # hit: cache row only, host row left stale
        else:
            eh[v] = upd[i]
    oracle.set_rows(host, gpu, q, upd, hashmap=h)
    assert np.array_equal(host, eh) and np.array_equal(gpu, eg)
    # the reference's own post-condition: fetch after set returns the update
    assert np.array_equal(oracle.fetch(host, gpu, q, hashmap=h), upd)


# ---- scans -------------------------------------------------------------------

@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [0, 1, 2, 63, 64, 65, 1000])
def test_exclusive_scan_is_shifted_cumsum(oracle, dt, n):
    a = RNG.integers(0, 1000, size=n + 1).astype(dt)
    expect = np.concatenate([[0], np.cumsum(a[:-1], dtype=dt)]).astype(dt)[: n + 1]
    assert np.array_equal(oracle.exclusive_scan(a), expect)


def test_scan_wraparound(oracle):
    a = np.array([2**31 - 1, 1, 5, 0], dtype=np.int32)
    assert oracle.exclusive_scan(a).tolist() == [0, 2**31 - 1, -2**31, -2**31 + 5]
    assert oracle.inclusive_scan_i32(a).tolist() == [2**31 - 1, -2**31, -2**31 + 5, -2**31 + 5]
    b = np.array([2**63 - 1, 2, 0], dtype=np.int64)
    assert oracle.exclusive_scan(b).tolist() == [0, 2**63 - 1, -2**63 + 1]


# ---- relabel -------------------------------------------------------------------

def _relabel_closed_form(arrays):
    total = np.concatenate(arrays).tolist()
    first = {}
    for x in total:
        first.setdefault(x, len(first))
    return list(first.keys()), [first[x] for x in total]


@pytest.mark.parametrize("algo", ["passes", "sweep", "parallel"])
def test_relabel_reference_kat(oracle, algo):
    g = load_golden("relabel_kat.json")
    u, labels = oracle.relabel([np.array(x) for x in g["inputs"]], algo=algo)
    assert u.tolist() == g["unique"]
    assert [l.tolist() for l in labels] == g["labels"]


@pytest.mark.parametrize("algo", ["passes", "sweep", "parallel"])
@pytest.mark.parametrize("n", [1, 2, 7, 8, 9, 255, 256, 257, 5000])
def test_relabel_closed_form(oracle, n, algo):
    a = RNG.integers(0, max(2, n // 2), size=n)
    b = RNG.integers(2**31, 2**31 + max(2, n // 2), size=n // 2 + 1)   # ids >= 2^31
    u, labels = oracle.relabel([a, b], algo=algo)
    eu, el = _relabel_closed_form([a, b])
    assert u.tolist() == eu
    assert np.concatenate(labels).tolist() == el


@pytest.mark.parametrize("ids", ["narrow", "wide", "negative"])
@pytest.mark.parametrize("algo", ["parallel", "sweep"])
def test_relabel_forms_that_keep_their_tables_on_repeated_calls(oracle, ids, algo):
    """Both tuned forms keep their tables between calls and empty only the slots they used: calls of
    different sizes one after the other, with ids that fit 32 bits, ids beyond and negative ids (not -1, the
    reference's empty key, src/tensor_relabel.cu:141), must all equal the closed form."""
    for n in (50_000, 300, 120_000, 7):
        a = RNG.integers(0, max(2, n // 3), size=n)
        if ids == "wide":
            a = a + (1 << 40)
        elif ids == "negative":
            a = a - n // 6 - 2                      # some below -1, some above
            a[a == -1] = -2
        u, (labels,) = oracle.relabel([a], algo=algo)
        eu, el = _relabel_closed_form([a])
        assert u.tolist() == eu and labels.tolist() == el


def test_relabel_mixed_dtypes_and_prefix(oracle):
    seeds = RNG.choice(1000, size=50, replace=False).astype(np.int64)
    nbrs = RNG.integers(0, 1000, size=400).astype(np.int32)
    u, (ls, ln) = oracle.relabel([seeds, nbrs])
    assert u.dtype == np.int64 and ls.dtype == np.int64
    assert np.array_equal(u[: seeds.size], seeds)            # destination nodes are a prefix
    assert np.array_equal(ls, np.arange(seeds.size))
    assert np.array_equal(u[ln], nbrs)
    same = oracle.relabel([np.full(33, 9)])
    assert same[0].tolist() == [9] and same[1][0].tolist() == [0] * 33


# ---- philox --------------------------------------------------------------------

def test_philox_known_answers(oracle):
    for v in load_golden("philox4x32_10_kat.json"):
        out = oracle.philox4x32_10([int(x, 16) for x in v["ctr"]], [int(x, 16) for x in v["key"]])
        assert ["%08x" % x for x in out] == v["out"]


# ---- sub-CSR and sampling --------------------------------------------------------

def test_subcsr_reference_kat(oracle):
    g = load_golden("subcsr_kat.json")
    gp, gi = oracle.create_subcsr(np.array(g["indptr"]), np.arange(g["num_indices"]), np.array(g["cache_seeds"]))
    assert gp.tolist() == g["gpu_indptr"] and gi.tolist() == g["gpu_indices"]


def test_subcsr_is_concat(oracle):
    deg = RNG.integers(0, 9, size=300)
    indptr = np.concatenate([[0], np.cumsum(deg)])
    indices = RNG.integers(0, 300, size=indptr[-1]).astype(np.int32)
    rows = RNG.choice(300, size=90, replace=False)
    gp, gi = oracle.create_subcsr(indptr, indices, rows)
    assert gi.dtype == np.int32
    assert np.array_equal(gp, np.concatenate([[0], np.cumsum(deg[rows])]))
    assert np.array_equal(gi, np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in rows]))


def _check_sampling_kat(g, sub_indptr, sub_indices, replace):
    exp = g["replace_true" if replace else "replace_false"]
    assert sub_indptr.tolist() == exp["sub_indptr"]
    assert sub_indices.size == exp["sub_indptr"][-1]
    seg = lambda i: sub_indices[sub_indptr[i]:sub_indptr[i + 1]]
    if replace:
        for i, (lo, hi) in enumerate(exp["segment_ranges"]):
            assert ((seg(i) >= lo) & (seg(i) < hi)).all()
    else:
        for i, vals in exp["exact_segments"].items():
            assert seg(int(i)).tolist() == vals
        for i, (lo, hi) in exp["distinct_in_range"].items():
            s = seg(int(i))
            assert ((s >= lo) & (s < hi)).all() and np.unique(s).size == s.size == g["num_picks"]


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
@pytest.mark.parametrize("replace", [True, False])
@pytest.mark.parametrize("cached", [False, True])
def test_sampling_reference_kat(oracle, algo, replace, cached):
    g = load_golden("csr_sampling_kat.json")
    indptr, indices = np.array(g["indptr"]), np.arange(g["num_indices"])
    seeds = np.array(g["seeds"], dtype=np.int32)
    cache = None
    if cached:
        cs = np.array(g["cache_seeds"])
        gp, gi = oracle.create_subcsr(indptr, indices, cs)
        cache = (gp, gi, oracle.Hashmap(cs, np.arange(cs.size), 0.8))
    sp, si = oracle.sample(indptr, indices, seeds, g["num_picks"], replace, cache=cache, algo=algo)
    _check_sampling_kat(g, sp, si, replace)


@pytest.mark.parametrize("algo", ["reservoir", "floyd"])
def test_sampling_uniform_subsets(oracle, algo):
    """deg > k: every element is selected with probability k/deg (chi-square,
    df = deg-1, checked at the 1e-6 level) and every pair equally often."""
    deg, k, trials = 12, 5, 20000
    indptr = np.arange(0, (trials + 1) * deg, deg)
    indices = np.tile(np.arange(deg), trials)
    sp, si = oracle.sample(indptr, indices, np.arange(trials), k, False, seed=99, algo=algo)
    assert np.array_equal(sp, np.arange(trials + 1) * k)
    picks = si.reshape(trials, k)
    assert all(np.unique(r).size == k for r in picks[:2000])
    counts = np.bincount(si, minlength=deg)
    expected = trials * k / deg
    chi2 = ((counts - expected) ** 2 / expected).sum() / (1 - k / deg)   # hypergeometric variance
    from scipy.stats import chi2 as chi2_dist
    assert chi2 < chi2_dist.ppf(1 - 1e-6, deg - 1), counts
    pair = np.zeros((deg, deg))
    for r in picks:
        pair[np.ix_(r, r)] += 1
    off = pair[~np.eye(deg, dtype=bool)]
    exp_pair = trials * k * (k - 1) / (deg * (deg - 1))
    assert np.abs(off - exp_pair).max() < 6 * np.sqrt(exp_pair)


def test_sampling_replace_uniform(oracle):
    deg, k, trials = 9, 4, 20000
    indptr = np.arange(0, (trials + 1) * deg, deg)
    indices = np.tile(np.arange(deg), trials)
    _, si = oracle.sample(indptr, indices, np.arange(trials), k, True, seed=5)
    counts = np.bincount(si, minlength=deg)
    expected = trials * k / deg
    from scipy.stats import chi2 as chi2_dist
    assert ((counts - expected) ** 2 / expected).sum() < chi2_dist.ppf(1 - 1e-6, deg - 1)
