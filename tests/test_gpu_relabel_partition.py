"""Relabel of large inputs through hash partitions with their tables in LDS: the size from
which that form is used is lowered (shmt_relabel_tuning) so that inputs the oracle finishes
quickly take it, through every entry point that relabels. Bit-exact against the oracle and
against the same call with the default setting; the rare paths of a partition whose ids do
not fit its table (rounds, all pairs) are driven by shrinking the table."""
import numpy as np
import pytest
import torch

from shmtensor_amd.synthetic import rmat_csr

pytestmark = pytest.mark.gpu


@pytest.fixture
def tuning(cabi):
    lib = cabi.load()

    def set_(min_ids, slots_log2=0, rounds_log2=-1):
        cabi.check(lib.shmt_relabel_tuning(min_ids, slots_log2, rounds_log2))

    yield set_
    lib.shmt_relabel_tuning(0, 0, -1)


def _ids(kind, n, rng, dt):
    a = rng.integers(0, max(2, n // 3), size=n).astype(np.int64)
    if kind == "spread32":
        a[::5] = rng.integers(0, 2**32 if dt == np.int64 else 2**31, size=a[::5].size)
    elif kind == "wide":
        a[1::3] += 2**40
    elif kind == "one_wide_id_at_the_end":
        a[-1] = 2**32
    elif kind == "negative":
        a[::7] = -a[::7] - 2
    elif kind == "minus_one":
        a[::11] = -1
    elif kind == "hub":
        a[rng.random(n) < 0.3] = 5
    elif kind == "all_equal":
        a[:] = 123456
    elif kind == "all_distinct":
        a = rng.permutation(n).astype(np.int64) * 3 + 1
    elif kind == "uint32_max":
        a[::9] = 2**32 - 1
    return a.astype(dt)


KINDS64 = ["spread32", "wide", "one_wide_id_at_the_end", "negative", "minus_one", "hub", "all_equal", "all_distinct",
           "uint32_max"]
KINDS32 = ["spread32", "negative", "hub", "all_equal", "all_distinct"]


@pytest.mark.parametrize("n", [5462, 9000, 70_001, 600_000])
@pytest.mark.parametrize("dt,kind", [(np.int64, k) for k in KINDS64] + [(np.int32, k) for k in KINDS32])
def test_partitioned_relabel_matches_oracle(capi, oracle, tuning, n, dt, kind):
    rng = np.random.default_rng(n)
    a = _ids(kind, n, rng, dt)
    b = rng.integers(0, max(2, n // 3), size=n // 2 + 1).astype(dt)
    tuning(8193)
    u, (la, lb) = capi.tensor_relabel([torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()])
    eu, (ea, eb) = oracle.relabel([a, b])
    assert np.array_equal(u.cpu().numpy(), eu)
    assert np.array_equal(la.cpu().numpy(), ea) and np.array_equal(lb.cpu().numpy(), eb)


@pytest.mark.parametrize("n", [8193, 100_000, 1_000_000])
@pytest.mark.parametrize("bytes_,kind", [(8, "spread32"), (8, "wide"), (8, "negative"), (4, "spread32"), (4, "negative")])
def test_c_abi_partitioned_relabel_of_one_array(cabi, oracle, tuning, n, bytes_, kind):
    """shmt_relabel: no earlier kernel has seen the ids, the count pass decides the record format."""
    lib = cabi.load()
    ids = _ids(kind, n, np.random.default_rng(n + bytes_), np.int32 if bytes_ == 4 else np.int64)
    total = torch.from_numpy(ids).cuda()
    sbytes = lib.shmt_relabel_scratch_bytes(n)
    outs = []
    for min_ids in (8193, 0):
        tuning(min_ids)
        unique, labels = torch.full_like(total, -7), torch.full_like(total, -7)
        scratch = torch.empty(sbytes, dtype=torch.uint8).cuda()
        count = torch.full((1,), -1, dtype=torch.int64).cuda()
        cabi.check(lib.shmt_relabel(total.data_ptr(), n, bytes_, scratch.data_ptr(), sbytes, unique.data_ptr(),
                                    labels.data_ptr(), count.data_ptr(), cabi.current_stream()))
        torch.cuda.synchronize()
        outs.append((int(count.item()), unique.cpu().numpy(), labels.cpu().numpy()))
    eu, (el,) = oracle.relabel([ids])
    for cnt, unique, labels in outs:
        assert cnt == eu.size
        assert np.array_equal(unique[:cnt], eu) and np.array_equal(labels, el)


@pytest.mark.parametrize("slots_log2,rounds_log2", [(6, -1), (3, -1), (4, 2), (2, 0)])
@pytest.mark.parametrize("kind", ["spread32", "wide", "minus_one", "hub"])
def test_partition_that_does_not_fit_its_table(capi, oracle, tuning, slots_log2, rounds_log2, kind):
    """Tables of 64 / 8 / 16 / 4 slots for partitions of some 300 distinct ids: the partition is worked
    through in rounds over classes of its ids, and by comparing all pairs once the rounds are used up."""
    n = 40_000
    rng = np.random.default_rng(slots_log2)
    a = _ids(kind, n, rng, np.int64)
    b = rng.integers(0, n // 3, size=n // 2).astype(np.int64)
    tuning(8193, slots_log2, rounds_log2)
    u, (la, lb) = capi.tensor_relabel([torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()])
    eu, (ea, eb) = oracle.relabel([a, b])
    assert np.array_equal(u.cpu().numpy(), eu)
    assert np.array_equal(la.cpu().numpy(), ea) and np.array_equal(lb.cpu().numpy(), eb)


def _same(a, b):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and x.shape == y.shape and torch.equal(x, y)


@pytest.mark.parametrize("idx_dt", [torch.int32, torch.int64])
@pytest.mark.parametrize("n_batches,in_flight", [(4, 4), (8, 8), (11, 8), (3, 3)])
def test_fused_hop_and_chained_batches_through_partitions(capi, tuning, idx_dt, n_batches, in_flight):
    """The fused hop (the pick kernel writes the relabel input and would have emptied the table) and
    sample_blocks (hops chained on the device; from four batches on their partition passes share their
    launches, fewer keep the table in memory) give what they give with the default setting."""
    indptr, indices = rmat_csr(15, 12, 3)
    indptr, indices = indptr.cuda(), indices.to(idx_dt).cuda()
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(4)
    seeds = torch.randint(0, n, (3000,), generator=g).to(idx_dt).cuda()
    batches = [torch.randperm(n, generator=g)[:700 - 13 * b].to(idx_dt).cuda() for b in range(n_batches)]
    got = {}
    for min_ids in (0, 8193):
        tuning(min_ids)
        hop = capi.sample_hop(indptr, indices, None, None, None, seeds, 10, False, seed=5)
        blocks = capi.sample_blocks(indptr, indices, None, None, None, batches, [5, 6, 7], False,
                                    seeds_rng=list(range(5, 5 + n_batches)), max_in_flight=in_flight)
        torch.cuda.synchronize()
        got[min_ids] = (hop, blocks)
    _same(got[0][0], got[8193][0])
    assert len(got[0][1]) == len(got[8193][1]) == len(batches)
    for x, y in zip(got[0][1], got[8193][1]):
        assert len(x) == len(y) == 3
        for hop_x, hop_y in zip(x, y):
            _same(hop_x, hop_y)


@pytest.mark.parametrize("seed", range(8))
def test_random_inputs_tables_and_round_limits(capi, cabi, oracle, tuning, seed):
    """Seeded random cases: sizes, id universes from 3 values to 2^40, one to three tensors of mixed widths,
    tables of 4 to 16,384 slots, round limits from 'all pairs at once' to the default."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(6):
        n = int(rng.choice([rng.integers(8193, 20000), rng.integers(20000, 200000)]))
        universe = int(rng.choice([3, 100, n // 10 + 2, n, 10 * n, 2**31 - 1, 2**40]))
        slots = int(rng.choice([0, 0, 2, 3, 5, 8, 11, 14]))
        rounds = int(rng.choice([-1, -1, 0, 1, 3]))
        kind = str(rng.choice(["plain", "neg", "hub", "top32"]))
        print("case", seed, case, n, universe, slots, rounds, kind, flush=True)
        ids = rng.integers(0, universe, size=n).astype(np.int64)
        if kind == "neg":
            ids[::7] = -ids[::7] - 2
        elif kind == "hub":
            ids[rng.random(n) < rng.random() * 0.6] = ids[0]
        elif kind == "top32":
            ids[::5] = 2**32 - 1 - (ids[::5] % 3)
        fits32 = ids.min() >= -2**31 and ids.max() < 2**31
        nseg = int(rng.integers(1, 4))
        parts = np.split(ids, np.sort(rng.integers(0, n, size=nseg - 1)))
        parts = [p.astype(np.int32 if (fits32 and rng.random() < 0.5) else np.int64) for p in parts]
        tuning(8193, slots, rounds)
        u, labs = capi.tensor_relabel([torch.from_numpy(p).cuda() for p in parts])
        ou, olabs = oracle.relabel([p.astype(np.int64) for p in parts])
        assert np.array_equal(u.cpu().numpy().astype(np.int64), ou)
        for l, o in zip(labs, olabs):
            assert np.array_equal(l.cpu().numpy().astype(np.int64), o)


def test_tuning_rejects_bad_values(cabi):
    lib = cabi.load()
    assert lib.shmt_relabel_tuning(0, 1, -1) != 0
    assert lib.shmt_relabel_tuning(0, 15, -1) != 0
    assert lib.shmt_relabel_tuning(0, 0, 21) != 0
    assert lib.shmt_relabel_tuning(0, 0, -1) == 0
