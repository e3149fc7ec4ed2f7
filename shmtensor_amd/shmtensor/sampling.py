"""GPUSamplingDataloader: mini-batch neighbour sampling on top of the
ShmTensorLib operators. Same constructor, iteration protocol, cache
management and return values as python/shmtensor/sampling.py:30-237 in the
reference; the per-hop work is `csr_sampling` / `csr_cache_sampling` followed
by `tensor_relabel([seeds, sub_indices])`, issued through the fused
`sample_blocks` operator (same results; one host wait per hop instead of two,
and optionally several batches in flight at once).

Without DGL installed a block is a `CSCBlock` tuple (indptr, indices,
num_src, num_dst), or with `block_format="coo"` a `COOBlock` tuple (row, col,
num_src, num_dst) holding the source and destination of every edge; with DGL
it is the DGLBlock the reference builds from either form
(python/shmtensor/sampling.py:9-27)."""
import collections
import queue
import threading
import weakref

import torch
import torch.distributed as dist

from .. import install_aliases

capi = install_aliases()

CSCBlock = collections.namedtuple("CSCBlock", ["indptr", "indices", "num_src", "num_dst"])
# row[e] / col[e]: source / destination node of edge e, as positions in the block's source /
# destination node lists (the arguments of create_block_from_coo, sampling.py:21-27)
COOBlock = collections.namedtuple("COOBlock", ["row", "col", "num_src", "num_dst"])


def _dgl():
    try:
        import dgl  # noqa: F401
        return dgl
    except Exception:
        return None


def create_block_from_csc(indptr, indices, e_ids, num_src, num_dst):
    dgl = _dgl()
    if dgl is None:
        return CSCBlock(indptr, indices, num_src, num_dst)
    from dgl.heterograph import DGLBlock
    hgidx = dgl.heterograph_index.create_unitgraph_from_csr(
        2, num_src, num_dst, indptr, indices, e_ids, formats=["coo", "csr", "csc"], transpose=True)
    return DGLBlock(hgidx, (["_N"], ["_N"]), ["_E"])


def create_block_from_coo(row, col, num_src, num_dst):
    dgl = _dgl()
    if dgl is None:
        return COOBlock(row, col, num_src, num_dst)
    from dgl.heterograph import DGLBlock
    hgidx = dgl.heterograph_index.create_unitgraph_from_coo(
        2, num_src, num_dst, row, col, formats=["coo", "csr", "csc"])
    return DGLBlock(hgidx, (["_N"], ["_N"]), ["_E"])


def _unpin(tensor):
    capi.unpin_memory(tensor)


class GPUSamplingDataloader:

    def __init__(self, indptr, indices, seeds, batchsize, num_picks, replace=False, use_ddp=False,
                 shuffle=True, drop_last=False, rng_seed=None, prefetch=1, background=False,
                 indptr_on_device=False, features=None, block_format="csc"):
        self.indptr = indptr
        self.indices = indices
        self.seeds = seeds
        self.batchsize = batchsize
        self.num_picks = num_picks
        self.replace = replace
        self.use_ddp = use_ddp
        self.shuffle = shuffle
        self.drop_last = drop_last
        # A sample here is a pure function of (RNG seed, RNG stream, node id, fanout,
        # degree); it does not depend on the node's position in the batch (the reference's
        # draws do: curand_init(7777 + lane, thread id), src/cache_graph_sampling.cu:107,204,
        # so re-batched or shuffled seeds see other samples there even with its fixed seed).
        # The loader therefore gives every batch its own seed and every hop its own stream:
        # batch number b (counted over all epochs) draws from (rng_seed + b, stream = hop).
        # rng_seed=None takes the base from torch's global seed (torch.initial_seed() when the
        # loader is built), so torch.manual_seed() makes a run repeatable and unseeded runs differ.
        self.rng_seed = rng_seed
        self._rng_base = (int(rng_seed) if rng_seed is not None else int(torch.initial_seed())) & ((1 << 62) - 1)
        self._batches_drawn = 0
        # prefetch > 1: that many consecutive batches are sampled together, their
        # kernels overlapping on separate streams (same batches, same order, same
        # results). background=True: a host thread samples ahead on a side stream
        # while the caller consumes the previous batches (feature fetch, training).
        self.prefetch = max(1, int(prefetch))
        self.background = bool(background)
        self._ready = collections.deque()
        self._producer = None
        # features=(uva_data, gpu_data, hashmap) (or (uva_data, None, None)): every batch also
        # carries the feature rows of its input nodes, as cache_fetch / uva_fetch return them, and
        # __next__ yields (input_nodes, output_nodes, blocks, input_features). The fetch is queued
        # behind the last relabel without a host wait between them, into an output sized from the
        # largest batch seen so far (a batch that outgrows it is fetched after its count is known).
        self.features = features
        self._feature_rows = 0
        # block_format="coo": blocks are built from (row, col) edge lists, the destination
        # positions written by the sampling kernel itself; "csc" (the reference loader's
        # choice, sampling.py:139-141): from (sub_indptr, relabelled indices)
        if block_format not in ("csc", "coo"):
            raise ValueError("block_format must be 'csc' or 'coo'")
        self.block_format = block_format

        self.has_cache = False
        self.gpu_indptr = None
        self.gpu_indices = None
        self.hashmap = None

        # indptr_on_device: the row offsets (8 bytes per node, small next to the adjacency) live in
        # HBM whatever the cache holds; a cold row then costs one host-link round trip per hop, not two
        if indptr_on_device and self.indptr.device.type == "cpu":
            self.indptr = self.indptr.cuda()
        for name in ("indptr", "indices"):
            t = getattr(self, name)
            if t.device.type == "cpu":
                capi.pin_memory(t)       # python/shmtensor/sampling.py:57-63
                weakref.finalize(self, _unpin, t)

        self._partition_seeds()
        if self.shuffle:
            self.seeds = self.seeds[torch.randperm(self.seeds.numel(), device=self.seeds.device)]
        self._set_length()
        self.curr = 0
        self.seeds = self.seeds.cuda()

    # ---- batching ---------------------------------------------------------

    def _partition_seeds(self):
        if self.use_ddp:   # each rank keeps its contiguous slice (sampling.py:65-71)
            world_size, rank = dist.get_world_size(), dist.get_rank()
            part = (self.seeds.numel() + world_size - 1) // world_size
            self.seeds = self.seeds[rank * part:(rank + 1) * part]

    def _set_length(self):
        n = self.seeds.numel()
        self.len = n // self.batchsize if self.drop_last else (n + self.batchsize - 1) // self.batchsize

    def __len__(self):
        return self.len

    def __iter__(self):
        self._stop_producer()
        self._ready.clear()
        if self.shuffle:
            self.seeds = self.seeds[torch.randperm(self.seeds.numel(), device=self.seeds.device)]
        self.curr = 0
        return self

    def _discard_prefetched(self):
        """Batches sampled ahead belong to the old parameters / cache: drop them."""
        self._stop_producer()
        self._ready.clear()

    def close(self):
        """Stop the background thread (it otherwise ends with the epoch)."""
        self._discard_prefetched()

    def update_params(self, **kwargs):
        self._discard_prefetched()
        for k, v in kwargs.items():
            setattr(self, k, v)
        if "seeds" in kwargs or "use_ddp" in kwargs:
            print("Updating seeds")
            self._partition_seeds()
            self.seeds = self.seeds.cuda()
            self._set_length()

    # ---- one hop / one batch ---------------------------------------------------

    def _sample(self, seeds, num_pick, hop, use_cache=True):
        extra = {"seed": self._rng_base + self._batches_drawn, "stream_id": hop}
        if use_cache and self.has_cache:
            return capi.csr_cache_sampling(self.indptr, self.indices, self.gpu_indptr, self.gpu_indices,
                                           self.hashmap, seeds, num_pick, self.replace, **extra)
        return capi.csr_sampling(self.indptr, self.indices, seeds, num_pick, self.replace, **extra)

    def _sample_group(self, first_batch, count, batches_drawn):
        """Sample `count` consecutive batches starting at batch `first_batch`; returns one
        (input_nodes, output_nodes, blocks) per batch."""
        groups = [self.seeds[b * self.batchsize:(b + 1) * self.batchsize]
                  for b in range(first_batch, first_batch + count)]
        rng = [self._rng_base + batches_drawn + j for j in range(count)]
        cached = self.has_cache
        graph = (self.indptr, self.indices, self.gpu_indptr if cached else None,
                 self.gpu_indices if cached else None, self.hashmap if cached else None)
        # the last fanout is applied to the seed layer (sampling.py:128)
        picks = list(reversed(self.num_picks))
        coo = self.block_format == "coo"
        if self.features is None:
            chains = capi.sample_blocks(*graph, groups, picks, self.replace, seeds_rng=rng,
                                        max_in_flight=self.prefetch, coo=coo)
            rows = [None] * len(groups)
        else:
            uva_data, gpu_data, data_map = self.features
            guess = self._feature_rows + self._feature_rows // 4 + 1024 if self._feature_rows else 0
            fetched = capi.sample_blocks_fetch(*graph, groups, picks, self.replace, uva_data, gpu_data, data_map,
                                               seeds_rng=rng, max_in_flight=self.prefetch, max_rows=guess, coo=coo)
            chains = [hops for hops, _ in fetched]
            rows = [x for _, x in fetched]
            self._feature_rows = max([self._feature_rows] + [x.shape[0] for x in rows])
        out = []
        for seeds, chain, x in zip(groups, chains, rows):
            blocks, dst = [], seeds
            for hop in chain:
                sub_indptr, _, unique_tensor, relabel_indices = hop[:4]
                if coo:
                    blocks.insert(0, create_block_from_coo(relabel_indices, hop[4], unique_tensor.numel(),
                                                           dst.numel()))
                else:
                    blocks.insert(0, create_block_from_csc(sub_indptr, relabel_indices, torch.Tensor(),
                                                           unique_tensor.numel(), dst.numel()))
                dst = unique_tensor
            out.append((dst, seeds, blocks) if self.features is None else (dst, seeds, blocks, x))
        return out

    def _produce(self, first_batch, batches_drawn, out_queue, stop):
        """Body of the background thread: groups of batches, each handed over with the
        event that marks its results complete on the producer's stream."""
        try:
            torch.cuda.set_device(self.seeds.device)
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                b = first_batch
                while b < self.len and not stop.is_set():
                    count = min(self.prefetch, self.len - b)
                    group = self._sample_group(b, count, batches_drawn)
                    done = torch.cuda.Event()
                    done.record(side)
                    out_queue.put((group, done))
                    b += count
                    batches_drawn += count
            out_queue.put(None)
        except BaseException as exc:       # surfaces in the consumer's __next__
            out_queue.put(exc)

    def _stop_producer(self):
        if self._producer is not None:
            thread, out_queue, stop = self._producer
            stop.set()
            while thread.is_alive():
                try:
                    out_queue.get(timeout=0.05)
                except queue.Empty:
                    pass
            thread.join()
            self._producer = None

    def _refill(self):
        if not self.background:
            count = min(self.prefetch, self.len - self.curr)
            self._ready.extend(self._sample_group(self.curr, count, self._batches_drawn))
            return
        if self._producer is None:
            out_queue, stop = queue.Queue(maxsize=2), threading.Event()
            thread = threading.Thread(target=self._produce, daemon=True,
                                      args=(self.curr, self._batches_drawn, out_queue, stop))
            self._producer = (thread, out_queue, stop)
            thread.start()
        item = self._producer[1].get()
        if isinstance(item, BaseException):
            self._stop_producer()
            raise item
        if item is None:
            raise StopIteration
        group, done = item
        current = torch.cuda.current_stream()
        current.wait_event(done)
        for item in group:                 # produced on other streams, consumed on this one
            dst, blocks = item[0], item[2]
            for t in (dst,) + tuple(item[3:]) + tuple(x for blk in blocks if isinstance(blk, (CSCBlock, COOBlock))
                                                      for x in blk[:2]):
                if t.numel() > 0:
                    t.record_stream(current)
        self._ready.extend(group)

    def __next__(self):
        if self.curr >= self.len:
            self._stop_producer()
            raise StopIteration
        if not self._ready:
            self._refill()
        batch = self._ready.popleft()      # (input_nodes, output_nodes, blocks[, input_features])
        self.curr += 1
        self._batches_drawn += 1
        return batch

    # ---- cache ---------------------------------------------------------------------

    def create_cache(self, cache_capacity, hotness):
        """Cache the adjacency of the hottest nodes that fit `cache_capacity` bytes
        (sampling.py:149-189). Cost model per node: deg * index bytes + one indptr
        entry + 10 bytes of hashmap (int32 key and value at load factor 0.8)."""
        if cache_capacity <= 0:
            return
        self._discard_prefetched()
        full_size = self.indptr.nbytes + self.indices.nbytes
        if full_size <= cache_capacity:      # everything fits: plain GPU sampling
            self.has_cache = False
            self.indices = self.indices.cuda()
            self.indptr = self.indptr.cuda()
            print("Cache Ratio for GPU sampling: {:.2f}".format(cache_capacity / full_size))
            return

        degrees = (self.indptr[1:] - self.indptr[:-1]).cpu()
        _, candidates = torch.sort(hotness.cpu(), descending=True)
        size = degrees[candidates] * self.indices.element_size() + self.indptr.element_size() + 1.25 * 2 * 4
        prefix = torch.cumsum(size, dim=0)
        cache_size = torch.searchsorted(prefix, cache_capacity).item()
        # the cached rows are kept in id order: a node's slot is then its rank among the cached ids, which the
        # map stores as a bitmap with running counts instead of a table (samples do not depend on the slot)
        candidates = torch.sort(candidates[:cache_size]).values.cuda()
        if candidates.numel() > 0:
            self.gpu_indptr, self.gpu_indices = capi.create_subcsr(self.indptr, self.indices, candidates)
            self.hashmap = capi.CUCOStaticHashmap(
                candidates.int(), torch.arange(candidates.numel(), device="cuda", dtype=torch.int32), 0.8)
            self.has_cache = True
            covered = prefix[min(cache_size, prefix.numel() - 1)].item()
            print("Cache Ratio for GPU sampling: {:.2f}".format(covered / full_size))
            print("create cache success")

    def clear_cache(self):
        self._discard_prefetched()
        self.has_cache = False
        self.gpu_indptr = None
        self.gpu_indices = None
        self.hashmap = None

    def presampling(self):
        """One uncached pass over all batches counting how often each node is
        sampled from / fetched (sampling.py:200-228)."""
        num_nodes = self.indptr.numel() - 1
        sampling_hotness = torch.zeros(num_nodes, device="cuda")
        feature_hotness = torch.zeros(num_nodes, device="cuda")
        one = torch.ones(1, device="cuda")
        for i in range(self.len):
            seeds = self.seeds[i * self.batchsize:(i + 1) * self.batchsize]
            for hop, num_pick in enumerate(reversed(self.num_picks)):
                sampling_hotness.index_add_(0, seeds.long(), one.expand(seeds.numel()))
                _, sub_indices = self._sample(seeds, num_pick, hop, use_cache=False)
                unique_tensor, _ = capi.tensor_relabel([seeds, sub_indices])
                seeds = unique_tensor
                feature_hotness.index_add_(0, unique_tensor.long(), one.expand(unique_tensor.numel()))
        if self.use_ddp:
            dist.all_reduce(sampling_hotness)
            dist.all_reduce(feature_hotness)
        return sampling_hotness.cpu(), feature_hotness.cpu()

    def compute_weight_size(self, hotness):
        full_size = self.indptr.nbytes + self.indices.nbytes
        degree = (self.indptr[1:] - self.indptr[:-1]).clip(max=self.num_picks[0] * 1.3).float().cpu()
        hot = hotness > 0
        item_size = (degree[hot] * self.indices.element_size() + self.indptr.element_size()) * hotness[hot]
        return full_size, item_size.mean().item()
