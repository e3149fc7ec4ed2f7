"""GPUSamplingDataloader: mini-batch neighbour sampling on top of the
ShmTensorLib operators. Same constructor, iteration protocol, cache
management and return values as python/shmtensor/sampling.py:30-237 in the
reference; the per-hop work is `csr_sampling` / `csr_cache_sampling` followed
by `tensor_relabel([seeds, sub_indices])`, issued through the fused
`sample_hop` operator (same results, one host wait per hop instead of two).

Without DGL installed a block is a `CSCBlock` tuple (indptr, indices,
num_src, num_dst); with DGL it is the DGLBlock the reference builds
(python/shmtensor/sampling.py:9-18)."""
import collections
import weakref

import torch
import torch.distributed as dist

from .. import install_aliases

capi = install_aliases()

CSCBlock = collections.namedtuple("CSCBlock", ["indptr", "indices", "num_src", "num_dst"])


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


def _unpin(tensor):
    capi.unpin_memory(tensor)


class GPUSamplingDataloader:

    def __init__(self, indptr, indices, seeds, batchsize, num_picks, replace=False, use_ddp=False,
                 shuffle=True, drop_last=False, rng_seed=None):
        self.indptr = indptr
        self.indices = indices
        self.seeds = seeds
        self.batchsize = batchsize
        self.num_picks = num_picks
        self.replace = replace
        self.use_ddp = use_ddp
        self.shuffle = shuffle
        self.drop_last = drop_last
        # None: every call uses the fixed default seed, as the reference does
        # (src/cache_graph_sampling.cu:204,407); an int: batch b, hop h draw from
        # (rng_seed + b, stream h), so epochs and batches differ reproducibly.
        self.rng_seed = rng_seed
        self._batches_drawn = 0

        self.has_cache = False
        self.gpu_indptr = None
        self.gpu_indices = None
        self.hashmap = None

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
        if self.shuffle:
            self.seeds = self.seeds[torch.randperm(self.seeds.numel(), device=self.seeds.device)]
        self.curr = 0
        return self

    def update_params(self, **kwargs):
        for k, v in kwargs.items():
            setattr(self, k, v)
        if "seeds" in kwargs or "use_ddp" in kwargs:
            print("Updating seeds")
            self._partition_seeds()
            self.seeds = self.seeds.cuda()
            self._set_length()

    # ---- one hop / one batch ---------------------------------------------------

    def _sample(self, seeds, num_pick, hop, use_cache=True):
        extra = {}
        if self.rng_seed is not None:
            extra = {"seed": int(self.rng_seed) + self._batches_drawn, "stream_id": hop}
        if use_cache and self.has_cache:
            return capi.csr_cache_sampling(self.indptr, self.indices, self.gpu_indptr, self.gpu_indices,
                                           self.hashmap, seeds, num_pick, self.replace, **extra)
        return capi.csr_sampling(self.indptr, self.indices, seeds, num_pick, self.replace, **extra)

    def _hop(self, seeds, num_pick, hop):
        """Sampling and relabel of one hop as one operator: all its kernels are
        queued before the host waits for either data-dependent size."""
        extra = {}
        if self.rng_seed is not None:
            extra = {"seed": int(self.rng_seed) + self._batches_drawn, "stream_id": hop}
        cached = self.has_cache
        return capi.sample_hop(self.indptr, self.indices, self.gpu_indptr if cached else None,
                               self.gpu_indices if cached else None, self.hashmap if cached else None,
                               seeds, num_pick, self.replace, **extra)

    def __next__(self):
        if self.curr >= self.len:
            raise StopIteration
        seeds = self.seeds[self.curr * self.batchsize:(self.curr + 1) * self.batchsize]
        self.curr += 1

        output_nodes = seeds
        blocks = []
        # the last fanout is applied to the seed layer (sampling.py:128)
        for hop, num_pick in enumerate(reversed(self.num_picks)):
            sub_indptr, _, unique_tensor, relabel_indices = self._hop(seeds, num_pick, hop)
            blocks.insert(0, create_block_from_csc(sub_indptr, relabel_indices, torch.Tensor(),
                                                   unique_tensor.numel(), seeds.numel()))
            seeds = unique_tensor
        self._batches_drawn += 1
        input_nodes = seeds
        return input_nodes, output_nodes, blocks

    # ---- cache ---------------------------------------------------------------------

    def create_cache(self, cache_capacity, hotness):
        """Cache the adjacency of the hottest nodes that fit `cache_capacity` bytes
        (sampling.py:149-189). Cost model per node: deg * index bytes + one indptr
        entry + 10 bytes of hashmap (int32 key and value at load factor 0.8)."""
        if cache_capacity <= 0:
            return
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
        candidates = candidates[:cache_size].cuda()
        if candidates.numel() > 0:
            self.gpu_indptr, self.gpu_indices = capi.create_subcsr(self.indptr, self.indices, candidates)
            self.hashmap = capi.CUCOStaticHashmap(
                candidates.int(), torch.arange(candidates.numel(), device="cuda", dtype=torch.int32), 0.8)
            self.has_cache = True
            covered = prefix[min(cache_size, prefix.numel() - 1)].item()
            print("Cache Ratio for GPU sampling: {:.2f}".format(covered / full_size))
            print("create cache success")

    def clear_cache(self):
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
