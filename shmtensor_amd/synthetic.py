"""Seeded synthetic inputs of the benchmark configurations: R-MAT graphs in
CSR form and Zipf-distributed query streams. Generation runs on the current
torch device (GPU when present) so that scale-21..24 graphs build in seconds."""
import torch


def rmat_csr(scale, edge_factor, seed, a=0.57, b=0.19, c=0.19, d=0.05, device=None,
             chunk=1 << 25):
    """R-MAT graph -> (indptr int64 [N+1], indices int32 [E]) with self-loops and
    duplicate edges removed and the edge set symmetrised; neighbours sorted."""
    assert abs(a + b + c + d - 1.0) < 1e-9
    device = device or ("cuda" if torch.cuda.is_available() else "cpu")
    n = 1 << scale
    m = n * edge_factor
    g = torch.Generator(device=device).manual_seed(seed)
    keys = []
    for start in range(0, m, chunk):
        e = min(chunk, m - start)
        src = torch.zeros(e, dtype=torch.int64, device=device)
        dst = torch.zeros(e, dtype=torch.int64, device=device)
        for _ in range(scale):
            r = torch.rand(e, device=device, generator=g)
            sbit = r >= (a + b)
            dbit = ((r >= a) & (r < a + b)) | (r >= a + b + c)
            src = (src << 1) | sbit
            dst = (dst << 1) | dbit
        keep = src != dst
        src, dst = src[keep], dst[keep]
        keys.append(torch.unique(torch.cat([src * n + dst, dst * n + src])))
        del src, dst, keep
    key = torch.unique(torch.cat(keys)) if len(keys) > 1 else keys[0]
    del keys
    rows = key >> scale
    indices = (key & (n - 1)).to(torch.int32)
    del key
    counts = torch.bincount(rows, minlength=n)
    indptr = torch.zeros(n + 1, dtype=torch.int64, device=device)
    torch.cumsum(counts, 0, out=indptr[1:])
    return indptr, indices


def zipf_ranks(n, num_items, s, seed, device=None, head=1 << 20):
    """n ranks in [0, num_items) with P(rank r) proportional to (r + 1)^-s (bounded Zipf law), by inverting
    the CDF: the first `head` ranks through the exact cumulative sums of their weights, the ranks beyond them
    through the integral of x^-s over [r + 1/2, r + 3/2), which differs from (r + 1)^-s by less than
    s (s + 1) / (24 r^2) of it (below 1e-12 relative at r = 2^20)."""
    device = device or ("cuda" if torch.cuda.is_available() else "cpu")
    g = torch.Generator(device=device).manual_seed(seed)
    k = min(int(head), int(num_items))
    weights = torch.arange(1, k + 1, device=device, dtype=torch.float64).pow_(-s)
    cdf = torch.cumsum(weights, 0)
    head_mass = float(cdf[-1])
    one_minus_s = 1.0 - s
    lo = (k + 0.5) ** one_minus_s
    tail_mass = ((num_items + 0.5) ** one_minus_s - lo) / one_minus_s if num_items > k else 0.0
    u = torch.rand(n, device=device, generator=g, dtype=torch.float64) * (head_mass + tail_mass)
    ranks = torch.searchsorted(cdf, u, right=True).clamp_(max=k - 1)          # 0-based rank within the head
    if num_items > k:
        in_tail = u >= head_mass
        x = (lo + (u - head_mass).clamp_(min=0.0) * one_minus_s).pow_(1.0 / one_minus_s)   # in [k + 1/2, N + 1/2)
        tail_rank = (torch.round(x).to(torch.int64) - 1).clamp_(min=k, max=num_items - 1)
        ranks = torch.where(in_tail, tail_rank, ranks)
    return ranks.contiguous()
