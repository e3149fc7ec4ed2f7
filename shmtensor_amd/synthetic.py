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


def zipf_ranks(n, num_items, s, seed, device=None):
    """n ranks in [0, num_items) with P(rank r) proportional to (r+1)^-s, by
    inverting the continuous approximation of the Zipf CDF and rejecting the
    (rare) draws that fall outside the support."""
    device = device or ("cuda" if torch.cuda.is_available() else "cpu")
    g = torch.Generator(device=device).manual_seed(seed)
    out = torch.empty(0, dtype=torch.int64, device=device)
    one_minus_s = 1.0 - s
    hi = (num_items + 0.5) ** one_minus_s
    lo = 0.5 ** one_minus_s
    while out.numel() < n:
        u = torch.rand(n, device=device, generator=g, dtype=torch.float64)
        x = (lo + u * (hi - lo)) ** (1.0 / one_minus_s)
        r = torch.round(x).to(torch.int64) - 1
        r = r[(r >= 0) & (r < num_items)]
        out = torch.cat([out, r])
    return out[:n].contiguous()
