"""Seeded synthetic inputs of the shapes the hot path sees: CSR graphs (uniform out-degree,
R-MAT power law, stochastic block model) and boundary feature blocks.  Pure torch, so the same
generator runs on the CPU for small test cases and on the GPU for full-size benchmark cases."""
import math

import torch


def _gen(device, seed):
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def csr_from_pairs(src, dst, num_rows, num_cols, dedupe=True):
    """Rows = src, columns = dst; sorted by (row, col); duplicates dropped when ``dedupe``.
    Returns (rowptr int64[M+1], col int32[nnz])."""
    key = src.to(torch.int64) * int(num_cols) + dst.to(torch.int64)
    key = torch.unique(key) if dedupe else torch.sort(key).values
    row = torch.div(key, int(num_cols), rounding_mode="floor")
    col = (key - row * int(num_cols)).to(torch.int32)
    counts = torch.bincount(row, minlength=int(num_rows))
    rowptr = torch.zeros(int(num_rows) + 1, dtype=torch.int64, device=key.device)
    torch.cumsum(counts, 0, out=rowptr[1:])
    return rowptr, col


def uniform_degree_graph(num_nodes, degree, seed=0, self_loops=True, device="cpu"):
    """Every row draws ``degree`` uniform neighbours (duplicates kept) plus its own self loop;
    each row sorted by column."""
    g = _gen(device, seed)
    col = torch.randint(0, num_nodes, (num_nodes, degree), generator=g, device=device, dtype=torch.int64)
    if self_loops:
        col = torch.cat([col, torch.arange(num_nodes, device=device).view(-1, 1)], dim=1)
    col = torch.sort(col, dim=1).values
    per = col.shape[1]
    rowptr = torch.arange(num_nodes + 1, device=device, dtype=torch.int64) * per
    return rowptr, col.reshape(-1).to(torch.int32).contiguous()


def rmat_graph(num_nodes, num_undirected_edges, a=0.57, b=0.19, c=0.19, seed=1, device="cpu", chunk=1 << 24):
    """R-MAT edges (ids >= num_nodes rejected, self loops dropped), symmetrised and de-duplicated.
    Returns (rowptr, col) of the undirected graph's CSR (both directions stored)."""
    scale = max(1, math.ceil(math.log2(max(num_nodes, 2))))
    g = _gen(device, seed)
    keys = []
    have = 0
    want = int(num_undirected_edges)
    ab, abc = a + b, a + b + c
    while have < want:
        n = min(chunk, max(int((want - have) * 1.3) + 1024, 1024))
        src = torch.zeros(n, dtype=torch.int64, device=device)
        dst = torch.zeros(n, dtype=torch.int64, device=device)
        for _ in range(scale):
            r = torch.rand(n, generator=g, device=device)
            src = src * 2 + (r >= ab).to(torch.int64)
            dst = dst * 2 + (((r >= a) & (r < ab)) | (r >= abc)).to(torch.int64)
        ok = (src < num_nodes) & (dst < num_nodes) & (src != dst)
        lo = torch.minimum(src[ok], dst[ok])
        hi = torch.maximum(src[ok], dst[ok])
        keys.append(lo * num_nodes + hi)
        allk = torch.unique(torch.cat(keys))
        keys = [allk]
        have = allk.numel()
    allk = keys[0]
    if allk.numel() > want:
        perm = torch.randperm(allk.numel(), generator=g, device=device)[:want]
        allk = allk[perm]
    lo = torch.div(allk, num_nodes, rounding_mode="floor")
    hi = allk - lo * num_nodes
    return csr_from_pairs(torch.cat([lo, hi]), torch.cat([hi, lo]), num_nodes, num_nodes, dedupe=False)


def sbm_graph(num_nodes, num_blocks, p_in, p_out, seed=3, device="cpu"):
    """Stochastic block model with equal blocks: per block pair a binomial edge count, then
    uniform pairs inside the pair of blocks; symmetrised and de-duplicated."""
    g = _gen(device, seed)
    cpu_g = _gen("cpu", seed + 1)
    bs = num_nodes // num_blocks
    srcs, dsts = [], []
    for bi in range(num_blocks):
        for bj in range(bi, num_blocks):
            pairs = bs * (bs - 1) // 2 if bi == bj else bs * bs
            p = p_in if bi == bj else p_out
            mean, std = pairs * p, math.sqrt(pairs * p * (1 - p))
            cnt = max(0, int(round(mean + std * torch.randn((), generator=cpu_g).item())))
            if cnt == 0:
                continue
            u = torch.randint(0, bs, (cnt,), generator=g, device=device, dtype=torch.int64) + bi * bs
            v = torch.randint(0, bs, (cnt,), generator=g, device=device, dtype=torch.int64) + bj * bs
            srcs.append(u)
            dsts.append(v)
    u = torch.cat(srcs)
    v = torch.cat(dsts)
    keep = u != v
    u, v = u[keep], v[keep]
    return csr_from_pairs(torch.cat([u, v]), torch.cat([v, u]), num_nodes, num_nodes, dedupe=True)


def gcn_norm_weights(rowptr, col):
    """1/sqrt(d_u * d_v) per stored entry, d = row degree clamped to >= 1."""
    deg = (rowptr[1:] - rowptr[:-1]).clamp(min=1).to(torch.float32)
    row = torch.repeat_interleave(torch.arange(deg.numel(), device=col.device), rowptr[1:] - rowptr[:-1])
    return (1.0 / torch.sqrt(deg[row] * deg[col.to(torch.int64)])).to(torch.float32)


def boundary_features(num_rows, feat_len, seed=5, outlier_every=10, outlier_scale=100.0, device="cpu"):
    """~N(0,1) rows; every ``outlier_every``-th row scaled by ``outlier_scale``."""
    g = _gen(device, seed)
    x = torch.randn(num_rows, feat_len, generator=g, device=device, dtype=torch.float32)
    if outlier_every:
        x[::outlier_every] *= outlier_scale
    return x
