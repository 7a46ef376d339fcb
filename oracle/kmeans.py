"""Segmented spherical k-means of cache_hub/kmeans.py, restated on the CPU.

The reference accumulates cluster sums with fp32 atomics, so its own result depends on the
order the hardware retires them.  This restatement fixes the order the way the HIP kernels do:
a cluster's tokens in ascending index are cut into blocks of SUM_BLOCK; each block is summed
one fp32 add per token starting from +0, and the block sums are added in block order starting
from the first block's.  Up to SUM_BLOCK tokens that is the plain ascending-index sum.
"""
import numpy as np
import torch


def _f32(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.float32).numpy()


def _to_bf16(a: np.ndarray, dtype=torch.bfloat16) -> torch.Tensor:
    """fp32 array -> tensor of the 16-bit element type (round to nearest even)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype)


def init_indices(num_tokens: int, num_centroids: int) -> torch.Tensor:
    """kmeans.py:234-236: two separately rounded float32 operations, then truncation."""
    idx = torch.arange(num_centroids, dtype=torch.float32) * (num_tokens / num_centroids)
    idx += num_tokens / num_centroids / 2
    return idx.to(torch.int64)


def assign(data: torch.Tensor, cent: torch.Tensor):
    """argmax_c <data[n], cent[c]> with the smallest c on ties (kmeans.py:38-44).
    data [N, D], cent [nc, D] bf16.  Scores in fp64 (exact for bf16 inputs).  Returns
    (assign int64 [N], best score, runner-up score) — the gap tells a test how close a tie was."""
    s = data.double().numpy() @ cent.double().numpy().T
    a = np.argmax(s, axis=1)  # numpy returns the first maximum
    best = s[np.arange(s.shape[0]), a]
    s2 = s.copy()
    s2[np.arange(s.shape[0]), a] = -np.inf
    second = s2.max(axis=1) if s.shape[1] > 1 else np.full_like(best, -np.inf)
    return a.astype(np.int64), best, second


SUM_BLOCK = 256


def cluster_sums(rows: torch.Tensor, a: np.ndarray, nc: int):
    """sum[c] = blocked fp32 sum (see the module header) of rows with a[n] == c; cnt[c]
    (kmeans.py:48-49)."""
    a = np.asarray(a, dtype=np.int64)
    cnt = np.bincount(a, minlength=nc).astype(np.int32)
    order = np.argsort(a, kind="stable")                       # tokens grouped by cluster, ascending inside
    start = np.concatenate([[0], np.cumsum(cnt)])[:-1]
    pos = np.empty(a.shape[0], dtype=np.int64)
    pos[order] = np.arange(a.shape[0]) - np.repeat(start, cnt)  # rank of a token inside its cluster
    blk = pos // SUM_BLOCK
    maxblk = int(blk.max()) + 1 if a.shape[0] else 1
    item_key, item_of = np.unique(a * maxblk + blk, return_inverse=True)
    part = np.zeros((item_key.shape[0], rows.shape[1]), dtype=np.float32)
    np.add.at(part, item_of, _f32(rows))  # unbuffered, in index order: one fp32 add per token
    item_c, item_b = item_key // maxblk, item_key % maxblk
    s = np.zeros((nc, rows.shape[1]), dtype=np.float32)
    first = item_b == 0
    s[item_c[first]] = part[first]
    for b in range(1, maxblk):
        sel = item_b == b
        s[item_c[sel]] = (s[item_c[sel]] + part[sel]).astype(np.float32)
    return s, cnt


def _lane_butterfly_sumsq(x: np.ndarray) -> np.ndarray:
    """||x||^2 per row the way one 64-lane wave computes it: lane l holds dims 2l, 2l+1,
    squares and adds them (two roundings), then xor-butterfly over 32, 16, ..., 1."""
    k, d = x.shape
    assert d == 128
    pair = x.reshape(k, 64, 2)
    sq = (pair[:, :, 0] * pair[:, :, 0]).astype(np.float32) + (pair[:, :, 1] * pair[:, :, 1]).astype(np.float32)
    sq = sq.astype(np.float32)
    lanes = np.arange(64)
    for o in (32, 16, 8, 4, 2, 1):
        sq = (sq + sq[:, lanes ^ o]).astype(np.float32)
    return sq[:, 0]


def update(cent: torch.Tensor, s: np.ndarray, cnt: np.ndarray, normalize: bool) -> torch.Tensor:
    """kmeans.py:73-80: mean, optional L2 normalisation, store only where cnt > 0."""
    out = cent.clone()
    nz = cnt > 0
    if nz.any():
        x = (s[nz] / cnt[nz].astype(np.float32)[:, None]).astype(np.float32)
        if normalize:
            nrm = np.sqrt(_lane_butterfly_sumsq(x)).astype(np.float32)
            x = (x / nrm[:, None]).astype(np.float32)
        out[torch.from_numpy(nz)] = _to_bf16(x, cent.dtype)
    return out


def train_step(data, cent, normalize):
    """One _triton_k_means_train call (kmeans.py:83-125) on one problem."""
    a, _, _ = assign(data, cent)
    s, cnt = cluster_sums(data, a, cent.shape[0])
    return update(cent, s, cnt, normalize), a, cnt


def value_sum(value: torch.Tensor, a: np.ndarray, nc: int) -> torch.Tensor:
    """kmeans.py:205-221: fp32 sums cast to the value dtype."""
    s, _ = cluster_sums(value, a, nc)
    return _to_bf16(s, value.dtype)


def reverse_index(a: np.ndarray, nc: int):
    """kmeans.py:155-173: inverted lists [nc, max size] zero padded + sizes; ascending token
    order inside a list (the reference leaves that order to its atomics)."""
    cnt = np.bincount(a, minlength=nc).astype(np.int32)
    order = np.argsort(a, kind="stable")
    mx = max(int(cnt.max()), 1)
    lists = np.zeros((nc, mx), dtype=np.int32)
    off = np.concatenate([[0], np.cumsum(cnt)])
    for c in range(nc):
        lists[c, :cnt[c]] = order[off[c]:off[c + 1]]
    return lists, cnt


def segment_k_means(key, value, num_centroids, num_iters=10, num_segments=1):
    """kmeans.py:224-259.  key/value [G, N, D] bf16.  Returns (centroids [G, nc, D] bf16,
    value_sum [G, nc, D] bf16, clusters [G, nc, max] int32, cluster_size [G, nc] int32,
    assign [G, N])."""
    G, N, D = key.shape
    nc = num_centroids
    assert nc % num_segments == 0
    idx = init_indices(N, nc)
    cent = key[:, idx].clone()
    nseg = N // num_segments
    ncs = nc // num_segments
    for g in range(G):
        for s in range(num_segments):
            d = key[g, s * nseg:(s + 1) * nseg]
            c = cent[g, s * ncs:(s + 1) * ncs]
            for _ in range(num_iters - 1):
                c, _, _ = train_step(d, c, True)
            cent[g, s * ncs:(s + 1) * ncs] = c
    assigns = np.zeros((G, N), dtype=np.int64)
    vsum = torch.zeros(G, nc, D, dtype=value.dtype)
    lists, sizes = [], []
    for g in range(G):
        c, a, cnt = train_step(key[g], cent[g], False)
        cent[g] = c
        assigns[g] = a
        vsum[g] = value_sum(value[g], a, nc)
        l, sz = reverse_index(a, nc)
        lists.append(l)
        sizes.append(sz)
    mx = max(l.shape[1] for l in lists)
    clusters = np.zeros((G, nc, mx), dtype=np.int32)
    for g, l in enumerate(lists):
        clusters[g, :, :l.shape[1]] = l
    return cent, vsum, torch.from_numpy(clusters), torch.from_numpy(np.stack(sizes)), assigns
