"""segment_k_means with the reference's signature and return values
(cache_hub/kmeans.py:224-259 of the reference), driven by the gfx950 kernels.

Differences that a caller can observe, both within what the reference leaves open:
  * cluster sums are accumulated in a fixed order (fp32: ascending token order in blocks of 256
    tokens, block sums added in block order) instead of by atomics, so the result is
    reproducible run to run;
  * tokens inside a cluster list are ascending (the reference's order is whatever its atomics
    produced).
"""
import collections

import torch

from .. import kernels


def init_centroid_indices(num_tokens, num_centroids, device):
    """kmeans.py:234-236: float32 arithmetic, truncated to int64."""
    idx = torch.arange(num_centroids, dtype=torch.float32, device=device) * (num_tokens / num_centroids)
    idx += num_tokens / num_centroids / 2
    return idx.to(torch.int64)


class KMeansResult:
    """CSR form of the clustering, kept on the device."""
    __slots__ = ("centroids", "value_sum", "assign", "counts", "offsets", "members")


def _cluster(key, num_centroids, num_iters, num_segments, init_indices):
    """Everything of the clustering that reads the keys: centroids, assignment, inverted lists."""
    G, N, D = key.shape
    dev = key.device
    nc, S = num_centroids, num_segments
    if init_indices is None:
        init_indices = init_centroid_indices(N, nc, dev)
    centroids = torch.index_select(key, 1, init_indices).contiguous()
    nseg, ncs = N // S, nc // S
    P = G * S
    assign = torch.empty((P, max(nseg, 1)), dtype=torch.int32, device=dev)
    counts = torch.empty((P, ncs), dtype=torch.int32, device=dev)
    offsets = torch.empty((P, ncs + 1), dtype=torch.int32, device=dev)
    members = torch.empty((P, max(nseg, 1)), dtype=torch.int32, device=dev)
    if nseg > 0:
        for _ in range(num_iters - 1):
            kernels.kmeans_assign(key, centroids, assign, P, nseg, ncs, S, N)
            kernels.kmeans_build_lists(assign, counts, offsets, members, P, nseg, ncs)
            kernels.kmeans_update(key, counts, offsets, members, centroids, P, nseg, ncs, S, N, True)
    r = KMeansResult()
    r.assign = torch.empty((G, N), dtype=torch.int32, device=dev)
    r.counts = torch.empty((G, nc), dtype=torch.int32, device=dev)
    r.offsets = torch.empty((G, nc + 1), dtype=torch.int32, device=dev)
    r.members = torch.empty((G, N), dtype=torch.int32, device=dev)
    kernels.kmeans_assign(key, centroids, r.assign, G, N, nc, 1, N)
    kernels.kmeans_build_lists(r.assign, r.counts, r.offsets, r.members, G, N, nc)
    kernels.kmeans_update(key, r.counts, r.offsets, r.members, centroids, G, N, nc, 1, N, False)
    r.centroids = centroids
    return r


# Captured clusterings, newest last: (key pointer, shape, parameters) -> (graph, result).  A clustering is
# about a hundred short launches; replayed as one HIP graph it loses the gaps between them.  The graph
# reads the key tensor afresh on every replay, so only the address has to stay the same, not the content.
_GRAPHS = collections.OrderedDict()
_SEEN = collections.OrderedDict()
_MAX_GRAPHS = 4


def segment_k_means_csr(key, value, num_centroids, num_iters=10, num_segments=1, init_indices=None,
                        reuse_graph=False):
    """Runs the clustering and returns a KMeansResult (no dense cluster lists, no host copy).
    key/value [G, N, 128] bfloat16 or float16 contiguous device tensors.

    reuse_graph (off unless asked for): the second call with keys at the same address and the same
    shape and parameters captures the launches into a HIP graph, and later such calls replay it.
    Results of replayed calls live in the graph's own memory: THEY ARE OVERWRITTEN by the next replay
    for the same key tensor, so only a caller that consumes or copies them before its next call may
    turn this on (prefill_update_kv_cache does: it copies everything into the cache's tensors at once;
    value sums are always fresh)."""
    G, N, D = key.shape
    if D != 128 or key.dtype not in (torch.bfloat16, torch.float16) or not key.is_contiguous():
        raise ValueError("segment_k_means: expected contiguous bfloat16 or float16 [G, N, 128] keys")
    if value.dtype != key.dtype:
        raise ValueError("segment_k_means: keys and values must have the same element type")
    if num_centroids % num_segments != 0:
        raise AssertionError("num_centroids must be divisible by num_segments")
    nc, S = num_centroids, num_segments
    if (nc // S) % 32 != 0 or nc % 32 != 0:
        raise AssertionError("centroids per segment must be a multiple of 32")  # kmeans.py:99
    value = value.contiguous()
    r = None
    if reuse_graph and not torch.cuda.is_current_stream_capturing():
        gkey = (key.data_ptr(), tuple(key.shape), str(key.device), nc, num_iters, S,
                None if init_indices is None else init_indices.data_ptr())
        hit = _GRAPHS.get(gkey)
        if hit is None and gkey in _SEEN:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                res = _cluster(key, nc, num_iters, S, init_indices)
            hit = (graph, res, init_indices)          # (the index tensor stays alive with the graph)
            _GRAPHS[gkey] = hit
            while len(_GRAPHS) > _MAX_GRAPHS:
                _GRAPHS.popitem(last=False)
        if hit is not None:
            _GRAPHS.move_to_end(gkey)
            hit[0].replay()
            r = KMeansResult()
            for f in ("centroids", "assign", "counts", "offsets", "members"):
                setattr(r, f, getattr(hit[1], f))
        else:
            _SEEN[gkey] = True
            while len(_SEEN) > 64:
                _SEEN.popitem(last=False)
    if r is None:
        r = _cluster(key, nc, num_iters, S, init_indices)
    r.value_sum = torch.empty((G, nc, D), dtype=value.dtype, device=key.device)
    kernels.kmeans_value_sum(value, r.counts, r.offsets, r.members, r.value_sum, G, N, nc)
    return r


def csr_to_dense(counts, offsets, members):
    """[G, nc, max_cluster_size] zero-padded lists as triton_reverse_index returns them
    (kmeans.py:155-173)."""
    G, nc = counts.shape
    mx = max(int(counts.max().item()), 1)
    col = torch.arange(mx, device=counts.device)[None, None, :]
    valid = col < counts[:, :, None]
    src = (offsets[:, :nc, None].long() + col).clamp_max(members.shape[1] - 1)
    dense = torch.gather(members.long()[:, None, :].expand(G, nc, -1), 2, src)
    return torch.where(valid, dense, torch.zeros_like(dense)).to(torch.int32)


def segment_k_means(key, value, num_centroids, num_iters=10, num_segments=1):
    """Reference signature: returns (centroids, value_sum, clusters, cluster_size), tensors of the
    caller's own (no captured graph: its results would be overwritten by a later call)."""
    r = segment_k_means_csr(key.contiguous(), value, num_centroids, num_iters, num_segments, reuse_graph=False)
    return r.centroids, r.value_sum, csr_to_dense(r.counts, r.offsets, r.members), r.counts
