"""Torch-facing wrappers of the C ABI.  The first block keeps the names and argument order of
the reference's `retroinfer_kernels` extension and of `weighted_flash_decoding`
(library/retroinfer/retroinfer_kernels/src/*.cu, *.cpp pybind sections), so code written
against the reference runs unchanged; the second block exposes the fused MI355X entry points.

Tensors only provide memory and the current stream; all arithmetic happens in the library.
"""
import contextlib
import functools
import math

import torch

from ._lib import lib, check

# 16-bit element types of the reference's operators and cache (batch_gemm_softmax.cu:185-197,
# gather_copy.cu:63-67): every wrapper takes either and calls the entry point of that type (name or name_f16).
_DT = (torch.bfloat16, torch.float16)


def _fn(name, dtype):
    """The entry point `name` for 16-bit tensors of `dtype`."""
    if dtype not in _DT:
        raise RuntimeError("Only Half and BFloat16 are supported")
    return getattr(lib(), name + "_f16" if dtype == torch.float16 else name)

# Named profiler ranges around the stages of a decode step, with the names the reference gives its NVTX
# ranges (cache_hub/retroinfer_cache.py:558-678); torch's nvtx calls are roctx ranges on ROCm, so
# rocprofv3 --marker-trace shows them.  Off except inside `with profiler_ranges(True)`, which a cache built
# with profiler_ranges=True holds around its own calls (so one cache's ranges do not switch on another's).
PROFILER_RANGES = False


@contextlib.contextmanager
def profiler_ranges(enabled):
    global PROFILER_RANGES
    before, PROFILER_RANGES = PROFILER_RANGES, bool(enabled)
    try:
        yield
    finally:
        PROFILER_RANGES = before


def _ranged(name):
    def deco(fn):
        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            if not PROFILER_RANGES:
                return fn(*args, **kwargs)
            torch.cuda.nvtx.range_push(name)
            try:
                return fn(*args, **kwargs)
            finally:
                torch.cuda.nvtx.range_pop()
        return wrapper
    return deco


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


def _need(t, dtype, name, cuda=True):
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if cuda and not t.is_cuda:
        raise ValueError(f"{name}: expected a device tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous tensor")


_workspaces = {}
_retired_workspaces = []   # superseded scratch tensors: captured HIP graphs may still hold their addresses


def _workspace(nbytes, device, tag):
    """Per-(device, tag) scratch tensor, grown on demand and reused across calls.  It starts
    zeroed: the attention kernels keep arrival counters in it that they leave at zero.
    A scratch tensor that is outgrown is never freed: a HIP graph captured earlier replays with its
    address, so handing the block back to the allocator would let that replay write into someone else's
    memory.  Growing (or first use) during a capture is refused: the allocation would land in the graph's
    private pool and its zero fill would become a memset node of the graph."""
    key = (str(device), tag)
    w = _workspaces.get(key)
    if w is None or w.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(f"scratch area '{tag}' must grow to {nbytes} bytes during a stream capture: run the "
                               "same call once before capturing")
        if w is not None:
            _retired_workspaces.append(w)
            nbytes = max(nbytes, w.numel() * 3 // 2)
        w = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=device)
        _workspaces[key] = w
    return w


def reset_attention_workspaces():
    """Clears the arrival counters of every attention scratch tensor (on the current stream of its device).
    The attention launches leave them at zero; call this after a launch that did not run to its end."""
    for (dev, tag), w in _workspaces.items():
        if tag.startswith("attn"):
            with torch.cuda.device(w.device):
                check(lib().ri_attention_workspace_reset(_p(w), w.numel(), _stream()), "attention_workspace_reset")


def release_cached_graphs(retired_workspaces=True):
    """Drops what the library keeps alive for replays: the captured clusterings of segment_k_means_csr (only the
    library replays those, so this is always safe) and, with retired_workspaces, the scratch tensors that were
    outgrown.  A graph that a caller captured while such a tensor was current still holds its address: drop the
    retired tensors only when every graph captured before the last growth of a scratch area is gone, or a replay
    would write into memory that has been handed back.  Refused during a stream capture."""
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("release_cached_graphs during a stream capture")
    from .cache_hub import kmeans as _km
    _km._GRAPHS.clear()
    _km._SEEN.clear()
    if retired_workspaces:
        _retired_workspaces.clear()


# limits of the fused decode path (checked by the entry points; callers can check them up front)
MAX_PROBES = 4096          # ri_score_select / ri_wave_attention / ri_lru_access_update: retrieval zone per group
MAX_CLUSTERS = 65536       # ri_score_select / ri_lru_access_update: clusters per group (16-bit ids in the selection)
MAX_GROUP_SIZE = 16        # query heads per KV head
MAX_GROUPS = 4096          # ri_wave_attention / ri_weighted_flash_decoding: batch x KV heads of one launch


# ----------------------------------------------------------------------------------------
# retroinfer_kernels-compatible surface
# ----------------------------------------------------------------------------------------
def batch_gemm_softmax(A, B, D, Norm, Sum, Softmax, batch_count, m, n, k, alpha=1.0, beta=0.0):
    """batch_gemm_softmax.cu:201-209.  A [bc, m, k], B [bc, n, k]; D/Softmax [bc, m, n]."""
    if A.dtype not in _DT:
        raise RuntimeError("Only Half and BFloat16 are supported")      # batch_gemm_softmax.cu:196
    for t, nm in ((A, "A"), (B, "B"), (D, "D"), (Softmax, "Softmax")):
        _need(t, A.dtype, nm)
    _need(Norm, torch.float32, "Norm"); _need(Sum, torch.float32, "Sum")
    ntiles = (n + 255) // 256
    if A.numel() < batch_count * m * k or B.numel() < batch_count * n * k or \
            D.numel() < batch_count * m * n or Softmax.numel() < batch_count * m * n or \
            Norm.numel() < batch_count * ntiles * m or Sum.numel() < batch_count * ntiles * m:
        raise ValueError("batch_gemm_softmax: a buffer is smaller than its shape arguments")
    fn = lib().ri_batch_gemm_softmax_f16 if A.dtype == torch.float16 else lib().ri_batch_gemm_softmax
    check(fn(_p(A), _p(B), _p(D), _p(Norm), _p(Sum), _p(Softmax), batch_count, m, n, k, float(alpha), float(beta),
             _stream()), "batch_gemm_softmax")


def gather_copy_vectors(key_data, key_buffer, value_data, value_buffer, src_metadata, dst_metadata,
                        data_offsets, groups, data_length, buffer_length, index_size, copy_start, copy_num):
    """gather_copy.cu:288-292.  The rows are moved as 16-bit elements: Half or BFloat16 (gather_copy.cu:63-67)."""
    if key_data.dtype not in _DT:
        raise RuntimeError("Only Half and BFloat16 are supported")
    for t, nm in ((key_data, "key_data"), (key_buffer, "key_buffer"), (value_data, "value_data"),
                  (value_buffer, "value_buffer"), (src_metadata, "src_metadata"), (dst_metadata, "dst_metadata")):
        _need(t, key_data.dtype, nm)
    _need(data_offsets, torch.int64, "data_offsets")
    if key_data.numel() < groups * data_length * 128 or key_buffer.numel() < groups * buffer_length * 128 or \
            data_offsets.numel() < groups * index_size or src_metadata.numel() < groups * data_length or \
            dst_metadata.numel() < groups * buffer_length:
        raise ValueError("gather_copy_vectors: a buffer is smaller than its shape arguments")
    check(lib().ri_gather_copy_vectors(_p(key_data), _p(key_buffer), _p(value_data), _p(value_buffer),
                                       _p(src_metadata), _p(dst_metadata), _p(data_offsets), groups, data_length,
                                       buffer_length, index_size, copy_start, copy_num, _stream()),
          "gather_copy_vectors")


@_ranged("gather_copy_and_concat")
def gather_copy_and_concat(key_data1, key_data2, key_data3, key_buffer, value_data1, value_data2, value_data3,
                           value_buffer, data_offsets2, data_copy_sizes2, buffer_offsets2, copy_chunks2,
                           data_offsets3, data_copy_sizes3, buffer_offsets3, copy_chunks3, valid_lengths,
                           groups, data_length1, data_length2, data_length3, buffer_length, offset_length,
                           copy_vectors1):
    """gather_copy.cu:294-300.  key_data2/value_data2 and the index tensors may be pinned host
    tensors (read in place by the kernel), everything else lives on the device."""
    for t in (data_offsets2, data_copy_sizes2, buffer_offsets2, copy_chunks2, data_offsets3, data_copy_sizes3,
              buffer_offsets3, copy_chunks3, valid_lengths):
        _need(t, torch.int32, "index tensor", cuda=False)
        if not (t.is_cuda or t.is_pinned()):
            raise ValueError("index tensors must be device or pinned host tensors")
    for t in (key_data2, value_data2):
        if not (t.is_cuda or t.is_pinned()):
            raise ValueError("key_data2/value_data2 must be device or pinned host tensors")
    check(lib().ri_gather_copy_and_concat(
        _p(key_data1), _p(key_data2), _p(key_data3), _p(key_buffer), _p(value_data1), _p(value_data2),
        _p(value_data3), _p(value_buffer), _p(data_offsets2), _p(data_copy_sizes2), _p(buffer_offsets2),
        _p(copy_chunks2), _p(data_offsets3), _p(data_copy_sizes3), _p(buffer_offsets3), _p(copy_chunks3),
        _p(valid_lengths), groups, data_length1, data_length2, data_length3, buffer_length, offset_length,
        copy_vectors1, _stream()), "gather_copy_and_concat")


def gather_copy_and_scatter(key_data, key_buffer, value_data, value_buffer, s_offsets, copy_sizes, d_offsets,
                            copy_chunks, groups, data_length, buffer_length, offset_length, s_copy_start):
    """gather_copy.cu:302-305."""
    for t in (s_offsets, copy_sizes, d_offsets, copy_chunks):
        _need(t, torch.int32, "index tensor", cuda=False)
        if not (t.is_cuda or t.is_pinned()):
            raise ValueError("index tensors must be device or pinned host tensors")
    check(lib().ri_gather_copy_and_scatter(_p(key_data), _p(key_buffer), _p(value_data), _p(value_buffer),
                                           _p(s_offsets), _p(copy_sizes), _p(d_offsets), _p(copy_chunks), groups,
                                           data_length, buffer_length, offset_length, s_copy_start, _stream()),
          "gather_copy_and_scatter")


@_ranged("flash_attention")
def weighted_flash_decoding(q, k, v, weight=None, previous_out=None, previous_lse=None, cache_seqlens=None,
                            return_softmax_lse=False):
    """Signature of the calls at cache_hub/retroinfer_cache.py:611-617 and :666-674.
    q [BG, 1, gs, D]; k, v [BG, S, 1, D]; weight [BG, 1, 1, S]; previous_out [BG, 1, gs, D];
    previous_lse [BG, gs] (any shape with BG*gs elements); cache_seqlens [BG] int32."""
    BG, one, gs, D = q.shape
    S = k.shape[1]
    if one != 1 or D != 128 or k.shape[2] != 1:
        raise ValueError("weighted_flash_decoding: expected q [BG,1,gs,128], k/v [BG,S,1,128]")
    dt = q.dtype
    for t, nm in ((q, "q"), (k, "k"), (v, "v")):
        _need(t, dt, nm)
    if weight is not None:
        _need(weight, dt, "weight")
    if previous_out is not None:
        _need(previous_out, dt, "previous_out")
        _need(previous_lse, torch.float32, "previous_lse")
    if cache_seqlens is not None:
        _need(cache_seqlens, torch.int32, "cache_seqlens")
    out = torch.empty_like(q)
    lse = torch.empty((BG, gs), dtype=torch.float32, device=q.device) if return_softmax_lse else None
    nb = lib().ri_flash_decoding_workspace_bytes(BG, gs)
    ws = _workspace(nb, q.device, "attn")
    check(_fn("ri_weighted_flash_decoding", dt)(_p(q), _p(k), _p(v), _p(weight), _p(cache_seqlens), _p(previous_out),
                                           _p(previous_lse), _p(out), _p(lse), BG, gs, S, S,
                                           1.0 / math.sqrt(D), _p(ws), ws.numel(), _stream()),
          "weighted_flash_decoding")
    return (out, lse) if return_softmax_lse else out


class ThreadPool:
    """wave_buffer_cpu.cpp:17-35.  first_core (None: workers run where the scheduler puts them): worker i is
    bound to core first_core + i, which is what the reference does with first_core = 0
    (thread_pool.hpp:18-23, 65-66); pinned_workers tells how many the system accepted."""

    def __init__(self, num_threads, first_core=None):
        self._destroy = lib().ri_threadpool_destroy   # bound now: module globals may be gone at interpreter exit
        if first_core is None:
            self._h = lib().ri_threadpool_create(int(num_threads))
        else:
            self._h = lib().ri_threadpool_create_pinned(int(num_threads), int(first_core))
        if not self._h:
            raise RuntimeError("ri_threadpool_create failed")
        self.pinned_workers = lib().ri_threadpool_pinned_workers(self._h)

    def get(self):
        return self

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._destroy(h)


class WaveBufferCPU:
    """wave_buffer_cpu.cpp:822-841.  Keeps references to every registered tensor, because the
    native object stores their addresses."""

    def __init__(self, batch_size, group_num, dim, nprobe, block_size, n_centroids, final_n_centroids,
                 buffer_size, capacity, threads, pool):
        self._pool = pool
        self._keep = {}
        self._destroy = lib().ri_wavebuf_destroy
        self._h = lib().ri_wavebuf_create(batch_size, group_num, dim, nprobe, block_size, n_centroids,
                                          final_n_centroids, buffer_size, capacity, threads, pool._h)
        if not self._h:
            raise ValueError("WaveBufferCPU: invalid construction arguments")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._destroy(h)

    def set_indices(self, hit_block_ids, hit_block_sizes, hit_block_sizes_cumsum, hit_block_nums,
                    miss_block_ids, miss_block_sizes, miss_block_sizes_cumsum, miss_block_nums,
                    update_buffer_indices, update_block_sizes, update_cache_indices, update_block_nums,
                    searched_clusters):
        ts = [hit_block_ids, hit_block_sizes, hit_block_sizes_cumsum, hit_block_nums, miss_block_ids,
              miss_block_sizes, miss_block_sizes_cumsum, miss_block_nums, update_buffer_indices,
              update_block_sizes, update_cache_indices, update_block_nums]
        for t in ts:
            _need(t, torch.int32, "index tensor", cuda=False)
        _need(searched_clusters, torch.int64, "searched_clusters", cuda=False)
        self._keep["indices"] = ts + [searched_clusters]
        check(lib().ri_wavebuf_set_indices(self._h, *[_p(t) for t in ts], _p(searched_clusters)), "set_indices")

    def set_kv(self, ivf_key, ivf_value, input_keys, input_values):
        self._keep["kv"] = [ivf_key, ivf_value, input_keys, input_values]
        check(lib().ri_wavebuf_set_kv(self._h, _p(ivf_key), _p(ivf_value), ivf_key.size(2), _p(input_keys),
                                      _p(input_values), input_keys.size(1)), "set_kv")

    def async_construction(self, clusters, cluster_size, batch_idx):
        _need(clusters, torch.int32, "clusters", cuda=False)
        _need(cluster_size, torch.int32, "cluster_size", cuda=False)
        self._keep["construction"] = [clusters, cluster_size]
        check(lib().ri_wavebuf_async_construction(self._h, _p(clusters), _p(cluster_size), clusters.size(2),
                                                  int(batch_idx)), "async_construction")

    def construction_sync(self):
        check(lib().ri_wavebuf_construction_sync(self._h), "construction_sync")

    def update_kv(self, update_keys, update_values, clusters, cluster_size):
        _need(clusters, torch.int32, "clusters", cuda=False)
        _need(cluster_size, torch.int32, "cluster_size", cuda=False)
        check(lib().ri_wavebuf_update_kv(self._h, _p(update_keys), _p(update_values), update_keys.size(1),
                                         _p(clusters), _p(cluster_size), clusters.size(1), clusters.size(2)),
              "update_kv")

    def batch_access(self):
        check(lib().ri_wavebuf_batch_access(self._h), "batch_access")

    def sync(self):
        check(lib().ri_wavebuf_sync(self._h), "sync")

    def overflow_events(self):
        return int(lib().ri_wavebuf_overflow_events(self._h))


# ----------------------------------------------------------------------------------------
# fused MI355X entry points
# ----------------------------------------------------------------------------------------
@_ranged("search_topk_clusters")
def score_select(q, centroids, mask, cluster_size_i32, cluster_start, logits, dist, cI, ret_ids, est_ids,
                 ret_tok_off, row_src, meta, nprobe, es, page, max_pages, scale, slot=0, ret_start=None):
    """Centroid scoring + retrieval/estimation selection + token layout.  `slot` names the
    scratch area: calls that may run concurrently (different streams) must use different slots.
    The layout goes out as a row table (row_src), as rank tables (ret_tok_off + ret_start), or both."""
    BG, gs, D = q.shape
    nc = centroids.shape[1]
    nb = lib().ri_score_select_workspace_bytes(BG, gs, nc)
    ws = _workspace(nb, q.device, f"score{slot}")
    _need(centroids, q.dtype, "centroids")
    check(_fn("ri_score_select", q.dtype)(_p(q), _p(centroids), _p(mask), _p(cluster_size_i32), _p(cluster_start),
                                _p(logits), _p(dist), _p(cI), _p(ret_ids), _p(est_ids), _p(ret_tok_off),
                                _p(ret_start), _p(row_src), 0 if row_src is None else row_src.shape[1], _p(meta),
                                BG, gs, nc,
                                nprobe, es, page, max_pages, float(scale), _p(ws), ws.numel(), _stream()),
          "score_select")


def score_logits(q, centroids, logits, scale, slot=0):
    """logits [BG, gs, nc] fp32 = scale * q . centroids^T, no selection."""
    BG, gs, D = q.shape
    nc = centroids.shape[1]
    ws = _workspace(lib().ri_score_select_workspace_bytes(BG, gs, nc), q.device, f"score{slot}")
    _need(centroids, q.dtype, "centroids")
    check(_fn("ri_score_logits", q.dtype)(_p(q), _p(centroids), _p(logits), BG, gs, nc, float(scale), _p(ws), ws.numel(),
                                _stream()), "score_logits")


@_ranged("flash_attention")
def wave_attention(q, steady_k, steady_v, static_len, store_k, store_v, row_src, meta, est_ids, logits,
                   value_sum, cluster_size_bf16, out, valid_lengths, es, scale, slot=0, ret_tok_off=None,
                   ret_start=None, est_centroids=None, static_len_dev=None):
    """Attention over steady zone + retrieved clusters (read in place) + estimation zone.
    The retrieved rows come from a row table (row_src) or, with row_src None, from the rank tables
    ret_tok_off [BG, np+1] and ret_start [BG, np].  The estimation zone's scores are read from `logits`
    or, with logits None, computed in the launch from the rows of `est_centroids` [BG, nc, 128].
    With static_len_dev (int32 tensor of one element on the device) the number of steady rows is read
    from it when the kernel runs; static_len then only sizes the split.
    `slot`: scratch area, one per concurrent call."""
    BG, gs, D = q.shape
    nc = value_sum.shape[1]
    nb = lib().ri_wave_attention_workspace_bytes(BG, gs)
    ws = _workspace(nb, q.device, f"attn{slot}")
    for t, nm in ((steady_k, "steady_k"), (store_k, "store_k"), (value_sum, "value_sum"), (out, "out")):
        _need(t, q.dtype, nm)
    check(_fn("ri_wave_attention", q.dtype)(_p(q), _p(steady_k), _p(steady_v), steady_k.shape[-2], static_len,
                                  _p(static_len_dev), _p(store_k),
                                  _p(store_v), store_k.shape[-2], _p(row_src),
                                  0 if row_src is None else row_src.shape[1], _p(ret_tok_off), _p(ret_start),
                                  0 if ret_start is None else ret_start.shape[1], _p(meta), _p(est_ids), _p(logits),
                                  _p(est_centroids), _p(value_sum), _p(cluster_size_bf16), _p(out),
                                  _p(valid_lengths), BG, gs, nc, es, float(scale), _p(ws), ws.numel(), _stream()),
          "wave_attention")


@_ranged("flash_attention")
def wave_attention_part(q, steady_k, steady_v, static_len, store_k, store_v, row_src, src_row_lo, src_row_hi, meta,
                        est_ids, logits, value_sum, cluster_size_bf16, out, lse_out, es, scale, prev_out=None,
                        prev_lse=None, valid_lengths=None, slot=0):
    """wave_attention over the rows of the row table whose source row lies in [src_row_lo, src_row_hi), merging an
    earlier part's (prev_out, prev_lse) and returning this part's log-sum-exp in lse_out [BG, gs] fp32."""
    BG, gs, D = q.shape
    nc = value_sum.shape[1]
    ws = _workspace(lib().ri_wave_attention_workspace_bytes(BG, gs), q.device, f"attn{slot}")
    check(_fn("ri_wave_attention_part", q.dtype)(
        _p(q), _p(steady_k), _p(steady_v), steady_k.shape[-2], static_len, None, _p(store_k), _p(store_v),
        store_k.shape[-2], _p(row_src), row_src.shape[1], int(src_row_lo), int(src_row_hi), _p(meta), _p(est_ids),
        _p(logits), _p(value_sum), _p(cluster_size_bf16), _p(prev_out), _p(prev_lse), _p(out), _p(lse_out),
        _p(valid_lengths), BG, gs, nc, es, float(scale), _p(ws), ws.numel(), _stream()), "wave_attention_part")


@_ranged("flash_attention")
def wave_attention_static(q, steady_k, steady_v, static_len, store_k, store_v, row_src, meta, est_ids, logits,
                          value_sum, cluster_size_bf16, out, valid_lengths, es, scale, ret_tok_off=None,
                          ret_start=None, est_centroids=None, static_len_dev=None):
    """wave_attention without a scratch tensor: the library keeps the scratch in a static device array
    (ri_wave_attention_static), so the call allocates nothing.  Calls on one GPU must not overlap."""
    BG, gs, D = q.shape
    nc = value_sum.shape[1]
    check(_fn("ri_wave_attention_static", q.dtype)(
        _p(q), _p(steady_k), _p(steady_v), steady_k.shape[-2], static_len, _p(static_len_dev), _p(store_k),
        _p(store_v), store_k.shape[-2], _p(row_src), 0 if row_src is None else row_src.shape[1], _p(ret_tok_off),
        _p(ret_start), 0 if ret_start is None else ret_start.shape[1], _p(meta), _p(est_ids), _p(logits),
        _p(est_centroids), _p(value_sum), _p(cluster_size_bf16), _p(out), _p(valid_lengths), BG, gs, nc, es,
        float(scale), _stream()), "wave_attention_static")


def buffer_attention(q, buf_k, buf_v, cache_seqlens, est_ids, logits, value_sum, cluster_size_bf16, out, es, scale,
                     slot=0):
    """Attention over the rows [0, cache_seqlens[g]) of an execution buffer [BG, stride, 128] with the
    estimation zone (ids and logits from score_select) merged in the same launch."""
    BG, gs, D = q.shape
    nc = value_sum.shape[1]
    stride = buf_k.shape[-3] if buf_k.dim() == 4 else buf_k.shape[-2]
    ws = _workspace(lib().ri_wave_attention_workspace_bytes(BG, gs), q.device, f"attn{slot}")
    check(_fn("ri_buffer_attention", q.dtype)(_p(q), _p(buf_k), _p(buf_v), stride, _p(cache_seqlens), stride, _p(est_ids),
                                    _p(logits), _p(value_sum), _p(cluster_size_bf16), _p(out), BG, gs, nc, es,
                                    float(scale), _p(ws), ws.numel(), _stream()), "buffer_attention")


class DeviceLru:
    """State of the device-side block cache manager of one layer (ri_lru_access_update)."""

    def __init__(self, BG, max_clusters, max_blocks, capacity, buffer_size, block, device):
        i32 = lambda *s: torch.zeros(s, dtype=torch.int32, device=device)
        self.BG, self.capacity, self.buffer_size, self.block = BG, capacity, buffer_size, block
        self.stamp = i32(BG, max_clusters)     # step that last touched a resident cluster (0: not resident)
        self.order = i32(BG, max_clusters)     # ... and the cluster's position inside that step
        self.blk_off = i32(BG, max_clusters + 1)
        self.blk_ids = i32(BG, max_blocks)
        self.free_list = torch.arange(capacity, dtype=torch.int32, device=device).repeat(BG, 1).contiguous()
        self.free_count = torch.full((BG,), capacity, dtype=torch.int32, device=device)
        self.epoch = i32(BG)

    def set_sizes(self, sizes_i32):
        """sizes_i32 [BG, ncl]: recompute the block offsets (offsets of existing clusters do not move
        when clusters are appended)."""
        nb = (sizes_i32.to(torch.int64) + self.block - 1) // self.block
        ncl = sizes_i32.shape[1]
        self.blk_off[:, 1:ncl + 1] = torch.cumsum(nb, 1).to(torch.int32)
        assert int(self.blk_off[:, ncl].max()) <= self.blk_ids.shape[1]

    def access_update(self, ret_ids, sizes, starts, lists, row_src=None, stage_row0=0, meta=None):
        """lists: the 12 tensors hit (ids, sizes, cumsum, num), miss (...), update (buf, sizes, cache, num).
        row_src / meta: row table for attention in place (hits are then not listed for copying)."""
        BG, np_ = ret_ids.shape
        ncl = sizes.shape[1]
        check(lib().ri_lru_access_update(
            _p(ret_ids), _p(sizes), _p(starts), sizes.stride(0), _p(self.blk_off), self.blk_off.shape[1],
            _p(self.stamp), _p(self.order), self.stamp.shape[1], _p(self.blk_ids), self.blk_ids.shape[1], _p(self.free_list),
            _p(self.free_count), _p(self.epoch), *[_p(t) for t in lists], _p(row_src),
            0 if row_src is None else row_src.shape[1], stage_row0, _p(meta), BG, np_, ncl, self.buffer_size,
            self.capacity, self.block, _stream()), "lru_access_update")


def kmeans_assign(data, centroids, assign, P, N, nc, seg, head_rows):
    check(_fn("ri_kmeans_assign", data.dtype)(_p(data), _p(centroids), _p(assign), P, N, nc, seg, head_rows, _stream()),
          "kmeans_assign")


def kmeans_build_lists(assign, counts, offsets, members, P, N, nc, slot=0):
    """`slot` names the scratch area: calls that may run concurrently (different streams) use different slots."""
    nb = lib().ri_kmeans_workspace_bytes(P, N, nc)
    ws = _workspace(nb, assign.device, f"kmeans{slot}")
    check(lib().ri_kmeans_build_lists(_p(assign), _p(counts), _p(offsets), _p(members), P, N, nc, _p(ws),
                                      ws.numel(), _stream()), "kmeans_build_lists")


def kmeans_update(data, counts, offsets, members, centroids, P, N, nc, seg, head_rows, normalize, slot=0):
    ws = _workspace(lib().ri_kmeans_reduce_workspace_bytes(P, N, nc), data.device, f"kmeans_reduce{slot}")
    check(_fn("ri_kmeans_update", data.dtype)(_p(data), _p(counts), _p(offsets), _p(members), _p(centroids), P, N, nc, seg,
                                 head_rows, int(bool(normalize)), _p(ws), ws.numel(), _stream()), "kmeans_update")


def kmeans_value_sum(values, counts, offsets, members, value_sum, P, N, nc, slot=0):
    ws = _workspace(lib().ri_kmeans_reduce_workspace_bytes(P, N, nc), values.device, f"kmeans_reduce{slot}")
    check(_fn("ri_kmeans_value_sum", values.dtype)(_p(values), _p(counts), _p(offsets), _p(members), _p(value_sum), P, N, nc,
                                    _p(ws), ws.numel(), _stream()), "kmeans_value_sum")


def permute_rows(src, members, dst, P, N, in_stride_rows, out_stride_rows):
    check(lib().ri_permute_rows(_p(src), _p(members), _p(dst), P, N, in_stride_rows, out_stride_rows, _stream()),
          "permute_rows")
