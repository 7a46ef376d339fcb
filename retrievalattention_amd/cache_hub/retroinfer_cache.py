"""retroinfer_cache: the wave-index KV cache with the reference's constructor, methods and
attributes (cache_hub/retroinfer_cache.py of the reference), running on the gfx950 library.

Two residencies of the clustered K/V:

  "device"  every cluster's K/V stays in HBM in cluster-contiguous order.  A decode step is
            two fused calls: score_select (scores, zones, rank tables) and wave_attention
            (steady zone + retrieved clusters read in place + estimation zone).  No host
            round trip, no execution buffer, no block cache.
  "host"    the reference's arrangement: clustered K/V in pinned host memory, an LRU block
            cache in HBM managed by the host wave buffer, misses read by the gather kernel
            straight from host memory, admission after the attention.

"auto" picks "device" when the store fits the memory the base class estimates to be free.
Buffer names follow the reference so that code poking at them keeps working.
"""
import math
import warnings

import torch

from .. import kernels
from .cache import KV_Cache
from .kmeans import segment_k_means_csr, csr_to_dense

# generated tokens are folded into the index every THRESHOLD_LENGTH steps
THRESHOLD_LENGTH = 1024


def _pinned(shape, dtype, fill=None):
    t = torch.empty(shape, dtype=dtype, pin_memory=True)
    if fill is not None:
        t.fill_(fill)
    return t


class retroinfer_cache(KV_Cache):
    def __init__(self, valid_start, layer_num, batch_size, max_length, num_key_value_heads, num_heads,
                 head_dim, dtype, layer_mapping, max_new_length, static_pattern_start, static_pattern_end, core,
                 n_centroids, n_segment, nprobe, max_compute_cluster_num, cache_unit_size, cache_cluster_num,
                 num_gpus, model_size, use_cluster_estimation=False, kv_residency="auto",
                 block_cache="device", device_positions=False, overlap_miss_staging=False, pin_workers=False,
                 profiler_ranges=False, reference_stale_row=False):
        super().__init__(layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                         layer_mapping, num_gpus, model_size)
        if head_dim != 128 or dtype not in (torch.bfloat16, torch.float16):
            raise ValueError("the gfx950 kernels are built for head_dim 128 and bfloat16 or float16")
        if cache_unit_size != 8:
            raise ValueError("cache_unit_size must be 8 (block size of the copy kernels)")
        # limits of the kernels, checked here so that they surface at construction and not at the first decode step
        n_new = ((max_new_length - 2) // THRESHOLD_LENGTH) * (((THRESHOLD_LENGTH // 16) // 32) * 32)
        if num_heads % num_key_value_heads != 0 or num_heads // num_key_value_heads > kernels.MAX_GROUP_SIZE:
            raise ValueError(f"at most {kernels.MAX_GROUP_SIZE} query heads per KV head (got {num_heads} / "
                             f"{num_key_value_heads})")
        if batch_size * num_key_value_heads > kernels.MAX_GROUPS:
            raise ValueError(f"at most {kernels.MAX_GROUPS} groups (batch x KV heads) per attention launch (got "
                             f"{batch_size} x {num_key_value_heads})")
        if not 1 <= nprobe <= kernels.MAX_PROBES:
            raise ValueError(f"nprobe must be in 1..{kernels.MAX_PROBES} (got {nprobe})")
        if n_centroids % 8 != 0 or n_centroids + n_new > kernels.MAX_CLUSTERS:
            raise ValueError(f"n_centroids must be a multiple of 8 and, with the clusters of generated tokens "
                             f"({n_new}), at most {kernels.MAX_CLUSTERS} (got {n_centroids})")
        if not nprobe <= max_compute_cluster_num <= n_centroids:
            raise ValueError(f"max_compute_cluster_num must lie between nprobe ({nprobe}) and n_centroids "
                             f"({n_centroids}) (got {max_compute_cluster_num})")
        if cache_cluster_num < 0:
            raise ValueError("cache_cluster_num must not be negative (0: no block cache, every retrieved cluster "
                             "is read from the host store)")
        self.valid_start = valid_start
        self.static_pattern_start = static_pattern_start
        self.static_pattern_end = static_pattern_end
        self.static_pattern_total = static_pattern_start + static_pattern_end
        self.group_size = self.num_heads // self.kv_head
        self.batch_groups = self.batch_size * self.kv_head
        self.page_size = cache_unit_size
        self.core = core
        self.use_cluster_estimation = use_cluster_estimation
        if block_cache not in ("device", "host"):
            raise ValueError("block_cache must be 'device' or 'host'")
        # who runs the block cache of a host-resident store: a kernel (no host round trip per step) or
        # the reference's worker threads (WaveBufferCPU.batch_access / sync)
        self.block_cache = block_cache
        # host-resident store with the device-side manager: attend the rows already in the block cache
        # (with the steady and estimation zones) while the missed blocks are still crossing the host link
        # on the copy stream, then the staged rows (reference: retroinfer_cache.py:629-657 overlaps that
        # transfer with other work of the step).  Off by default: the attention over the hits is ~30 us
        # of a step whose miss staging takes hundreds, and the second launch and the stream join cost
        # more than the overlap returns (measured at B=8, 8 KV heads, 120K tokens: 287 vs 270 us per
        # layer-step at 70 % hits, 93 vs 66 us with every block a hit)
        self.overlap_miss_staging = bool(overlap_miss_staging)
        # the reference's NVTX ranges (retroinfer_cache.py:558-678) as roctx ranges of the same names
        self.profiler_ranges = bool(profiler_ranges)
        self.pin_workers = bool(pin_workers)
        # worker-thread manager with next-layer estimation only: leave the layer's new token out of the
        # pre-assembled execution buffer, as the reference does (its attention then reads the stale row there)
        self.reference_stale_row = bool(reference_stale_row)

        self.input_length = self.max_length - max_new_length
        self.max_new_length = min(max_new_length - 1, THRESHOLD_LENGTH)  # one token comes out of prefill
        self.input_length_new = ((max_new_length - 2) // THRESHOLD_LENGTH) * THRESHOLD_LENGTH
        self.n_centroids_per_update_segment = ((THRESHOLD_LENGTH // 16) // 32) * 32
        self.n_centroids_new = ((max_new_length - 2) // THRESHOLD_LENGTH) * self.n_centroids_per_update_segment
        self.RSQRT_DIM = 1.0 / math.sqrt(self.head_dim)
        self.DTYPE_MIN = torch.finfo(self.dtype).min

        self.n_centroids = n_centroids
        self.n_segment = n_segment
        self.nprobe = nprobe
        self.max_compute_cluster_num = max_compute_cluster_num
        self.es_cluster_num = max_compute_cluster_num - nprobe

        avg_cluster_size = (self.input_length - self.static_pattern_total) // self.n_centroids
        pages_per_cluster = max(1, math.ceil(avg_cluster_size / self.page_size))
        self.cache_size = cache_cluster_num * pages_per_cluster
        self.buffer_size = max(int(self.nprobe * 4), 16) * pages_per_cluster
        self.static_stride = self.static_pattern_total + self.max_new_length
        self.list_stride = self.input_length - self.static_pattern_total + self.input_length_new
        self.execution_stride = self.buffer_size * self.page_size + self.static_stride
        self.cache_stride = self.cache_size

        if kv_residency not in ("auto", "device", "host"):
            raise ValueError("kv_residency must be 'auto', 'device' or 'host'")
        if kv_residency == "auto":
            store_gib = 2 * layer_num * self.batch_groups * self.list_stride * head_dim * 2 / 1024 ** 3
            kv_residency = "device" if store_gib * 1.25 < self.free_memory else "host"
        self.kv_residency = kv_residency
        if self.overlap_miss_staging and not (kv_residency == "host" and block_cache == "device"):
            warnings.warn("overlap_miss_staging only applies to a host-resident store with the device-side block "
                          "cache manager: ignored")
            self.overlap_miss_staging = False
        self.allocated = True  # the GPU side is always allocated up front on a 288 GB part

        dev = lambda ldx: self.layer_mapping[str(ldx)]
        BG, D = self.batch_groups, self.head_dim
        zeros = lambda shape, dt, d: torch.zeros(shape, dtype=dt, device=d)
        L = range(self.layer_num)
        self.steady_zone_keys = [zeros((batch_size, self.kv_head, self.static_stride, D), dtype, dev(l)) for l in L]
        self.steady_zone_values = [zeros((batch_size, self.kv_head, self.static_stride, D), dtype, dev(l)) for l in L]
        # meta index
        self.centroids = [zeros((BG, n_centroids, D), dtype, dev(l)) for l in L]
        self.value_sum = [zeros((BG, n_centroids, D), dtype, dev(l)) for l in L]
        self.centroids_mask = [zeros((BG, n_centroids), torch.bool, dev(l)) for l in L]
        self.cluster_size = [zeros((BG, n_centroids), dtype, dev(l)) for l in L]
        if self.input_length_new > 0 and self.kv_residency == "host":
            self.offload_update_keys = _pinned((BG, THRESHOLD_LENGTH, D), dtype)
            self.offload_update_values = _pinned((BG, THRESHOLD_LENGTH, D), dtype)

        # per cluster: first row in the (device or host) store and token count
        self.cluster_start = [zeros((BG, n_centroids), torch.int32, dev(l)) for l in L]
        self.cluster_size_i32 = [zeros((BG, n_centroids), torch.int32, dev(l)) for l in L]
        self.store_rows = [[0] * BG for _ in L]  # rows of the store in use, per group
        self._centred_keys = {}                  # (device, tokens) -> buffer of centred keys for the clustering
        if self.kv_residency == "device":
            self._init_device_store()
        else:
            self._init_wave_buffer()
        self.allocate_computation_buffer()

        # device_positions: the steady zone's length also lives in device memory, the new token's K/V is
        # written at that position by an indexed copy and the attention reads the length when it runs,
        # so a captured decode step (decode_update_kv_cache + compute of every layer) can be replayed
        # token after token; the host counters are then advanced by token_replayed()
        self.device_positions = bool(device_positions)
        if self.device_positions:
            if self.kv_residency != "device" or use_cluster_estimation or len(set(self.layer_mapping.values())) != 1:
                raise ValueError("device_positions needs a device-resident store on one device, without "
                                 "next-layer estimation")
            d0 = self.layer_mapping[str(0)]
            self.steady_len_dev = torch.tensor([self.static_pattern_total + 1], dtype=torch.int32, device=d0)
            self.steady_pos_dev = torch.tensor([self.static_pattern_total], dtype=torch.int64, device=d0)

        self.copystream = torch.cuda.Stream()
        self.mainevents, self.copyevents = {}, {}
        for d in sorted(set(self.layer_mapping.values()), key=lambda x: int(str(x).split(":")[-1])):
            with torch.cuda.device(d):
                self.mainevents[d] = torch.cuda.Event()
                self.copyevents[d] = torch.cuda.Event()

    # ------------------------------------------------------------------ allocation
    def _init_device_store(self):
        dev = lambda ldx: self.layer_mapping[str(ldx)]
        BG, D = self.batch_groups, self.head_dim
        L = range(self.layer_num)
        shape = (self.batch_size, self.kv_head, self.list_stride, D)
        self.list_keys = [torch.zeros(shape, dtype=self.dtype, device=dev(l)) for l in L]
        self.list_values = [torch.zeros(shape, dtype=self.dtype, device=dev(l)) for l in L]

    def _init_wave_buffer(self):
        dev = lambda ldx: self.layer_mapping[str(ldx)]
        zeros = lambda shape, dt, d: torch.zeros(shape, dtype=dt, device=d)
        BG, D = self.batch_groups, self.head_dim
        L = range(self.layer_num)
        # pin_workers: worker i on core i like the reference's pool (thread_pool.hpp:65-66); off by default,
        # because cores 0..n-1 are also where the interpreter's own thread usually runs
        self.thread_pool = kernels.ThreadPool(self.core, 0 if self.pin_workers else None)
        pool = self.thread_pool.get()
        self.wave_buffer = [kernels.WaveBufferCPU(
            self.batch_size, self.kv_head, D, self.nprobe, self.page_size, self.n_centroids,
            self.n_centroids + self.n_centroids_new, self.buffer_size, self.cache_size, self.core, pool) for _ in L]
        names = ["hit_unit_idices", "hit_unit_sizes", "hit_unit_sizes_cumsum", "miss_unit_idices", "miss_unit_sizes",
                 "miss_unit_sizes_cumsum", "update_buffer_indices", "update_unit_sizes", "update_cache_indices"]
        for nm in names:
            setattr(self, nm, [_pinned((BG, self.buffer_size), torch.int32, 0) for _ in L])
        for nm in ("hit_num_units", "miss_num_units", "update_num_units"):
            setattr(self, nm, [_pinned((BG,), torch.int32, 0) for _ in L])
        self._host_lists = None
        if self.block_cache == "device":
            # the worker-thread manager keeps its (unused) pinned lists; the copy kernels read these instead
            self._host_lists = {nm: getattr(self, nm) for nm in names + ["hit_num_units", "miss_num_units",
                                                                         "update_num_units"]}
            for nm in names:
                setattr(self, nm, [zeros((BG, self.buffer_size), torch.int32, dev(l)) for l in L])
            for nm in ("hit_num_units", "miss_num_units", "update_num_units"):
                setattr(self, nm, [zeros((BG,), torch.int32, dev(l)) for l in L])
            max_blocks = self.list_stride // self.page_size + self.n_centroids + self.n_centroids_new + 1
            self.device_lru = [kernels.DeviceLru(BG, self.n_centroids + self.n_centroids_new, max_blocks,
                                                 self.cache_size, self.buffer_size, self.page_size, dev(l)) for l in L]
        self.cluster_ids = [_pinned((BG, self.nprobe), torch.int64, 0) for _ in range(2)]
        for l in L:
            hl = self._host_lists if self._host_lists is not None else {nm: getattr(self, nm) for nm in names + [
                "hit_num_units", "miss_num_units", "update_num_units"]}
            self.wave_buffer[l].set_indices(
                hl["hit_unit_idices"][l], hl["hit_unit_sizes"][l], hl["hit_unit_sizes_cumsum"][l],
                hl["hit_num_units"][l], hl["miss_unit_idices"][l], hl["miss_unit_sizes"][l],
                hl["miss_unit_sizes_cumsum"][l], hl["miss_num_units"][l], hl["update_buffer_indices"][l],
                hl["update_unit_sizes"][l], hl["update_cache_indices"][l], hl["update_num_units"][l],
                self.cluster_ids[l % 2])
        # with the device-side manager the staging blocks of the misses sit behind the cache blocks in the
        # same tensor, so that attention can read hits in place and staged misses through one row table
        self.cache_blocks = self.cache_size + (self.buffer_size if self.block_cache == "device" else 0)
        self.cache_stride = max(self.cache_blocks, 1)
        # (a cache without blocks still gets one physical block: the copy kernels take a base address)
        self.cache_keys = [torch.zeros((self.batch_size, self.kv_head, max(self.cache_blocks, 1), self.page_size, D),
                                       dtype=self.dtype, device=dev(l)) for l in L]
        self.cache_values = [torch.zeros_like(self.cache_keys[l]) for l in L]
        n_in = self.input_length - self.static_pattern_total
        self.offload_keys = _pinned((self.kv_head, n_in, D), self.dtype)
        self.offload_values = _pinned((self.kv_head, n_in, D), self.dtype)
        self.list_keys = [_pinned((self.batch_size, self.kv_head, self.list_stride, D), self.dtype) for _ in L]
        self.list_values = [_pinned((self.batch_size, self.kv_head, self.list_stride, D), self.dtype) for _ in L]
        for l in L:
            self.wave_buffer[l].set_kv(self.list_keys[l], self.list_values[l], self.offload_keys, self.offload_values)

    def allocate_computation_buffer(self):
        """Layer-shared scratch (reference: retroinfer_cache.py:302-334)."""
        d0 = self.layer_mapping[str(0)]
        BG, D, gs = self.batch_groups, self.head_dim, self.group_size
        i32 = lambda *s: torch.zeros(s, dtype=torch.int32, device=d0)
        self.logits = torch.zeros((BG, gs, self.n_centroids), dtype=torch.float32, device=d0)
        # int64 id lists [BG, nprobe + es] as the reference keeps them: real tensors on the staged
        # operator path (gather_copy_vectors and the host id copy read them), views put together from the
        # int32 lists on demand elsewhere
        staged = self.kv_residency == "host" and self.block_cache == "host"
        self._cI = [torch.zeros((BG, self.max_compute_cluster_num), dtype=torch.int64, device=d0)
                    for _ in range(2)] if staged else None
        self.ret_ids = [i32(BG, self.nprobe) for _ in range(2)]
        self.est_ids = [i32(BG, max(self.es_cluster_num, 1)) for _ in range(2)]
        self.valid_lengths = [i32(BG) for _ in range(2)]
        if self.kv_residency == "device" or self.block_cache == "device":
            # token layout of the retrieval zone; a second set when the next layer's zones are chosen
            # while this layer's are still in use
            sets = 2 if self.use_cluster_estimation else 1
            # device residency: rank tables (token prefix and first store row of every rank); host
            # residency with the device-side manager: a row table (hits are scattered cache blocks)
            rows = self.buffer_size * self.page_size if self.kv_residency != "device" else 1
            self.layouts = [(i32(BG, self.nprobe + 1), i32(BG, self.nprobe), i32(BG, rows), i32(BG, 4))
                            for _ in range(sets)]
            self.ret_tok_off, self.ret_start, self.row_src, self.meta = self.layouts[0]
        if self.kv_residency != "device" and self.block_cache == "device":
            self._part_out = torch.zeros((BG, gs, D), dtype=self.dtype, device=d0)
            self._part_lse = torch.zeros((BG, gs), dtype=torch.float32, device=d0)
            # the miss staging reports the rows it assembled; the attention launch writes the real valid lengths,
            # and the staging may run on the copy stream beside it, so its report goes to a tensor of its own
            self._staged_rows = i32(BG)
        if self.kv_residency != "device":
            shape = (BG, self.execution_stride, 1, D)
            self.execution_buffer_keys = [torch.zeros(shape, dtype=self.dtype, device=d0) for _ in range(2)]
            self.execution_buffer_values = [torch.zeros(shape, dtype=self.dtype, device=d0) for _ in range(2)]
            es = max(self.es_cluster_num, 1)
            self.es_centroids = torch.zeros((BG, es, 1, D), dtype=self.dtype, device=d0)
            self.es_value_sum = torch.zeros((BG, es, 1, D), dtype=self.dtype, device=d0)
            self.es_cluster_size = torch.zeros((BG, 1, 1, es), dtype=self.dtype, device=d0)

    def pre_allocate_decision(self):
        """Kept for callers of the reference API; this build always pre-allocates."""
        return True

    def prepare_cache(self):
        """End of prefill (reference: retroinfer_cache.py:336-365)."""
        torch.cuda.synchronize()
        if self.kv_residency == "host":
            if self.block_cache == "host":
                self.wave_buffer[self.layer_num - 1].construction_sync()
            else:
                for l in range(self.layer_num):
                    self.device_lru[l].set_sizes(self.cluster_size_i32[l])
                self.stage_keys = self.stage_values = None
        self.clusters_cpu = self.cluster_size_cpu = None
        self.temp_keys = self.temp_values = None
        self._centred_keys.clear()
        # the clusterings captured during this prefill replay with the addresses of the buffers just dropped
        # (scratch tensors that were outgrown stay: a decode graph of another cache may still replay with them)
        if not torch.cuda.is_current_stream_capturing():
            kernels.release_cached_graphs(retired_workspaces=False)

    # ------------------------------------------------------------------ prefill
    def prefill_update_kv_cache(self, query_states, key_states, value_states, layer_idx, batch_idx):
        """Clusters one sequence of one layer (reference: retroinfer_cache.py:368-441).
        key/value_states [1, seq_len, kv_heads, dim].  Returns the K/V past valid_start."""
        bsz, seq_len, group_num, head_dim = key_states.shape
        assert bsz == 1, "Multi-batch prefilling only support prefill single batch one by one."
        assert seq_len <= self.input_length, f"seq_len({seq_len}) should less than input_length({self.input_length})"
        vs = self.valid_start[batch_idx]
        sps, spe, spt = self.static_pattern_start, self.static_pattern_end, self.static_pattern_total
        valid_length = seq_len - spt - vs
        H = self.kv_head
        rows = slice(batch_idx * H, (batch_idx + 1) * H)
        dkey = self.layer_mapping[str(layer_idx)]

        # host store filled by the worker threads (reference flow) or by a device permutation + one copy
        cpu_organise = self.kv_residency == "host" and self.block_cache == "host"
        dev_organise = self.kv_residency == "host" and self.block_cache == "device"
        if cpu_organise:
            # the previous construction must have consumed the shared offload buffers
            prev = layer_idx - 1 if layer_idx > 0 else (self.layer_num - 1 if batch_idx > 0 else None)
            if prev is not None:
                self.wave_buffer[prev].construction_sync()

        self.temp_keys = key_states[0, vs + sps:seq_len - spe].transpose(0, 1).contiguous()      # [H, N, D]
        self.temp_values = value_states[0, vs + sps:seq_len - spe].transpose(0, 1).contiguous()
        if cpu_organise:
            self.mainevents[dkey].record()
            with torch.cuda.stream(self.copystream):
                self.mainevents[dkey].wait()
                self.offload_keys[:, :valid_length].copy_(self.temp_keys, non_blocking=True)
                self.offload_values[:, :valid_length].copy_(self.temp_values, non_blocking=True)
                self.copyevents[dkey].record()

        for zone, src in ((self.steady_zone_keys, key_states), (self.steady_zone_values, value_states)):
            zone[layer_idx][batch_idx, :, :sps] = src[0, vs:vs + sps].transpose(0, 1)
            zone[layer_idx][batch_idx, :, sps:spt] = src[0, seq_len - spe:seq_len].transpose(0, 1)

        mean_key = torch.mean(self.temp_keys, dim=1, keepdim=True)
        # the centred keys go to a buffer that keeps its address from call to call: the clustering of
        # every further layer and sequence of this length then replays one captured graph
        ck = self._centred_keys.get((dkey, valid_length))
        if ck is None:
            if len(self._centred_keys) >= 2:
                self._centred_keys.clear()
            ck = torch.empty_like(self.temp_keys)
            self._centred_keys[(dkey, valid_length)] = ck
        torch.sub(self.temp_keys, mean_key, out=ck)
        km = segment_k_means_csr(ck, self.temp_values, self.n_centroids, num_segments=self.n_segment,
                                 reuse_graph=True)   # results are copied out below, before the next call
        self.centroids[layer_idx][rows].copy_(km.centroids + mean_key)
        self.value_sum[layer_idx][rows].copy_(km.value_sum)
        self.centroids_mask[layer_idx][rows].copy_(km.counts == 0)
        self.cluster_size[layer_idx][rows].copy_(km.counts.to(self.dtype))

        # clusters sit in the store in id order, tokens ascending inside (device: permute below; host:
        # WaveBufferCPU's organisation)
        self.cluster_start[layer_idx][rows].copy_(km.offsets[:, :self.n_centroids])
        self.cluster_size_i32[layer_idx][rows].copy_(km.counts)
        for h in range(H):
            self.store_rows[layer_idx][batch_idx * H + h] = valid_length
        if self.kv_residency == "device":
            # cluster-contiguous store built on the device (stands in for organize_kv on the host)
            lk = self.list_keys[layer_idx][batch_idx]
            lv = self.list_values[layer_idx][batch_idx]
            kernels.permute_rows(self.temp_keys, km.members, lk, H, valid_length, valid_length, self.list_stride)
            kernels.permute_rows(self.temp_values, km.members, lv, H, valid_length, valid_length, self.list_stride)
        elif dev_organise:
            # the same permutation on the device into a staging buffer, then one copy per tensor into
            # the pinned store on the copy stream (no host-side re-organisation, no dense cluster lists)
            self.copyevents[dkey].synchronize()   # the previous copy has left the staging buffers
            if getattr(self, "stage_keys", None) is None or self.stage_keys.device != self.temp_keys.device:
                n_in = self.input_length - self.static_pattern_total
                self.stage_keys = torch.empty((H, n_in, self.head_dim), dtype=self.dtype, device=self.temp_keys.device)
                self.stage_values = torch.empty_like(self.stage_keys)
            n_st = self.stage_keys.shape[1]
            kernels.permute_rows(self.temp_keys, km.members, self.stage_keys, H, valid_length, valid_length, n_st)
            kernels.permute_rows(self.temp_values, km.members, self.stage_values, H, valid_length, valid_length, n_st)
            self.mainevents[dkey].record()
            with torch.cuda.stream(self.copystream):
                self.mainevents[dkey].wait()
                self.list_keys[layer_idx][batch_idx, :, :valid_length].copy_(self.stage_keys[:, :valid_length],
                                                                             non_blocking=True)
                self.list_values[layer_idx][batch_idx, :, :valid_length].copy_(self.stage_values[:, :valid_length],
                                                                               non_blocking=True)
                self.copyevents[dkey].record()
        else:
            self.cluster_size_cpu = km.counts.cpu().contiguous()
            self.clusters_cpu = csr_to_dense(km.counts, km.offsets, km.members).cpu().contiguous()

        if layer_idx == self.layer_num - 1 and batch_idx + bsz == self.batch_size:
            self.context += seq_len
        return key_states[:, vs:], value_states[:, vs:]

    def sync(self, layer_idx, batch_idx):
        """After the prefill attention of (layer, sequence): hand the offloaded K/V to the host
        re-organisation (reference: retroinfer_cache.py:443-458).  Nothing to do on the device."""
        if self.kv_residency == "host" and self.block_cache == "host":
            self.copyevents[self.layer_mapping[str(layer_idx)]].synchronize()
            self.wave_buffer[layer_idx].async_construction(self.clusters_cpu, self.cluster_size_cpu, batch_idx)

    # ------------------------------------------------------------------ decode-time index growth
    def _update_kv_cache(self):
        """Folds the last THRESHOLD_LENGTH generated tokens into the index
        (reference: retroinfer_cache.py:462-524)."""
        sps, spe = self.static_pattern_start, self.static_pattern_end
        BG, D, ncu = self.batch_groups, self.head_dim, self.n_centroids_per_update_segment
        lo, hi = sps, self.static_pattern_total - spe
        for ldx in range(self.layer_num):
            dkey = self.layer_mapping[str(ldx)]
            torch.cuda.set_device(dkey)
            uk = self.steady_zone_keys[ldx][:, :, lo:hi].clone().reshape(BG, THRESHOLD_LENGTH, D).contiguous()
            uv = self.steady_zone_values[ldx][:, :, lo:hi].clone().reshape(BG, THRESHOLD_LENGTH, D).contiguous()
            for zone in (self.steady_zone_keys, self.steady_zone_values):   # slide the local window
                zone[ldx][:, :, sps:sps + spe] = zone[ldx][:, :, hi:hi + spe].clone()
            if self.kv_residency == "host" and self.block_cache == "host":
                self.mainevents[dkey].record()
                with torch.cuda.stream(self.copystream):
                    self.mainevents[dkey].wait()
                    self.offload_update_keys.copy_(uk, non_blocking=True)
                    self.offload_update_values.copy_(uv, non_blocking=True)
                    self.copyevents[dkey].record()
            mean_key = torch.mean(uk, dim=1, keepdim=True)
            km = segment_k_means_csr(uk - mean_key, uv, ncu, num_segments=1)
            self.centroids[ldx] = torch.cat((self.centroids[ldx], km.centroids + mean_key), dim=1)
            self.value_sum[ldx] = torch.cat((self.value_sum[ldx], km.value_sum), dim=1)
            self.centroids_mask[ldx] = torch.cat((self.centroids_mask[ldx], km.counts == 0), dim=1)
            self.cluster_size[ldx] = torch.cat((self.cluster_size[ldx], km.counts.to(self.dtype)), dim=1)
            # every group appends behind its own rows: sequences with different left padding hold
            # different numbers of clustered tokens (reference: wave_buffer_cpu.cpp:658, per group)
            bases = list(self.store_rows[ldx])
            base_t = torch.tensor(bases, dtype=torch.int32, device=km.offsets.device)[:, None]
            self.cluster_start[ldx] = torch.cat((self.cluster_start[ldx], km.offsets[:, :ncu] + base_t), dim=1)
            self.cluster_size_i32[ldx] = torch.cat((self.cluster_size_i32[ldx], km.counts), dim=1)
            self.store_rows[ldx] = [b + THRESHOLD_LENGTH for b in bases]
            runs, g0 = [], 0          # runs of consecutive groups that share a base
            for g1 in range(1, BG + 1):
                if g1 == BG or bases[g1] != bases[g0]:
                    runs.append((g0, g1, bases[g0]))
                    g0 = g1
            if self.kv_residency == "device":
                assert max(bases) + THRESHOLD_LENGTH <= self.list_stride, "cluster store is full"
                lk = self.list_keys[ldx].view(BG, self.list_stride, D)
                lv = self.list_values[ldx].view(BG, self.list_stride, D)
                for g0, g1, base in runs:
                    kernels.permute_rows(uk[g0:g1], km.members[g0:g1], lk[g0:g1, base:], g1 - g0, THRESHOLD_LENGTH,
                                         THRESHOLD_LENGTH, self.list_stride)
                    kernels.permute_rows(uv[g0:g1], km.members[g0:g1], lv[g0:g1, base:], g1 - g0, THRESHOLD_LENGTH,
                                         THRESHOLD_LENGTH, self.list_stride)
            elif self.block_cache == "device":
                assert max(bases) + THRESHOLD_LENGTH <= self.list_stride, "cluster store is full"
                pk, pv = torch.empty_like(uk), torch.empty_like(uv)
                kernels.permute_rows(uk, km.members, pk, BG, THRESHOLD_LENGTH, THRESHOLD_LENGTH, THRESHOLD_LENGTH)
                kernels.permute_rows(uv, km.members, pv, BG, THRESHOLD_LENGTH, THRESHOLD_LENGTH, THRESHOLD_LENGTH)
                lk = self.list_keys[ldx].view(BG, self.list_stride, D)
                lv = self.list_values[ldx].view(BG, self.list_stride, D)
                for g0, g1, base in runs:
                    lk[g0:g1, base:base + THRESHOLD_LENGTH].copy_(pk[g0:g1])
                    lv[g0:g1, base:base + THRESHOLD_LENGTH].copy_(pv[g0:g1])
                self.device_lru[ldx].set_sizes(self.cluster_size_i32[ldx])
            else:
                self.copyevents[dkey].synchronize()
                self.wave_buffer[ldx].update_kv(self.offload_update_keys, self.offload_update_values,
                                                csr_to_dense(km.counts, km.offsets, km.members).cpu().contiguous(),
                                                km.counts.cpu().contiguous())
        torch.cuda.set_device(self.layer_mapping[str(0)])
        self.n_centroids += ncu
        self.logits = torch.zeros((BG, self.group_size, self.n_centroids), dtype=torch.float32,
                                  device=self.layer_mapping[str(0)])
        self.static_pattern_total = sps + spe
        if self.device_positions:
            self.steady_len_dev.fill_(self.static_pattern_total + 1)
            self.steady_pos_dev.fill_(self.static_pattern_total)

    def fold_due(self):
        """True when the next token has to fold the generated tokens into the index first (every
        THRESHOLD_LENGTH tokens).  A loop that replays captured steps calls prepare_token() then,
        outside any capture, and captures its steps again: the fold re-allocates the score buffer."""
        return self.static_pattern_total == self.static_pattern_start + self.static_pattern_end + THRESHOLD_LENGTH

    def prepare_token(self):
        if self.fold_due():
            self._update_kv_cache()

    def token_replayed(self):
        """Host-side bookkeeping for one token decoded by replaying captured steps (device_positions):
        the replay advanced the device-side position, this advances the host counters."""
        self.context += 1
        self.static_pattern_total += 1

    def decode_update_kv_cache(self, key_states, value_states, layer_idx):
        """Appends the new token's K/V to the steady zone (reference: retroinfer_cache.py:527-546)."""
        last = layer_idx == self.layer_num - 1
        if self.device_positions:
            capturing = torch.cuda.is_current_stream_capturing()
            if not capturing:
                self.prepare_token()
            self.steady_zone_keys[layer_idx].index_copy_(2, self.steady_pos_dev, key_states.transpose(1, 2))
            self.steady_zone_values[layer_idx].index_copy_(2, self.steady_pos_dev, value_states.transpose(1, 2))
            # (the device-side position moves on after the last layer's attention, in compute())
            if last and not capturing:
                self.token_replayed()
            return None, None
        self.prepare_token()
        self.steady_zone_keys[layer_idx][:, :, self.static_pattern_total] = key_states[:, 0]
        self.steady_zone_values[layer_idx][:, :, self.static_pattern_total] = value_states[:, 0]
        if last:
            self.context += 1
            self.static_pattern_total += 1
        return None, None

    @property
    def cI(self):
        """[2] tensors [BG, nprobe + es] int64: retrieval ids in rank order, then estimation ids
        (reference attribute: retroinfer_cache.py:573)."""
        if self._cI is not None:
            return self._cI
        es = self.es_cluster_num
        return [torch.cat((self.ret_ids[b], self.est_ids[b][:, :es]), dim=1).to(torch.int64) for b in range(2)]

    # ------------------------------------------------------------------ decode
    def _select(self, queries, layer, buf, with_layout, layout=0):
        BG, gs, D = self.batch_groups, self.group_size, self.head_dim
        q = queries.view(BG, gs, D)
        es = self.es_cluster_num
        dev_mode = with_layout and self.kv_residency == "device"
        ret_tok_off, ret_start, _, meta = self.layouts[layout] if dev_mode else (None, None, None, None)
        # the int64 id list of the reference is only written where something reads it (the staged
        # operator path); elsewhere cI is put together from the int32 lists on demand
        cI = self._cI[buf] if self._cI is not None else None
        kernels.score_select(
            q, self.centroids[layer], self.centroids_mask[layer],
            self.cluster_size_i32[layer] if dev_mode else None, self.cluster_start[layer] if dev_mode else None,
            self.logits, None, cI, self.ret_ids[buf], self.est_ids[buf] if es > 0 else None,
            ret_tok_off, None, meta, self.nprobe, es, self.page_size, self.buffer_size, self.RSQRT_DIM,
            ret_start=ret_start)

    def compute(self, queries, layer_idx, queries_next=None):
        """Decode attention of one layer (reference: retroinfer_cache.py:549-697).
        queries [batch, 1, heads, dim] on the device; returns the same shape."""
        last = layer_idx == self.layer_num - 1
        static_len = self.static_pattern_total if last else self.static_pattern_total + 1
        if self.profiler_ranges:
            with kernels.profiler_ranges(True):
                torch.cuda.nvtx.range_push("kv_cache_compute")
                try:
                    out = self._compute(queries, layer_idx, queries_next, static_len)
                finally:
                    torch.cuda.nvtx.range_pop()
        else:
            out = self._compute(queries, layer_idx, queries_next, static_len)
        if last and self.device_positions:   # the token is done: its row now belongs to the steady zone
            self.steady_len_dev.add_(1)
            self.steady_pos_dev.add_(1)
        return out

    def _compute(self, queries, layer_idx, queries_next, static_len):
        """compute() for a given number of steady-zone tokens."""
        buf, nbuf = layer_idx % 2, (layer_idx + 1) % 2
        search_here = layer_idx < 2 or not self.use_cluster_estimation
        search_next = (self.use_cluster_estimation and 0 < layer_idx < self.layer_num - 1
                       and queries_next is not None)
        if self.kv_residency == "device" and not self.use_cluster_estimation:
            return self._compute_device(queries, layer_idx, static_len, buf)
        if self.kv_residency == "host" and self.block_cache == "device":
            return self._compute_host_in_place(queries, layer_idx, queries_next, static_len, buf, nbuf, search_here,
                                               search_next)
        return self._compute_staged(queries, layer_idx, queries_next, static_len, buf, nbuf, search_here,
                                    search_next)

    def _compute_device(self, queries, layer_idx, static_len, buf):
        BG, gs, D = self.batch_groups, self.group_size, self.head_dim
        self._select(queries, layer_idx, buf, True)
        out = torch.empty((BG, gs, D), dtype=self.dtype, device=queries.device)
        es = self.es_cluster_num
        kernels.wave_attention(
            queries.view(BG, gs, D), self.steady_zone_keys[layer_idx], self.steady_zone_values[layer_idx],
            static_len, self.list_keys[layer_idx], self.list_values[layer_idx], None, self.meta,
            self.est_ids[buf] if es > 0 else None, self.logits if es > 0 else None, self.value_sum[layer_idx],
            self.cluster_size[layer_idx], out, self.valid_lengths[buf], es, self.RSQRT_DIM,
            ret_tok_off=self.ret_tok_off, ret_start=self.ret_start,
            static_len_dev=self.steady_len_dev if self.device_positions else None)
        return out.view(self.batch_size, 1, self.num_heads, D)

    def block_cache_stats(self, layer_idx):
        """(hit blocks, miss blocks) of the layer's last look-up, summed over the groups (host residency)."""
        miss = int(self.miss_num_units[layer_idx].sum())
        if self.block_cache == "device":
            lay = (layer_idx % 2) if self.use_cluster_estimation else 0
            return int(self.layouts[lay][3][:, 2].sum()) - miss, miss
        return int(self.hit_num_units[layer_idx].sum()), miss

    # host-resident store, block cache managed on the device: hits are read in place from the cache
    # blocks, misses are staged behind them in the same tensor, both through one row table
    def _access_in_place(self, layer, buf):
        lay = buf if self.use_cluster_estimation else 0
        _, _, row_src, meta = self.layouts[lay]
        self.device_lru[layer].access_update(self.ret_ids[buf], self.cluster_size_i32[layer], self.cluster_start[layer],
                                             self._lists(layer), row_src=row_src,
                                             stage_row0=self.cache_size * self.page_size, meta=meta)

    def _stage_misses(self, layer, buf):
        BG, D = self.batch_groups, self.head_dim
        rows = self.cache_blocks * self.page_size
        stage_k = self.cache_keys[layer].view(BG, rows, D)[:, self.cache_size * self.page_size:]
        stage_v = self.cache_values[layer].view(BG, rows, D)[:, self.cache_size * self.page_size:]
        kernels.gather_copy_and_concat(
            self.steady_zone_keys[layer], self.list_keys[layer], self.cache_keys[layer], stage_k,
            self.steady_zone_values[layer], self.list_values[layer], self.cache_values[layer], stage_v,
            self.miss_unit_idices[layer], self.miss_unit_sizes[layer], self.miss_unit_sizes_cumsum[layer],
            self.miss_num_units[layer], self.hit_unit_idices[layer], self.hit_unit_sizes[layer],
            self.hit_unit_sizes_cumsum[layer], self.hit_num_units[layer], self._staged_rows, BG,
            self.static_stride, self.list_stride, self.cache_stride, rows, self.buffer_size, 0)
        return stage_k, stage_v

    def _compute_host_in_place(self, queries, layer_idx, queries_next, static_len, buf, nbuf, search_here,
                               search_next):
        BG, gs, D = self.batch_groups, self.group_size, self.head_dim
        es = self.es_cluster_num
        q = queries.view(BG, gs, D)
        rows = self.cache_blocks * self.page_size
        stage0 = self.cache_size * self.page_size
        cur = torch.cuda.current_stream()
        staged_on_copystream = not search_here   # misses staged during the previous layer
        if search_here:
            self._select(queries, layer_idx, buf, False)
            self._access_in_place(layer_idx, buf)
            if self.overlap_miss_staging:
                self.copystream.wait_stream(cur)
                with torch.cuda.stream(self.copystream):
                    self._stage_misses(layer_idx, buf)
                staged_on_copystream = True
            else:
                self._stage_misses(layer_idx, buf)
        elif es > 0:   # zones came from the predicted query: the estimation zone is scored by the true one
            kernels.score_logits(q, self.centroids[layer_idx], self.logits, self.RSQRT_DIM)
        _, _, row_src, meta = self.layouts[buf if self.use_cluster_estimation else 0]
        out = torch.empty((BG, gs, D), dtype=self.dtype, device=queries.device)
        ck = self.cache_keys[layer_idx].view(BG, rows, D)
        cv = self.cache_values[layer_idx].view(BG, rows, D)
        est_ids = self.est_ids[buf] if es > 0 else None
        logits = self.logits if es > 0 else None
        if staged_on_copystream and self.overlap_miss_staging:
            # rows in the cache blocks (source rows below the staging area), steady zone and estimation
            # zone first; then, once the staging has landed, the staged rows, merging the first part
            kernels.wave_attention_part(
                q, self.steady_zone_keys[layer_idx], self.steady_zone_values[layer_idx], static_len, ck, cv, row_src,
                0, stage0, meta, est_ids, logits, self.value_sum[layer_idx], self.cluster_size[layer_idx],
                self._part_out, self._part_lse, es, self.RSQRT_DIM, valid_lengths=self.valid_lengths[buf])
            cur.wait_stream(self.copystream)
            kernels.wave_attention_part(
                q, self.steady_zone_keys[layer_idx], self.steady_zone_values[layer_idx], 0, ck, cv, row_src,
                stage0, rows, meta, None, None, self.value_sum[layer_idx], self.cluster_size[layer_idx], out, None, 0,
                self.RSQRT_DIM, prev_out=self._part_out, prev_lse=self._part_lse)
        else:
            if staged_on_copystream:
                cur.wait_stream(self.copystream)
            kernels.wave_attention(
                q, self.steady_zone_keys[layer_idx], self.steady_zone_values[layer_idx], static_len, ck, cv, row_src,
                meta, est_ids, logits, self.value_sum[layer_idx], self.cluster_size[layer_idx], out,
                self.valid_lengths[buf], es, self.RSQRT_DIM)
        # admission: staged blocks of the admitted misses into the cache blocks handed out for them
        kernels.gather_copy_and_scatter(
            ck[:, stage0:], self.cache_keys[layer_idx], cv[:, stage0:], self.cache_values[layer_idx],
            self.update_buffer_indices[layer_idx], self.update_unit_sizes[layer_idx],
            self.update_cache_indices[layer_idx], self.update_num_units[layer_idx], BG, rows, self.cache_stride,
            self.buffer_size, 0)
        if search_next:
            self._select(queries_next, layer_idx + 1, nbuf, False)
            self._access_in_place(layer_idx + 1, nbuf)
            self.copystream.wait_stream(cur)
            with torch.cuda.stream(self.copystream):
                self._stage_misses(layer_idx + 1, nbuf)
        return out.view(self.batch_size, 1, self.num_heads, D)

    # staged path: the reference's sequence of operators, one call each
    def _search(self, queries, layer, buf):
        self._select(queries, layer, buf, False)
        if self.kv_residency == "host" and self.block_cache == "host":
            self.cluster_ids[buf].copy_(self._cI[buf][:, :self.nprobe])  # blocking copy into pinned memory

    def _lists(self, layer):
        return [self.hit_unit_idices[layer], self.hit_unit_sizes[layer], self.hit_unit_sizes_cumsum[layer],
                self.hit_num_units[layer], self.miss_unit_idices[layer], self.miss_unit_sizes[layer],
                self.miss_unit_sizes_cumsum[layer], self.miss_num_units[layer], self.update_buffer_indices[layer],
                self.update_unit_sizes[layer], self.update_cache_indices[layer], self.update_num_units[layer]]

    def _access(self, layer, buf):
        """Hit / miss / admission lists of the clusters chosen for `layer` (in buffer `buf`)."""
        if self.block_cache == "device":
            self.device_lru[layer].access_update(self.ret_ids[buf], self.cluster_size_i32[layer],
                                                 self.cluster_start[layer], self._lists(layer))
        else:
            self.wave_buffer[layer].batch_access()

    def _assemble(self, layer, buf, static_len):
        if self.kv_residency == "host":
            kernels.gather_copy_and_concat(
                self.steady_zone_keys[layer], self.list_keys[layer], self.cache_keys[layer],
                self.execution_buffer_keys[buf], self.steady_zone_values[layer], self.list_values[layer],
                self.cache_values[layer], self.execution_buffer_values[buf],
                self.miss_unit_idices[layer], self.miss_unit_sizes[layer], self.miss_unit_sizes_cumsum[layer],
                self.miss_num_units[layer], self.hit_unit_idices[layer], self.hit_unit_sizes[layer],
                self.hit_unit_sizes_cumsum[layer], self.hit_num_units[layer], self.valid_lengths[buf],
                self.batch_groups, self.static_stride, self.list_stride, self.cache_stride, self.execution_stride,
                self.buffer_size, static_len)

    def _compute_staged(self, queries, layer_idx, queries_next, static_len, buf, nbuf, search_here, search_next):
        BG, gs, D = self.batch_groups, self.group_size, self.head_dim
        q4 = queries.view(BG, 1, gs, D)
        if self.kv_residency == "device":
            return self._compute_device_estimated(queries, layer_idx, queries_next, static_len, buf, nbuf,
                                                  search_here, search_next)
        if search_here:
            self._search(queries, layer_idx, buf)
        if search_next:
            self._search(queries_next, layer_idx + 1, nbuf)
        # without next-layer estimation the logits of this layer's own query are at hand, so the
        # estimation zone is merged inside the final attention launch; otherwise it is computed the
        # reference's way, from gathered centroids and the true query
        fuse_est = self.es_cluster_num > 0 and not self.use_cluster_estimation
        if self.es_cluster_num > 0 and not fuse_est:
            kernels.gather_copy_vectors(
                self.centroids[layer_idx], self.es_centroids, self.value_sum[layer_idx], self.es_value_sum,
                self.cluster_size[layer_idx], self.es_cluster_size, self._cI[buf], BG, self.n_centroids,
                self.es_cluster_num, self.max_compute_cluster_num, self.nprobe, self.es_cluster_num)
            es_out, es_lse = kernels.weighted_flash_decoding(q4, self.es_centroids, self.es_value_sum,
                                                             self.es_cluster_size, return_softmax_lse=True)
        else:
            es_out = es_lse = None
        if search_here:
            self._access(layer_idx, buf)
        if search_next:
            self._access(layer_idx + 1, nbuf)
        if search_here:
            self._assemble(layer_idx, buf, static_len)
        if search_next:
            cur = torch.cuda.current_stream()
            self.copystream.wait_stream(cur)
            with torch.cuda.stream(self.copystream):
                self._assemble(layer_idx + 1, nbuf, static_len)
        if not search_here:
            # this layer's buffer was assembled on the copy stream during the previous layer, before this
            # layer's new token was appended to its steady zone (as in the reference, retroinfer_cache.py:644-652
            # against :541-542, whose attention then sees a stale row there): the token's row is brought in now,
            # so that every residency attends the same rows
            torch.cuda.current_stream().wait_stream(self.copystream)
            if not self.reference_stale_row:
                BGd = (BG, -1, D)
                self.execution_buffer_keys[buf][:, static_len - 1, 0] = \
                    self.steady_zone_keys[layer_idx].view(BGd)[:, static_len - 1]
                self.execution_buffer_values[buf][:, static_len - 1, 0] = \
                    self.steady_zone_values[layer_idx].view(BGd)[:, static_len - 1]
        if fuse_est:
            attn = torch.empty((BG, gs, D), dtype=self.dtype, device=queries.device)
            kernels.buffer_attention(
                queries.view(BG, gs, D), self.execution_buffer_keys[buf], self.execution_buffer_values[buf],
                self.valid_lengths[buf], self.est_ids[buf], self.logits, self.value_sum[layer_idx],
                self.cluster_size[layer_idx], attn, self.es_cluster_num, self.RSQRT_DIM)
        else:
            attn = kernels.weighted_flash_decoding(
                q4, self.execution_buffer_keys[buf], self.execution_buffer_values[buf], previous_out=es_out,
                previous_lse=es_lse, cache_seqlens=self.valid_lengths[buf])
        if self.block_cache == "host":
            self.wave_buffer[layer_idx].sync()
        kernels.gather_copy_and_scatter(
            self.execution_buffer_keys[buf], self.cache_keys[layer_idx], self.execution_buffer_values[buf],
            self.cache_values[layer_idx], self.update_buffer_indices[layer_idx], self.update_unit_sizes[layer_idx],
            self.update_cache_indices[layer_idx], self.update_num_units[layer_idx], BG, self.execution_stride,
            self.cache_stride, self.buffer_size, static_len)
        return attn.view(self.batch_size, 1, self.num_heads, D)

    def _compute_device_estimated(self, queries, layer_idx, queries_next, static_len, buf, nbuf, search_here,
                                  search_next):
        """Device residency with next-layer cluster estimation (reference: retroinfer_cache.py:565,
        582-595): from the third layer on the zones come from the query the previous layer
        predicted; the estimation zone is scored with the true query (inside the attention launch,
        from the centroid rows), the retrieval zone is attended exactly.  A device-resident store has
        no transfer to hide, so this mode exists for behavioural parity, not speed: the next layer's
        zones are chosen after this layer's attention, on the same stream.  (Choosing them on a second
        stream during the attention was measured slower, 66-72 us against 59 us per layer-step at the
        benchmark shape: two branches inside a replayed graph cost more than the overlap gains.)"""
        BG, gs, D = self.batch_groups, self.group_size, self.head_dim
        es = self.es_cluster_num
        q = queries.view(BG, gs, D)
        if search_here:
            self._select(queries, layer_idx, buf, True, layout=buf)
        ret_tok_off, ret_start, _, meta = self.layouts[buf]
        out = torch.empty((BG, gs, D), dtype=self.dtype, device=queries.device)
        # zones from the layer's own query: its logits are at hand; zones from a predicted query: the
        # estimation zone is scored with the true query inside the attention launch
        own = search_here and es > 0
        kernels.wave_attention(
            q, self.steady_zone_keys[layer_idx], self.steady_zone_values[layer_idx], static_len,
            self.list_keys[layer_idx], self.list_values[layer_idx], None, meta,
            self.est_ids[buf] if es > 0 else None, self.logits if own else None, self.value_sum[layer_idx],
            self.cluster_size[layer_idx], out, self.valid_lengths[buf], es, self.RSQRT_DIM,
            ret_tok_off=ret_tok_off, ret_start=ret_start,
            est_centroids=self.centroids[layer_idx] if es > 0 and not own else None)
        if search_next:
            self._select(queries_next, layer_idx + 1, nbuf, True, layout=nbuf)
        return out.view(self.batch_size, 1, self.num_heads, D)

