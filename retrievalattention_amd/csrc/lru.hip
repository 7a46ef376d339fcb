// Device-side block cache manager for a host-resident cluster store (gfx950).
//
// Does on the GPU, in one launch and without a host round trip, what the reference does on CPU
// worker threads between the top-k search and the gather:
//   BufferManager::batch_access  (library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp:190-257)
//     walk the retrieved clusters in rank order, stop when their blocks no longer fit the
//     execution buffer, emit the hit list (cache block ids) and the miss list (host rows);
//   BufferManager::batch_update  (wave_buffer_cpu.cpp:102-188)
//     touch the hits, admit the longest prefix of the misses that fits the cache, evict
//     least-recently-used clusters until enough blocks are free, hand out block ids, emit the
//     admission list for the scatter kernel.
// The lists have the layout the copy kernels of gather.hip read.
//
// Recency is kept per resident cluster as a pair: the number of the last step that touched it and its order
// inside that step.  That reproduces the reference's list (wave_buffer_cpu.cpp:106-114: the hits are moved to
// the front in reverse rank order; :170-176: then the admitted misses are pushed in rank order): inside a
// step the admitted misses are the most recent, later-ranked ones first, then the hits, earlier-ranked ones
// first.  Eviction takes whole clusters from the least recent end until the request is covered, hits of the
// current step included (:140-142; their blocks have been listed for this step's attention, which runs
// before the admission copy overwrites them).  The victims are found without sorting: a radix selection over
// the step ages (four 8-bit digits) gives the boundary step, and inside that step the clusters are ranked by
// their order through an LDS table indexed by it.
#include "ri_common.h"

#define LRU_THREADS 1024
#define LRU_WAVES (LRU_THREADS / 64)
#define LRU_DIGIT 256

struct LruParams {
  const int32_t* ret_ids;   // [BG, np] cluster ids in rank order
  const int32_t* sizes;     // [BG, meta_stride] tokens per cluster
  const int32_t* starts;    // [BG, meta_stride] first row of the cluster in the host store
  const int32_t* blk_off;   // [BG, blk_off_stride] exclusive prefix of ceil(size / block)
  int32_t* stamp;           // [BG, stamp_stride] 0 = not resident, else last step that touched it
  int32_t* order;           // [BG, stamp_stride] order inside that step (larger = more recent)
  int32_t* blk_ids;         // [BG, blk_ids_stride] cache block ids of resident clusters, at blk_off
  int32_t* free_list;       // [BG, capacity] free block ids, the first free_count are valid
  int32_t* free_count;      // [BG]
  int32_t* epoch;           // [BG] step counter
  int32_t *hit_ids, *hit_sizes, *hit_cumsum, *hit_num;
  int32_t *miss_ids, *miss_sizes, *miss_cumsum, *miss_num;
  int32_t *upd_buf, *upd_sizes, *upd_cache, *upd_num;
  // optional row table for attention in place: row of every retrieved token in a tensor that holds the
  // cache blocks first and the staging area of the misses behind them; then no hit list is emitted
  int32_t* row_src;  // [BG, row_src_stride] or null
  int32_t* meta;     // [BG, 4]: {clusters kept, tokens, blocks, 0} or null
  int row_src_stride, stage_row0;
  int np, ncl, meta_stride, blk_off_stride, stamp_stride, blk_ids_stride, buffer_size, capacity, block;
};

// exclusive prefix sums of N values over the 1024 threads; totals in tot.  Wave scans on DPP, the sixteen
// wave totals scanned by the lanes of every wave (one LDS read, one DPP scan, two lane reads).
template <int N>
__device__ __forceinline__ void lru_scan(const int (&v)[N], int (&pre)[N], int (&tot)[N], int* sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    inc[k] = (int)ri_wave_incl_scan((uint32_t)v[k]);
    if (lane == 63) sh[k * LRU_WAVES + wave] = inc[k];
  }
  __syncthreads();
  const int wv = __builtin_amdgcn_readfirstlane(wave);
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const uint32_t x = (lane < LRU_WAVES) ? (uint32_t)sh[k * LRU_WAVES + lane] : 0u;
    const uint32_t sc = ri_wave_incl_scan(x);
    tot[k] = __builtin_amdgcn_readlane((int)sc, LRU_WAVES - 1);
    const int woff = wv > 0 ? __builtin_amdgcn_readlane((int)sc, wv - 1) : 0;
    pre[k] = woff + inc[k] - v[k];
  }
  __syncthreads();
}

// R: ranks of the probe list a thread owns (thread t: ranks [t*R, t*R + R)); 1 up to 1023 probes, 4 up to 4096.
template <int R>
__global__ __launch_bounds__(LRU_THREADS) void lru_kernel(LruParams P) {
  constexpr int NPMAX = LRU_THREADS * R;
  __shared__ int sh_scan[7 * LRU_WAVES];
  __shared__ int sh_hist[LRU_DIGIT];
  __shared__ int sh_cut[2];  // selected digit, blocks freed by clusters with a larger one
  // token offsets and sources of the ranks for the row table; later the blocks of the boundary step's
  // clusters by their order inside the step (2 * NPMAX entries: hits below, admitted misses above)
  __shared__ int sh_tab[2 * NPMAX];
  int* const sh_off = sh_tab;
  int* const sh_src = sh_tab + NPMAX;
  const int g = blockIdx.x;
  const int tid = threadIdx.x;
  const int block = P.block;
  const int32_t* sizes = P.sizes + (size_t)g * P.meta_stride;
  const int32_t* starts = P.starts + (size_t)g * P.meta_stride;
  const int32_t* boff = P.blk_off + (size_t)g * P.blk_off_stride;
  int32_t* stamp = P.stamp + (size_t)g * P.stamp_stride;
  int32_t* order = P.order + (size_t)g * P.stamp_stride;
  int32_t* bids = P.blk_ids + (size_t)g * P.blk_ids_stride;
  int32_t* flist = P.free_list + (size_t)g * P.capacity;
  const size_t lo = (size_t)g * P.buffer_size;
  const int E = P.epoch[g] + 1;
  const int F0 = P.free_count[g];
  const int rb = tid * R;

  // ---- access: every rank looks at its cluster ----
  // (everything the rank needs to know about its cluster is requested in one go: loads issued after a
  // barrier would each put another round trip to global memory on the kernel's critical path)
  int c[R], nb[R], sz[R], stamp_c[R], boff_c[R], start_c[R];
  int nb_sum = 0;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    c[i] = -1; nb[i] = 0; sz[i] = 0; stamp_c[i] = 0; boff_c[i] = 0; start_c[i] = 0;
    if (rb + i < P.np) {
      c[i] = P.ret_ids[(size_t)g * P.np + rb + i];
      if (c[i] < 0 || c[i] >= P.ncl) {
        c[i] = -1;
      } else {
        sz[i] = sizes[c[i]];
        stamp_c[i] = stamp[c[i]];
        boff_c[i] = boff[c[i]];
        start_c[i] = starts[c[i]];
        nb[i] = (sz[i] + block - 1) / block;
      }
    }
    nb_sum += nb[i];
  }
  // The walk stops at the first cluster whose blocks no longer fit: everything after it is dropped.  Whether
  // anything is dropped is only known from the block prefix, so the counts are first taken as if nothing were
  // (one scan for the block prefix and the counts together) and only recounted when the list was cut.
  bool keep[R], hit[R], miss[R];
  int v5[6], p5[6], t5[6];
  auto count = [&](int run) {
#pragma unroll
    for (int k = 0; k < 6; ++k) v5[k] = 0;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      keep[i] = c[i] >= 0 && nb[i] > 0 && run + nb[i] <= P.buffer_size;
      hit[i] = keep[i] && stamp_c[i] != 0;
      miss[i] = keep[i] && !hit[i];
      run += nb[i];
      v5[0] += hit[i] ? nb[i] : 0;
      v5[1] += keep[i] ? sz[i] : 0;
      v5[2] += miss[i] ? nb[i] : 0;
      v5[3] += miss[i] ? sz[i] : 0;
      v5[4] += keep[i] ? 1 : 0;
      v5[5] += hit[i] ? 1 : 0;
    }
  };
  {
    count(INT32_MIN / 2);   // no cut-off: every valid cluster with blocks is kept
    int v7[7], p7[7], t7[7];
#pragma unroll
    for (int k = 0; k < 6; ++k) v7[k] = v5[k];
    v7[6] = nb_sum;
    lru_scan<7>(v7, p7, t7, sh_scan);
    if (t7[6] <= P.buffer_size) {   // uniform: the whole list fits
#pragma unroll
      for (int k = 0; k < 6; ++k) { p5[k] = p7[k]; t5[k] = t7[k]; }
    } else {
      count(p7[6]);
      lru_scan<6>(v5, p5, t5, sh_scan);
    }
  }
  // per rank: hit blocks, kept tokens, miss blocks, miss tokens, hits of the lower ranks
  int hb_pre[R], tok_pre[R], mb_pre[R], mt_pre[R], hit_idx[R];
  {
    int a = p5[0], b = p5[1], cc = p5[2], d = p5[3], h = p5[5];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      hb_pre[i] = a; tok_pre[i] = b; mb_pre[i] = cc; mt_pre[i] = d; hit_idx[i] = h;
      a += hit[i] ? nb[i] : 0;
      b += keep[i] ? sz[i] : 0;
      cc += miss[i] ? nb[i] : 0;
      d += miss[i] ? sz[i] : 0;
      h += hit[i] ? 1 : 0;
    }
  }
  const int nhits = t5[5];
  // tok_pre: tokens of kept clusters of lower rank (position in the row table); the hit list's own
  // token offsets are only needed without a row table
  int hit_tok[R];
#pragma unroll
  for (int i = 0; i < R; ++i) hit_tok[i] = 0;
  if (!P.row_src) {
    int vh[1] = {0}, ph[1], th[1];
#pragma unroll
    for (int i = 0; i < R; ++i) vh[0] += hit[i] ? sz[i] : 0;
    lru_scan<1>(vh, ph, th, sh_scan);
    int a = ph[0];
#pragma unroll
    for (int i = 0; i < R; ++i) { hit_tok[i] = a; a += hit[i] ? sz[i] : 0; }
  }
  // the longest prefix of the misses whose blocks fit the whole cache may be admitted (none when the cache
  // has no blocks: every retrieved cluster then stays a miss, wave_buffer_cpu.cpp:119-130 with capacity 0)
  // (a step whose clusters all hit — the steady state of a warm cache — admits nothing and skips the scans)
  const bool any_miss = t5[2] > 0;  // uniform
  bool adm[R];
  int adm_pre[R];
  int need = 0;
#pragma unroll
  for (int i = 0; i < R; ++i) { adm[i] = false; adm_pre[i] = 0; }
  if (any_miss) {
    int va[1] = {0}, pa[1], ta[1];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      adm[i] = miss[i] && mb_pre[i] + nb[i] <= P.capacity;
      va[0] += adm[i] ? nb[i] : 0;
    }
    lru_scan<1>(va, pa, ta, sh_scan);
    need = ta[0];
    int a = pa[0];
#pragma unroll
    for (int i = 0; i < R; ++i) { adm_pre[i] = a; a += adm[i] ? nb[i] : 0; }
  }

  const bool rows = P.row_src != nullptr;
  if (rows) {
    // row table: every thread takes tokens t, t + 1024, ... and finds the rank that owns them by
    // bisection over the token offsets of the ranks (clusters that were dropped have no tokens)
#pragma unroll
    for (int i = 0; i < R; ++i) {
      sh_off[rb + i] = tok_pre[i];
      sh_src[rb + i] = hit[i] ? -(boff_c[i] + 1) : P.stage_row0 + mt_pre[i];  // hits: where their block ids are
    }
    __syncthreads();
    int32_t* table = P.row_src + (size_t)g * P.row_src_stride;
    for (int t = tid; t < t5[1]; t += LRU_THREADS) {
      int lo_r = 0, hi_r = min(NPMAX, P.np);  // first rank whose offset exceeds t (ranks past the list hold the total)
      while (lo_r < hi_r) {
        const int mid = (lo_r + hi_r) >> 1;
        if (sh_off[mid] > t) hi_r = mid; else lo_r = mid + 1;
      }
      const int r = lo_r - 1, i = t - sh_off[r], src = sh_src[r];
      table[t] = src < 0 ? bids[-src - 1 + i / block] * block + i % block : src + i;
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (hit[i]) {
      const int32_t* ids = bids + boff_c[i];
      if (!rows) {
        for (int j = 0; j < nb[i]; ++j) {
          P.hit_ids[lo + hb_pre[i] + j] = ids[j];
          P.hit_sizes[lo + hb_pre[i] + j] = (j == nb[i] - 1) ? sz[i] - (nb[i] - 1) * block : block;
          P.hit_cumsum[lo + hb_pre[i] + j] = hit_tok[i] + j * block;
        }
      }
      stamp[c[i]] = E;
      order[c[i]] = nhits - 1 - hit_idx[i];   // hits are moved to the front in reverse rank order
    }
    if (miss[i]) {
      const int row = start_c[i];
      for (int j = 0; j < nb[i]; ++j) {
        P.miss_ids[lo + mb_pre[i] + j] = row + j * block;
        P.miss_sizes[lo + mb_pre[i] + j] = (j == nb[i] - 1) ? sz[i] - (nb[i] - 1) * block : block;
        P.miss_cumsum[lo + mb_pre[i] + j] = mt_pre[i] + j * block;
      }
    }
  }
  if (tid == 0) {
    P.hit_num[g] = rows ? 0 : t5[0];
    P.miss_num[g] = t5[2];
    if (P.meta) {
      P.meta[g * 4 + 0] = t5[4];
      P.meta[g * 4 + 1] = t5[1];
      P.meta[g * 4 + 2] = t5[0] + t5[2];
      P.meta[g * 4 + 3] = 0;
    }
  }
  __syncthreads();  // the hits carry this step's stamp and order before anybody looks for victims

  // ---- eviction: free (need - F0) blocks from the least recently used clusters ----
  const int to_free = need - F0;  // uniform
  int F = F0;
  if (to_free > 0) {
    // thread t owns the ids [t*K, t*K + K)
    const int K = (P.ncl + LRU_THREADS - 1) / LRU_THREADS;
    const int c0 = tid * K, c1 = min(P.ncl, c0 + K);
    // boundary step: the age A such that every resident cluster older than A goes and the clusters of age A
    // cover the remaining `rem` blocks; radix selection over the four bytes of the age, oldest first
    uint32_t sel_mask = 0, sel_val = 0;
    int rem = to_free;
    for (int b = 3; b >= 0; --b) {
      if (tid < LRU_DIGIT) sh_hist[tid] = 0;
      if (tid == 0) { sh_cut[0] = 0; sh_cut[1] = 0; }
      __syncthreads();
      for (int cc = c0; cc < c1; ++cc) {
        const int st = stamp[cc];
        if (st == 0) continue;
        const uint32_t age = (uint32_t)(E - st);
        if ((age & sel_mask) == sel_val) atomicAdd(&sh_hist[(age >> (8 * b)) & 255u], boff[cc + 1] - boff[cc]);
      }
      __syncthreads();
      if (tid < 64) {
        // lane l holds the digits 255 - 4l .. 252 - 4l (oldest first); the lane whose running total crosses
        // rem holds the boundary digit
        int h[4], sum = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) { h[i] = sh_hist[255 - (4 * tid + i)]; sum += h[i]; }
        const int incl = (int)ri_wave_incl_scan((uint32_t)sum);
        int acc = incl - sum;
        if (acc < rem && rem <= incl) {
          int sel = 0;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (acc < rem && rem <= acc + h[i]) { sel = 255 - (4 * tid + i); sh_cut[1] = acc; }
            acc += h[i];
          }
          sh_cut[0] = sel;
        }
      }
      __syncthreads();
      sel_val |= (uint32_t)sh_cut[0] << (8 * b);
      sel_mask |= 255u << (8 * b);
      rem -= sh_cut[1];
    }
    const uint32_t cut = sel_val;   // boundary age; rem blocks are still wanted from the clusters of that age
    // the clusters of the boundary step, least recent first = ascending order inside the step
    for (int i = tid; i < 2 * NPMAX; i += LRU_THREADS) sh_tab[i] = 0;
    __syncthreads();
    for (int cc = c0; cc < c1; ++cc) {
      const int st = stamp[cc];
      if (st != 0 && (uint32_t)(E - st) == cut) sh_tab[min(max(order[cc], 0), 2 * NPMAX - 1)] = boff[cc + 1] - boff[cc];
    }
    __syncthreads();
    {
      // exclusive prefix of the table in place: thread t owns the entries [t * 2R, t * 2R + 2R)
      int own[2 * R], vt[1] = {0}, pt[1], tt[1];
#pragma unroll
      for (int i = 0; i < 2 * R; ++i) { own[i] = sh_tab[tid * 2 * R + i]; vt[0] += own[i]; }
      lru_scan<1>(vt, pt, tt, sh_scan);
      int run = pt[0];
#pragma unroll
      for (int i = 0; i < 2 * R; ++i) { sh_tab[tid * 2 * R + i] = run; run += own[i]; }
    }
    __syncthreads();
    int ev = 0;
    uint64_t ev_bits = 0;  // K <= 64 ids per thread
    for (int cc = c0; cc < c1; ++cc) {
      const int st = stamp[cc];
      if (st == 0) continue;
      const uint32_t age = (uint32_t)(E - st);
      const bool out = age > cut || (age == cut && sh_tab[min(max(order[cc], 0), 2 * NPMAX - 1)] < rem);
      if (out) {
        ev_bits |= 1ull << (cc - c0);
        ev += boff[cc + 1] - boff[cc];
      }
    }
    int ve[1] = {ev}, pe[1], te[1];
    lru_scan<1>(ve, pe, te, sh_scan);
    int w = F0 + pe[0];
    for (int cc = c0; cc < c1; ++cc) {
      if (!((ev_bits >> (cc - c0)) & 1ull)) continue;
      const int nbc = boff[cc + 1] - boff[cc];
      for (int j = 0; j < nbc; ++j) flist[w++] = bids[boff[cc] + j];
      stamp[cc] = 0;
    }
    F = F0 + te[0];
    __syncthreads();  // the freed ids are in the list before they are handed out
  }

  // ---- admission: block ids come off the end of the free list in rank order ----
  int vb[2] = {0, 0}, pb[2] = {0, 0}, tb[2] = {0, 0};
#pragma unroll
  for (int i = 0; i < R; ++i) {
    adm[i] = adm[i] && adm_pre[i] + nb[i] <= F;  // (always true: everything resident can be evicted)
    vb[0] += adm[i] ? nb[i] : 0;
    vb[1] += adm[i] ? 1 : 0;
  }
  if (any_miss) lru_scan<2>(vb, pb, tb, sh_scan);
  int adm_idx = pb[1];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (adm[i]) {
      order[c[i]] = nhits + adm_idx++;   // pushed to the front in rank order, after the hits
      int32_t* ids = bids + boff_c[i];
      for (int j = 0; j < nb[i]; ++j) {
        const int id = flist[F - 1 - (adm_pre[i] + j)];
        ids[j] = id;
        P.upd_cache[lo + adm_pre[i] + j] = id;
        P.upd_sizes[lo + adm_pre[i] + j] = (j == nb[i] - 1) ? sz[i] - (nb[i] - 1) * block : block;
        P.upd_buf[lo + adm_pre[i] + j] = mt_pre[i] + j * block;  // admitted misses lead the miss list
      }
      stamp[c[i]] = E;
    }
  }
  if (tid == 0) {
    P.upd_num[g] = tb[0];
    P.free_count[g] = F - tb[0];
    P.epoch[g] = E;
  }
}

extern "C" int ri_lru_access_update(const int32_t* ret_ids, const int32_t* sizes, const int32_t* starts,
                                    int meta_stride, const int32_t* blk_off, int blk_off_stride, int32_t* stamp,
                                    int32_t* order, int stamp_stride, int32_t* blk_ids, int blk_ids_stride, int32_t* free_list,
                                    int32_t* free_count, int32_t* epoch, int32_t* hit_ids, int32_t* hit_sizes,
                                    int32_t* hit_cumsum, int32_t* hit_num, int32_t* miss_ids, int32_t* miss_sizes,
                                    int32_t* miss_cumsum, int32_t* miss_num, int32_t* upd_buf, int32_t* upd_sizes,
                                    int32_t* upd_cache, int32_t* upd_num, int32_t* row_src, int row_src_stride,
                                    int stage_row0, int32_t* meta, int BG, int np, int ncl, int buffer_size,
                                    int capacity, int block, ri_stream_t stream) {
  // (a cache without blocks has an empty free list: its pointer may be null)
  if (!ret_ids || !sizes || !starts || !blk_off || !stamp || !order || !blk_ids || (!free_list && capacity > 0) || !free_count ||
      !epoch ||
      !hit_ids || !hit_sizes || !hit_cumsum || !hit_num || !miss_ids || !miss_sizes || !miss_cumsum || !miss_num ||
      !upd_buf || !upd_sizes || !upd_cache || !upd_num)
    return RI_ERR_ARG;
  if (BG <= 0 || np <= 0 || np > 4 * LRU_THREADS || ncl <= 0 || ncl > 64 * LRU_THREADS || buffer_size <= 0 ||
      capacity < 0 || block <= 0)
    return RI_ERR_ARG;
  if (meta_stride < ncl || blk_off_stride < ncl + 1 || stamp_stride < ncl || blk_ids_stride <= 0) return RI_ERR_ARG;
  if (row_src && (!meta || row_src_stride < buffer_size * block || stage_row0 < capacity * block)) return RI_ERR_ARG;
  LruParams P = {ret_ids, sizes, starts, blk_off, stamp, order, blk_ids, free_list, free_count, epoch,
                 hit_ids, hit_sizes, hit_cumsum, hit_num, miss_ids, miss_sizes, miss_cumsum, miss_num,
                 upd_buf, upd_sizes, upd_cache, upd_num, row_src, meta, row_src_stride, stage_row0,
                 np, ncl, meta_stride, blk_off_stride, stamp_stride, blk_ids_stride, buffer_size, capacity, block};
  if (np < LRU_THREADS)
    lru_kernel<1><<<BG, LRU_THREADS, 0, (hipStream_t)stream>>>(P);
  else
    lru_kernel<4><<<BG, LRU_THREADS, 0, (hipStream_t)stream>>>(P);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
