// Cluster selection for the decode step (gfx950): from the fp32 logits of the scoring pass to
// the retrieval zone (top nprobe clusters in rank order), the estimation zone (next es) and
// the layout of the retrieved tokens (rank tables, optionally a row table).  Follows cache_hub/retroinfer_cache.py:572-575
// (sum over the query group of the bf16 softmax, empty-cluster mask, top-k) and the buffer
// cut-off of library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp:207-216.
//
// Two launches:
//   dist_kernel    many workgroups per group: score = bf16(sum_j bf16(exp(bf16(x_j)-m_j)/Z_j)),
//                  mapped to a 16-bit key whose unsigned order is the score order.
//   select_kernel  one workgroup per group: exact rank thresholds from a histogram with one bin
//                  per distinct key (scores lie in [0, 16], so ~16.8k bins cover every key), zone
//                  membership with ties resolved by ascending id, rank order of the retrieval
//                  zone straight from the histogram prefix, and the token layout (page
//                  cut-off; token prefix and first store row per rank, a row per token on request).
#include <type_traits>

#include "ri_common.h"

#define SEL_THREADS 1024
#define SEL_MAX_PROBES 4096  // ranks of the retrieval zone one workgroup can lay out (four per thread)
#define SEL_WAVES (SEL_THREADS / 64)
#define DIST_IDS 1024  // ids per dist workgroup (4 per thread)

// Histogram add that survives a degenerate distribution: when the whole wave hits one bin
// (for instance every score equal) a single lane adds the lane count.
__device__ __forceinline__ void hist_add(uint32_t* hist, uint32_t bin, bool active) {
  const uint64_t act = __ballot(active);
  if (act == 0) return;
  const int lead = __ffsll((long long)act) - 1;
  const uint32_t first = (uint32_t)__builtin_amdgcn_readlane((int)bin, lead);
  const uint64_t same = __ballot(active && bin == first);
  if (same == act) {
    if ((int)(threadIdx.x & 63) == lead) atomicAdd(&hist[first], (uint32_t)__popcll(act));
  } else if (active) {
    atomicAdd(&hist[bin], 1u);
  }
}

// ------------------------------------------------------------------------------------
// dist_kernel: grid (ceil(nc / 1024), BG), 256 threads, 4 consecutive ids per thread.
// ------------------------------------------------------------------------------------
// HALF: scores are rounded to IEEE half instead of bfloat16 wherever the reference's tensors are (the D and
// Softmax outputs of batch_gemm_softmax and the score sum carry the cache's element type).
template <int GSM, bool HALF>
__global__ __launch_bounds__(256) void dist_kernel(const float* __restrict__ logits,
                                                   const float* __restrict__ tile_max,
                                                   const float* __restrict__ tile_sum,
                                                   const uint8_t* __restrict__ mask, uint16_t* __restrict__ keys,
                                                   uint16_t* __restrict__ dist_out, int gs, int nc, int ntiles) {
  __shared__ float sh_m[16], sh_iz[16];
  const int g = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = blockIdx.x * DIST_IDS + tid * 4;
  const bool in = c < nc;  // nc % 4 == 0

  // loads first, so that the row statistics below hide behind their latency
  float4 x4[GSM];
#pragma unroll
  for (int j = 0; j < GSM; ++j)
    if (j < gs && in) x4[j] = *reinterpret_cast<const float4*>(logits + ((size_t)g * gs + j) * nc + c);
  const uint32_t mk = (mask && in) ? *reinterpret_cast<const uint32_t*>(mask + (size_t)g * nc + c) : 0u;

  for (int j = wave; j < gs; j += 4) {
    float m, iz;
    ri_wave_reduce_partials(tile_max + (size_t)g * ntiles * gs, tile_sum + (size_t)g * ntiles * gs, ntiles, gs, j,
                            lane, &m, &iz);
    if (lane == 0) { sh_m[j] = m; sh_iz[j] = iz; }
  }
  __syncthreads();

  float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < GSM; ++j) {
    if (j < gs && in) {
      const float x[4] = {x4[j].x, x4[j].y, x4[j].z, x4[j].w};
      const float m = sh_m[j], iz = sh_iz[j];
#pragma unroll
      for (int i = 0; i < 4; ++i) d[i] += ri_round_e16<HALF>(__expf(ri_round_e16<HALF>(x[i]) - m) * iz);
    }
  }
  uint16_t bits[4], key[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bits[i] = ri_f32_to_e16<HALF>(d[i]);
    if ((mk >> (8 * i)) & 0xffu) bits[i] = ri_e16_lowest<HALF>();  // finfo(type).min
    key[i] = (uint16_t)ri_bf16_sort_key(bits[i]);
  }
  if (in) {
    uint2 w;
    w.x = (uint32_t)key[0] | ((uint32_t)key[1] << 16);
    w.y = (uint32_t)key[2] | ((uint32_t)key[3] << 16);
    *reinterpret_cast<uint2*>(keys + (size_t)g * nc + c) = w;
    if (dist_out) {
      w.x = (uint32_t)bits[0] | ((uint32_t)bits[1] << 16);
      w.y = (uint32_t)bits[2] | ((uint32_t)bits[3] << 16);
      *reinterpret_cast<uint2*>(dist_out + (size_t)g * nc + c) = w;
    }
  }
}

// ------------------------------------------------------------------------------------
// select_kernel helpers
// ------------------------------------------------------------------------------------
// Exclusive prefix sums of N values over the threads of the block with one barrier.
// sh: N * SEL_WAVES words that no other scan of the same parity is still reading: callers
// alternate between two buffers.  tot[] receives the block totals.
template <int N>
__device__ __forceinline__ void block_excl_scan(const uint32_t (&v)[N], uint32_t (&pre)[N], uint32_t (&tot)[N],
                                                uint32_t* sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t inc[N];
#pragma unroll
  for (int k = 0; k < N; ++k) {
    inc[k] = ri_wave_incl_scan(v[k]);
    if (lane == 63) sh[k * SEL_WAVES + wave] = inc[k];
  }
  __syncthreads();
  // the sixteen wave totals are scanned by the lanes (one LDS read, one DPP scan, two lane reads) instead of
  // being walked by every thread: a third of the kernel's vector instructions were that walk, and the kernel
  // is bound by instruction issue on its one compute unit as much as by latency
  const int wv = __builtin_amdgcn_readfirstlane(wave);
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const uint32_t x = (lane < SEL_WAVES) ? sh[k * SEL_WAVES + lane] : 0u;
    const uint32_t sc = ri_wave_incl_scan(x);
    tot[k] = (uint32_t)__builtin_amdgcn_readlane((int)sc, SEL_WAVES - 1);
    const uint32_t woff = wv > 0 ? (uint32_t)__builtin_amdgcn_readlane((int)sc, wv - 1) : 0u;
    pre[k] = woff + inc[k] - v[k];
  }
}

// Scores are sums of at most 16 probabilities, so their keys span a small range: key 0x8000
// (score +0) .. 0xC180 (score 16), plus the masked value far below.  One histogram bin per
// distinct key makes the rank search exact in a single pass.
// (IEEE half: 0x8000 .. 0xCC00, so 17 bins per thread cover bfloat16 scores and 20 cover half scores.)
#define SEL_KEY_LO 0x8000u
#define SEL_BPT_BF16 17                     // bins per thread: 17 * 1024 = 17408 >= 0x4181 + 1
#define SEL_BPT_F16 20                      //                  20 * 1024 = 20480 >= 0x4C01 + 1
template <int BPT>
__device__ __forceinline__ uint32_t sel_bin(uint32_t key) {
  constexpr uint32_t BINS = SEL_THREADS * BPT;
  const uint32_t b = key >= SEL_KEY_LO ? key - SEL_KEY_LO + 1u : 0u;
  return b < BINS ? b : BINS - 1;
}

// ------------------------------------------------------------------------------------
// select_kernel: one 1024-thread workgroup per group.
// The sizes of the retrieved clusters are read from global memory by the threads that own a rank (staging
// all nc sizes in LDS up front put 4 nc bytes per group on the load phase of the one compute unit that runs
// the group: 0.9 us slower per step at 8192 clusters, 2.2 us at 16384).
// Thread t owns the contiguous id range [t*E, t*E+E) and keeps those keys in registers: ties
// are ranked by ascending id with plain prefix sums.
// ------------------------------------------------------------------------------------
// E8: eights of keys a thread owns (1 up to 8192 clusters, 2 up to 16384, 4 up to 32768, 8 up to 65536): the
// loops over the owned keys are unrolled E8 times, so the common sizes do not carry (and fetch) the code of
// sixty-four keys per thread.
// R: ranks of the retrieval zone a thread owns in the token-layout phase (1 up to 1023 probes, 4 up to 4096).
// BPT: histogram bins per thread (SEL_BPT_BF16 or SEL_BPT_F16).
template <int E8, int R, int BPT>
__global__ __launch_bounds__(SEL_THREADS) void select_kernel(
    const uint16_t* __restrict__ keys, const int32_t* __restrict__ cluster_size,
    const int32_t* __restrict__ cluster_start, int64_t* __restrict__ cI, int32_t* __restrict__ ret_ids,
    int32_t* __restrict__ est_ids, int32_t* __restrict__ ret_tok_off, int32_t* __restrict__ ret_start,
    int32_t* __restrict__ row_src, int row_src_stride, int32_t* __restrict__ meta, int nc, int np, int es, int page, int max_pages) {
  constexpr int SEL_BPT = BPT;
  constexpr int SEL_BINS = SEL_THREADS * BPT;
  __shared__ uint32_t hist[SEL_BINS];
  __shared__ uint32_t sh_scan[2][3 * SEL_WAVES];  // two buffers, used alternately
  __shared__ uint32_t sh_sel[4];  // bin of T1, entries above it, bin of T2, entries above it
  constexpr int NPMAX = SEL_THREADS * R;
  __shared__ uint32_t sh_ret[NPMAX];
  // rank-ordered entries, then size and first store row of the cluster at each rank: arrays of their own for
  // the common case, laid over the histogram (which is dead by then) when a thread owns several ranks
  __shared__ uint32_t sh_lay[R == 1 ? 3 * NPMAX : 1];
  static_assert(R == 1 || 3 * NPMAX <= SEL_BINS, "the rank arrays must fit the histogram they are laid over");
  uint32_t* const sh_sorted = R == 1 ? sh_lay : hist;
  uint32_t* const sh_size = sh_sorted + NPMAX;
  int32_t* const sh_start = reinterpret_cast<int32_t*>(sh_sorted + 2 * NPMAX);
  __shared__ uint32_t sh_pages, sh_tret, sh_nkeep;

  const int g = blockIdx.x;
  const int tid = threadIdx.x;
  const int k2 = np + es;

  // ---- loads: this thread's keys (registers) ----
  // thread t owns the contiguous id range [t*E, t*E+E), E a multiple of 8 (nc % 8 == 0), E <= 64
  const int E = 8 * E8;  // >= ceil(nc / SEL_THREADS), a multiple of 8
  const int cbeg = min(tid * E, nc);
  const int cend = min(cbeg + E, nc);
  uint4 kreg[E8];
#pragma unroll
  for (int i = 0; i < E8; ++i)
    kreg[i] = (cbeg + 8 * i < cend) ? *reinterpret_cast<const uint4*>(keys + (size_t)g * nc + cbeg + 8 * i)
                                     : ri_zero16();
#pragma unroll
  for (int i = 0; i < SEL_BPT; ++i) hist[tid * SEL_BPT + i] = 0u;
  if (tid == 0) { sh_pages = 0; sh_tret = 0; sh_nkeep = 0; }
  __syncthreads();
  // calls f(id, key) for every owned key in ascending id order
  auto for_each_key = [&](auto&& f) {
#pragma unroll
    for (int i = 0; i < E8; ++i) {
      if (cbeg + 8 * i < cend) {
        const uint32_t w[4] = {kreg[i].x, kreg[i].y, kreg[i].z, kreg[i].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          f(cbeg + 8 * i + 2 * q, w[q] & 0xffffu);
          f(cbeg + 8 * i + 2 * q + 1, w[q] >> 16);
        }
      }
    }
  };
  for_each_key([&](int, uint32_t key) { hist_add(hist, sel_bin<BPT>(key), true); });
  __syncthreads();

  // ---- rank thresholds: T1 = key of descending rank np-1, T2 = key of rank k2-1 ----
  // thread t owns bins [t*17, t*17+17); afterwards hist[b] holds the number of keys above bin b
  {
    uint32_t hb[SEL_BPT], mine = 0;
#pragma unroll
    for (int i = 0; i < SEL_BPT; ++i) { hb[i] = hist[tid * SEL_BPT + i]; mine += hb[i]; }
    uint32_t vin[1] = {mine}, below[1], tot[1];
    block_excl_scan<1>(vin, below, tot, sh_scan[0]);
    uint32_t above = tot[0] - below[0] - mine;  // entries in bins above this thread's
    const uint32_t rankA = (uint32_t)(np - 1), rankB = (uint32_t)(k2 - 1);
    // only threads that hold keys of the retrieval zone (their bins' ranks are needed below) or one of
    // the two threshold ranks walk their bins
    if (mine > 0 && (above < (uint32_t)np || (above <= rankB && rankB < above + mine))) {
#pragma unroll
      for (int i = SEL_BPT - 1; i >= 0; --i) {
        if (above <= rankA && rankA < above + hb[i]) { sh_sel[0] = tid * SEL_BPT + i; sh_sel[1] = above; }
        if (above <= rankB && rankB < above + hb[i]) { sh_sel[2] = tid * SEL_BPT + i; sh_sel[3] = above; }
        hist[tid * SEL_BPT + i] = above;
        above += hb[i];
      }
    }
  }
  __syncthreads();
  const uint32_t B1 = sh_sel[0], B2 = sh_sel[2];  // threshold bins (bins order like keys)
  const uint32_t g1 = sh_sel[1], g2 = sh_sel[3];  // keys strictly above T1 / T2

  // ---- one scan ranks everything: ties at T1, ties at T2 and the keys strictly between ----
  // Tied keys are taken in ascending id order: tie rank r at T1 belongs to the retrieval zone
  // while g1 + r < np, then to the estimation zone while g1 + r < k2; at T2 while g2 + r < k2.
  // The owned keys are classified once, without branches, into four bit masks (bit i = owned key i); the
  // rare cases (keys of the retrieval zone: np of nc; ties at a threshold) are then walked bit by bit.
  typedef typename std::conditional<(E8 <= 4), uint32_t, uint64_t>::type mask_t;
  mask_t m_gt1 = 0, m_eq1 = 0, m_gt2 = 0, m_eq2 = 0;
  for_each_key([&](int c, uint32_t key) {
    const uint32_t bin = sel_bin<BPT>(key);
    const int i = c - cbeg;
    m_gt1 |= (mask_t)(bin > B1) << i;
    m_eq1 |= (mask_t)(bin == B1) << i;
    m_gt2 |= (mask_t)(bin > B2) << i;
    m_eq2 |= (mask_t)(bin == B2) << i;
  });
  if (B2 == B1) m_eq2 = 0;
  const mask_t m_mid = m_gt2 & ~m_gt1 & ~m_eq1;  // strictly between the thresholds: estimation zone
  auto popc = [](mask_t m) { return (uint32_t)(sizeof(mask_t) == 8 ? __popcll((unsigned long long)m) : __popc((unsigned)m)); };
  auto lowest = [](mask_t m) { return sizeof(mask_t) == 8 ? __ffsll((long long)m) - 1 : __ffs((int)m) - 1; };
  uint32_t cnt3[3] = {popc(m_eq1), popc(m_eq2), popc(m_mid)}, pre3[3], tot3[3];
  block_excl_scan<3>(cnt3, pre3, tot3, sh_scan[1]);
  const uint32_t r1 = pre3[0], r2 = pre3[1];
  const uint32_t mid_before = pre3[2];
  const uint32_t lo1 = (uint32_t)np > g1 ? (uint32_t)np - g1 : 0u;   // first tie rank of T1 in the est zone
  const uint32_t hi1r = (uint32_t)k2 > g1 ? (uint32_t)k2 - g1 : 0u;  // one past the last
  const uint32_t hi2r = (uint32_t)k2 > g2 ? (uint32_t)k2 - g2 : 0u;
  // Global stores are kept for the end of the kernel: a barrier waits for every outstanding
  // memory operation of the wave, stores included, so a store issued here would put its round
  // trip on the critical path of each later phase.
  const uint32_t est_first = mid_before + (min(max(r1, lo1), hi1r) - lo1) + min(r2, hi2r);
  // owned key i (a register half chosen at run time: only the rare walks below need it)
  auto key_at = [&](int i) {
    uint32_t w = 0;
#pragma unroll
    for (int v = 0; v < E8; ++v) {
      const uint32_t q[4] = {kreg[v].x, kreg[v].y, kreg[v].z, kreg[v].w};
#pragma unroll
      for (int u = 0; u < 4; ++u) w = ((i >> 1) == 4 * v + u) ? q[u] : w;
    }
    return (i & 1) ? (w >> 16) : (w & 0xffffu);
  };
  mask_t est_bits = m_mid;  // bit i: owned key i is in the estimation zone
  for (mask_t m = m_gt1; m; m &= m - 1) {  // above T1: the ranks of a bin start at hist[bin] = keys above it
    const int i = lowest(m);
    const uint32_t key = key_at(i);
    const uint32_t slot = atomicAdd(&hist[sel_bin<BPT>(key)], 1u);
    sh_ret[slot] = (key << 16) | (0xffffu - (uint32_t)(cbeg + i));
  }
  {
    uint32_t rk = r1;  // ties at T1 enter in id order
    for (mask_t m = m_eq1; m; m &= m - 1, ++rk) {
      const int i = lowest(m);
      if (rk < lo1) sh_ret[g1 + rk] = (key_at(i) << 16) | (0xffffu - (uint32_t)(cbeg + i));
      else if (rk < hi1r) est_bits |= (mask_t)1 << i;
    }
    rk = r2;
    for (mask_t m = m_eq2; m && rk < hi2r; m &= m - 1, ++rk) est_bits |= (mask_t)1 << lowest(m);
  }
  __syncthreads();

  // ---- rank order: sh_ret is ordered by score; order runs of equal scores by ascending id ----
  // The size and first store row of the entry's cluster are requested before the walk over its run and
  // travel to the entry's final rank through LDS: their round trip to global memory runs under the walk
  // instead of after the next barrier.
  for (int r = tid; r < np; r += SEL_THREADS) {
    const uint32_t mine = sh_ret[r];
    const uint32_t kk = mine >> 16;
    uint32_t sz_e = 0;
    int32_t st_e = 0;
    if (cluster_size) {
      const size_t at = (size_t)g * nc + (0xffffu - (mine & 0xffffu));
      sz_e = (uint32_t)cluster_size[at];
      if (cluster_start) st_e = cluster_start[at];
    }
    int lo = r, rank_in_run = 0;
    while (lo > 0 && (sh_ret[lo - 1] >> 16) == kk) { --lo; rank_in_run += (sh_ret[lo] > mine); }
    int hi = r;
    while (hi + 1 < np && (sh_ret[hi + 1] >> 16) == kk) { ++hi; rank_in_run += (sh_ret[hi] > mine); }
    sh_sorted[lo + rank_in_run] = mine;
    sh_size[lo + rank_in_run] = sz_e;
    sh_start[lo + rank_in_run] = st_e;
  }
  __syncthreads();

  // ---- token layout of the retrieved clusters with the page cut-off ----
  // thread t owns the ranks [t*R, t*R + R)
  const int rb = tid * R;
  uint32_t sz[R], pg[R];
  int32_t st[R];
  int my_c[R];
  uint32_t pg_sum = 0, sz_sum = 0;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    sz[i] = 0; pg[i] = 0; st[i] = 0; my_c[i] = -1;
    if (rb + i < np) {
      my_c[i] = (int)(0xffffu - (sh_sorted[rb + i] & 0xffffu));
      st[i] = sh_start[rb + i];
      sz[i] = sh_size[rb + i];
      pg[i] = (sz[i] + page - 1) / page;
    }
    pg_sum += pg[i];
    sz_sum += sz[i];
  }
  uint32_t tok_run[R];
  uint32_t keep_bits = 0;
  int nkeep = 0;
  int32_t T_ret = 0;
  if (cluster_size) {
    uint32_t lay[2] = {pg_sum, sz_sum}, layp[2], layt[2];
    block_excl_scan<2>(lay, layp, layt, sh_scan[0]);
    uint32_t pg_run = layp[0], tk = layp[1];
    // kept clusters form a prefix because the page prefix is monotone; tokens before a kept
    // cluster all belong to kept clusters
#pragma unroll
    for (int i = 0; i < R; ++i) {
      tok_run[i] = tk;
      const int r = rb + i;
      const bool keep = r < np && pg_run + pg[i] <= (uint32_t)max_pages;
      // the kept clusters are the ranks 0 .. nkeep-1: the last of them publishes the totals
      if (keep) {
        keep_bits |= 1u << i;
        const uint32_t next_pg = (i + 1 < R) ? pg[i + 1] : (r + 1 < np ? (sh_size[r + 1] + page - 1) / page : 0u);
        const bool next_keep = r + 1 < np && pg_run + pg[i] + next_pg <= (uint32_t)max_pages;
        if (!next_keep) {
          sh_pages = pg_run + pg[i];
          sh_tret = tk + sz[i];
          sh_nkeep = (uint32_t)r + 1u;
        }
      }
      pg_run += pg[i];
      tk += sz[i];
    }
    __syncthreads();
    nkeep = (int)sh_nkeep;
    T_ret = (int32_t)sh_tret;
  }

  // ---- all global stores ----
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (rb + i < np) {
      ret_ids[(size_t)g * np + rb + i] = my_c[i];
      if (cI) cI[(size_t)g * k2 + rb + i] = my_c[i];
    }
  }
  {
    uint32_t est_off = est_first;
    for (int i = 0; i < E; ++i) {
      if ((est_bits >> i) & 1u) {
        est_ids[(size_t)g * es + est_off] = cbeg + i;
        if (cI) cI[(size_t)g * k2 + np + est_off] = cbeg + i;
        ++est_off;
      }
    }
  }
  if (!cluster_size) return;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int r = rb + i;
    if (r < np) {
      ret_tok_off[(size_t)g * (np + 1) + r] = (r < nkeep) ? (int32_t)tok_run[i] : T_ret;
      if (ret_start) ret_start[(size_t)g * np + r] = st[i];
    }
  }
  if (tid == 0) {
    ret_tok_off[(size_t)g * (np + 1) + np] = T_ret;
    meta[g * 4 + 0] = nkeep;
    meta[g * 4 + 1] = T_ret;
    meta[g * 4 + 2] = (int32_t)sh_pages;
    meta[g * 4 + 3] = 0;
  }
  // row table: each kept cluster writes the rows of its tokens
  if (!row_src || !cluster_start) return;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (!((keep_bits >> i) & 1u)) continue;
    int32_t* dst = row_src + (size_t)g * row_src_stride + tok_run[i];
    const int room = row_src_stride - (int)tok_run[i];
    for (int k = 0; k < (int)sz[i] && k < room; ++k) dst[k] = st[i] + k;
  }
}

// ------------------------------------------------------------------------------------
// C entry points
// ------------------------------------------------------------------------------------
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

extern "C" size_t ri_score_select_workspace_bytes(int BG, int gs, int nc) {
  if (BG <= 0 || gs <= 0 || nc <= 0) return 0;
  const size_t ntiles = (size_t)(nc + RI_SCORE_TILE - 1) / RI_SCORE_TILE;
  return 2 * align256((size_t)BG * ntiles * gs * sizeof(float)) + align256((size_t)BG * nc * sizeof(uint16_t));
}

static int score_select_impl(const void* q, const void* centroids, const uint8_t* mask,
                             const int32_t* cluster_size_i32, const int32_t* cluster_start, float* logits, void* dist,
                             int64_t* cI, int32_t* ret_ids, int32_t* est_ids, int32_t* ret_tok_off, int32_t* ret_start,
                             int32_t* row_src, int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np, int es,
                             int page, int max_pages, float scale, void* workspace, size_t workspace_bytes, bool half,
                             ri_stream_t stream) {
  if (!q || !centroids || !logits || !ret_ids || !workspace) return RI_ERR_ARG;
  if (ri_any_misaligned16(q, centroids, logits, workspace)) return RI_ERR_ARG;
  if (BG <= 0 || gs <= 0 || gs > 16 || nc <= 0 || (nc % 8) != 0) return RI_ERR_ARG;
  if (np <= 0 || np > SEL_MAX_PROBES || es < 0 || np + es > nc || nc > 65536) return RI_ERR_ARG;
  if (es > 0 && !est_ids) return RI_ERR_ARG;
  if (cluster_size_i32 && (!ret_tok_off || !meta || page <= 0 || max_pages <= 0)) return RI_ERR_ARG;
  if (workspace_bytes < ri_score_select_workspace_bytes(BG, gs, nc)) return RI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const int ntiles = (nc + RI_SCORE_TILE - 1) / RI_SCORE_TILE;
  char* w = (char*)workspace;
  float* tmax = (float*)w;
  w += align256((size_t)BG * ntiles * gs * sizeof(float));
  float* tsum = (float*)w;
  w += align256((size_t)BG * ntiles * gs * sizeof(float));
  uint16_t* keys = (uint16_t*)w;
  int rc = ri_launch_score(q, centroids, logits, tmax, tsum, BG, gs, nc, scale, half, s);
  if (rc) return rc;
  const dim3 dgrid((nc + DIST_IDS - 1) / DIST_IDS, BG);
#define RI_DIST_LAUNCH(GSM)                                                                                       \
  do {                                                                                                            \
    if (half)                                                                                                     \
      dist_kernel<GSM, true><<<dgrid, 256, 0, s>>>(logits, tmax, tsum, mask, keys, (uint16_t*)dist, gs, nc, ntiles); \
    else                                                                                                          \
      dist_kernel<GSM, false><<<dgrid, 256, 0, s>>>(logits, tmax, tsum, mask, keys, (uint16_t*)dist, gs, nc, ntiles); \
  } while (0)
  if (gs <= 4) RI_DIST_LAUNCH(4);
  else if (gs <= 8) RI_DIST_LAUNCH(8);
  else RI_DIST_LAUNCH(16);
#undef RI_DIST_LAUNCH
  RI_HIP_CHECK_LAUNCH();
  const int per_thread = (nc + SEL_THREADS - 1) / SEL_THREADS;
#define RI_SELECT_LAUNCH_T(E8, R, BPT)                                                                               \
  select_kernel<E8, R, BPT><<<BG, SEL_THREADS, 0, s>>>(keys, cluster_size_i32, cluster_start, cI, ret_ids, est_ids,  \
                                                       ret_tok_off, ret_start, row_src, row_src_stride, meta, nc, np, \
                                                       es, page, max_pages)
#define RI_SELECT_LAUNCH(E8, R)                             \
  do {                                                      \
    if (half) RI_SELECT_LAUNCH_T(E8, R, SEL_BPT_F16);       \
    else RI_SELECT_LAUNCH_T(E8, R, SEL_BPT_BF16);           \
  } while (0)
  if (np < SEL_THREADS) {
    if (per_thread <= 8) RI_SELECT_LAUNCH(1, 1);
    else if (per_thread <= 16) RI_SELECT_LAUNCH(2, 1);
    else if (per_thread <= 32) RI_SELECT_LAUNCH(4, 1);
    else RI_SELECT_LAUNCH(8, 1);
  } else {  // long probe lists only occur with many clusters
    if (per_thread <= 16) RI_SELECT_LAUNCH(2, 4);
    else if (per_thread <= 32) RI_SELECT_LAUNCH(4, 4);
    else RI_SELECT_LAUNCH(8, 4);
  }
#undef RI_SELECT_LAUNCH
#undef RI_SELECT_LAUNCH_T
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" int ri_score_select(const void* q, const void* centroids, const uint8_t* mask,
                               const int32_t* cluster_size_i32, const int32_t* cluster_start,
                               float* logits, void* dist, int64_t* cI, int32_t* ret_ids,
                               int32_t* est_ids, int32_t* ret_tok_off, int32_t* ret_start,
                               int32_t* row_src, int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np,
                               int es, int page, int max_pages, float scale, void* workspace,
                               size_t workspace_bytes, ri_stream_t stream) {
  return score_select_impl(q, centroids, mask, cluster_size_i32, cluster_start, logits, dist, cI, ret_ids, est_ids,
                           ret_tok_off, ret_start, row_src, row_src_stride, meta, BG, gs, nc, np, es, page, max_pages,
                           scale, workspace, workspace_bytes, false, stream);
}

extern "C" int ri_score_select_f16(const void* q, const void* centroids, const uint8_t* mask,
                                   const int32_t* cluster_size_i32, const int32_t* cluster_start,
                                   float* logits, void* dist, int64_t* cI, int32_t* ret_ids,
                                   int32_t* est_ids, int32_t* ret_tok_off, int32_t* ret_start,
                                   int32_t* row_src, int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np,
                                   int es, int page, int max_pages, float scale, void* workspace,
                                   size_t workspace_bytes, ri_stream_t stream) {
  return score_select_impl(q, centroids, mask, cluster_size_i32, cluster_start, logits, dist, cI, ret_ids, est_ids,
                           ret_tok_off, ret_start, row_src, row_src_stride, meta, BG, gs, nc, np, es, page, max_pages,
                           scale, workspace, workspace_bytes, true, stream);
}

static int score_logits_impl(const void* q, const void* centroids, float* logits, int BG, int gs, int nc, float scale,
                             void* workspace, size_t workspace_bytes, bool half, ri_stream_t stream) {
  if (!q || !centroids || !logits || !workspace) return RI_ERR_ARG;
  if (ri_any_misaligned16(q, centroids, logits, workspace)) return RI_ERR_ARG;
  if (BG <= 0 || gs <= 0 || gs > 16 || nc <= 0 || (nc % 4) != 0) return RI_ERR_ARG;
  if (workspace_bytes < ri_score_select_workspace_bytes(BG, gs, nc)) return RI_ERR_WORKSPACE;
  const int ntiles = (nc + RI_SCORE_TILE - 1) / RI_SCORE_TILE;
  float* tmax = (float*)workspace;
  float* tsum = (float*)((char*)workspace + align256((size_t)BG * ntiles * gs * sizeof(float)));
  return ri_launch_score(q, centroids, logits, tmax, tsum, BG, gs, nc, scale, half, (hipStream_t)stream);
}

extern "C" int ri_score_logits(const void* q, const void* centroids, float* logits, int BG, int gs, int nc,
                               float scale, void* workspace, size_t workspace_bytes, ri_stream_t stream) {
  return score_logits_impl(q, centroids, logits, BG, gs, nc, scale, workspace, workspace_bytes, false, stream);
}

extern "C" int ri_score_logits_f16(const void* q, const void* centroids, float* logits, int BG, int gs, int nc,
                                   float scale, void* workspace, size_t workspace_bytes, ri_stream_t stream) {
  return score_logits_impl(q, centroids, logits, BG, gs, nc, scale, workspace, workspace_bytes, true, stream);
}
