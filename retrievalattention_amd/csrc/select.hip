// Cluster selection for the decode step (gfx950): from the fp32 logits of the scoring pass to
// the retrieval zone (top nprobe clusters in rank order), the estimation zone (next es) and
// the row table of the retrieved tokens.  Follows cache_hub/retroinfer_cache.py:572-575
// (sum over the query group of the bf16 softmax, empty-cluster mask, top-k) and the buffer
// cut-off of library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp:207-216.
//
// Two launches:
//   dist_kernel    many workgroups per group: score = bf16(sum_j bf16(exp(bf16(x_j)-m_j)/Z_j)),
//                  mapped to a 16-bit key whose unsigned order is the score order; keys go to
//                  global memory and into a per-group histogram of their top 11 bits.
//   select_kernel  one workgroup per group: exact rank thresholds by radix select on the key
//                  (11-bit histogram, then the low 5 bits inside the two boundary bins), zone
//                  membership with ties resolved by ascending id, rank order of the retrieval
//                  zone, and the token layout (page cut-off, row table).
#include "ri_common.h"

#define SEL_THREADS 1024
#define SEL_WAVES (SEL_THREADS / 64)
#define SEL_LO_BITS (16 - RI_SEL_HI_BITS)
#define SEL_LO_BINS (1 << SEL_LO_BITS)
#define DIST_IDS 1024  // ids per dist workgroup (4 per thread)

// Histogram add that survives a degenerate distribution: when the whole wave hits one bin
// (for instance every score equal) a single lane adds the lane count.
__device__ __forceinline__ void hist_add(uint32_t* hist, uint32_t bin, bool active) {
  const uint64_t act = __ballot(active);
  if (act == 0) return;
  const int lead = __ffsll((long long)act) - 1;
  const uint32_t first = __shfl(bin, lead);
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
template <int GSM>
__global__ __launch_bounds__(256) void dist_kernel(const float* __restrict__ logits,
                                                   const float* __restrict__ tile_max,
                                                   const float* __restrict__ tile_sum,
                                                   const uint8_t* __restrict__ mask, uint16_t* __restrict__ keys,
                                                   uint16_t* __restrict__ dist_out, uint32_t* __restrict__ ghist,
                                                   int gs, int nc, int ntiles) {
  __shared__ float sh_m[16], sh_iz[16];
  __shared__ uint32_t hist[RI_SEL_HI_BINS];
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
  for (int i = tid; i < RI_SEL_HI_BINS; i += 256) hist[i] = 0u;
  __syncthreads();

  float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < GSM; ++j) {
    if (j < gs && in) {
      const float x[4] = {x4[j].x, x4[j].y, x4[j].z, x4[j].w};
      const float m = sh_m[j], iz = sh_iz[j];
#pragma unroll
      for (int i = 0; i < 4; ++i) d[i] += ri_round_bf16(__expf(ri_round_bf16(x[i]) - m) * iz);
    }
  }
  uint16_t bits[4], key[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bits[i] = ri_f32_to_bf16(d[i]);
    if ((mk >> (8 * i)) & 0xffu) bits[i] = 0xff7f;  // finfo(bfloat16).min
    key[i] = (uint16_t)ri_bf16_sort_key(bits[i]);
    hist_add(hist, (uint32_t)key[i] >> SEL_LO_BITS, in);
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
  __syncthreads();
  for (int i = tid; i < RI_SEL_HI_BINS; i += 256) {
    const uint32_t v = hist[i];
    if (v) atomicAdd(&ghist[(size_t)g * RI_SEL_HI_BINS + i], v);
  }
}

// ------------------------------------------------------------------------------------
// select_kernel helpers
// ------------------------------------------------------------------------------------
// exclusive prefix sum over the threads of the block; *total receives the sum
template <typename T>
__device__ __forceinline__ T block_excl_scan(T v, T* sh, T* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const T n = __shfl_up(inc, d);
    if (lane >= d) inc += n;
  }
  __syncthreads();  // sh may still be read from a previous scan
  if (lane == 63) sh[wave] = inc;
  __syncthreads();
  T woff = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < SEL_WAVES; ++w) {
    const T s = sh[w];
    if (w < wave) woff += s;
    tot += s;
  }
  *total = tot;
  return woff + inc - v;
}

// Over a 32-bin histogram: bin holding descending rank `rank` and the count above it (one thread).
__device__ __forceinline__ void find_lo_bin(const uint32_t* hist, uint32_t rank, uint32_t* out) {
  uint32_t above = 0;
  for (int b = SEL_LO_BINS - 1; b >= 0; --b) {
    const uint32_t v = hist[b];
    if (rank < above + v) { out[0] = (uint32_t)b; out[1] = above; return; }
    above += v;
  }
}

// ------------------------------------------------------------------------------------
// select_kernel: one workgroup per group.  dynamic LDS: nc * 2 bytes of keys.
// Thread t owns the contiguous id range [t*E, t*E+E): ties are ranked by ascending id with
// plain prefix sums.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(SEL_THREADS) void select_kernel(
    const uint16_t* __restrict__ keys, const uint32_t* __restrict__ ghist,
    const int32_t* __restrict__ cluster_size, const int32_t* __restrict__ cluster_start,
    int64_t* __restrict__ cI, int32_t* __restrict__ ret_ids, int32_t* __restrict__ est_ids,
    int32_t* __restrict__ ret_tok_off, int32_t* __restrict__ row_src, int row_src_stride,
    int32_t* __restrict__ meta, int nc, int np, int es, int page, int max_pages) {
  extern __shared__ uint16_t sh_key[];
  __shared__ uint32_t hist_b[SEL_LO_BINS], hist_c[SEL_LO_BINS];
  __shared__ uint64_t sh_scan[SEL_WAVES];
  __shared__ uint32_t sh_sel[8];  // hi1, above, hi2, above, lo1, above, lo2, above
  __shared__ uint32_t sh_ret[1024];
  __shared__ uint32_t sh_sorted[1024];
  __shared__ int32_t sh_off[1025];
  __shared__ uint32_t sh_cnt, sh_pages, sh_tret;
  __shared__ int sh_nk;

  const int g = blockIdx.x;
  const int tid = threadIdx.x;
  const int k2 = np + es;
  constexpr int HB = RI_SEL_HI_BINS / SEL_THREADS;  // histogram bins per thread

  // ---- loads: the group's histogram and keys ----
  uint32_t hb[HB];
#pragma unroll
  for (int i = 0; i < HB; ++i) hb[i] = ghist[(size_t)g * RI_SEL_HI_BINS + tid * HB + i];
  const int E = (((nc + SEL_THREADS - 1) / SEL_THREADS) + 7) & ~7;  // multiple of 8 (nc % 8 == 0)
  const int cbeg = min(tid * E, nc);
  const int cend = min(cbeg + E, nc);
  for (int c = cbeg; c < cend; c += 8)
    *reinterpret_cast<uint4*>(&sh_key[c]) = *reinterpret_cast<const uint4*>(keys + (size_t)g * nc + c);
  if (tid < SEL_LO_BINS) hist_b[tid] = hist_c[tid] = 0;
  if (tid == 0) { sh_cnt = 0; sh_pages = 0; sh_tret = 0; sh_nk = 0; }

  // ---- bins of the two rank thresholds: T1 = key of rank np-1, T2 = key of rank k2-1 ----
  {
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < HB; ++i) mine += hb[i];
    uint64_t tot;
    const uint32_t below = (uint32_t)block_excl_scan<uint64_t>(mine, sh_scan, &tot);
    uint32_t above = (uint32_t)tot - below - mine;  // entries in bins above this thread's
    const uint32_t rankA = (uint32_t)(np - 1), rankB = (uint32_t)(k2 - 1);
#pragma unroll
    for (int i = HB - 1; i >= 0; --i) {
      if (above <= rankA && rankA < above + hb[i]) { sh_sel[0] = tid * HB + i; sh_sel[1] = above; }
      if (above <= rankB && rankB < above + hb[i]) { sh_sel[2] = tid * HB + i; sh_sel[3] = above; }
      above += hb[i];
    }
  }
  __syncthreads();
  const uint32_t hi1 = sh_sel[0], hi2 = sh_sel[2];
  for (int c = cbeg; c < cbeg + E; ++c) {  // same trip count in every lane
    const bool in = c < cend;
    const uint32_t key = in ? sh_key[c] : 0u;
    hist_add(hist_b, key & (SEL_LO_BINS - 1), in && (key >> SEL_LO_BITS) == hi1);
    hist_add(hist_c, key & (SEL_LO_BINS - 1), in && (key >> SEL_LO_BITS) == hi2);
  }
  __syncthreads();
  if (tid == 0) find_lo_bin(hist_b, (uint32_t)(np - 1) - sh_sel[1], sh_sel + 4);
  if (tid == 64) find_lo_bin(hist_c, (uint32_t)(k2 - 1) - sh_sel[3], sh_sel + 6);
  __syncthreads();
  const uint32_t T1 = (hi1 << SEL_LO_BITS) | sh_sel[4];
  const uint32_t T2 = (hi2 << SEL_LO_BITS) | sh_sel[6];
  const uint32_t g1 = sh_sel[1] + sh_sel[5];  // keys strictly above T1
  const uint32_t g2 = sh_sel[3] + sh_sel[7];  // keys strictly above T2

  // ---- one scan ranks everything: ties at T1, ties at T2 and the keys strictly between ----
  // Tied keys are taken in ascending id order: tie rank r at T1 belongs to the retrieval zone
  // while g1 + r < np, then to the estimation zone while g1 + r < k2; at T2 while g2 + r < k2.
  uint32_t n1 = 0, n2 = 0, nmid = 0;
  for (int c = cbeg; c < cend; ++c) {
    const uint32_t key = sh_key[c];
    n1 += (key == T1);
    n2 += (key == T2 && T2 != T1);
    nmid += (key < T1 && key > T2);
  }
  uint64_t tot64;
  const uint64_t pre = block_excl_scan<uint64_t>((uint64_t)n1 | ((uint64_t)n2 << 20) | ((uint64_t)nmid << 40),
                                                 sh_scan, &tot64);
  uint32_t r1 = (uint32_t)(pre & 0xfffff), r2 = (uint32_t)((pre >> 20) & 0xfffff);
  const uint32_t mid_before = (uint32_t)(pre >> 40);
  // estimation members among the first r ties
  const uint32_t lo1 = (uint32_t)np > g1 ? (uint32_t)np - g1 : 0u;          // first tie rank of T1 in the est zone
  const uint32_t hi1r = (uint32_t)k2 > g1 ? (uint32_t)k2 - g1 : 0u;         // one past the last
  const uint32_t hi2r = (uint32_t)k2 > g2 ? (uint32_t)k2 - g2 : 0u;
  auto est_of_t1 = [&](uint32_t r) { return min(max(r, lo1), hi1r) - lo1; };
  auto est_of_t2 = [&](uint32_t r) { return min(r, hi2r); };
  uint32_t est_off = mid_before + est_of_t1(r1) + est_of_t2(r2);
  for (int c = cbeg; c < cend; ++c) {
    const uint32_t key = sh_key[c];
    bool in_ret, in_est;
    if (key == T1) {
      in_ret = r1 < lo1;
      in_est = !in_ret && r1 < hi1r;
      ++r1;
    } else if (key == T2) {
      in_ret = false;
      in_est = r2 < hi2r;
      ++r2;
    } else {
      in_ret = key > T1;
      in_est = !in_ret && key > T2;
    }
    if (in_ret) {
      const uint32_t slot = atomicAdd(&sh_cnt, 1u);
      sh_ret[slot] = (key << 16) | (0xffffu - (uint32_t)c);
    }
    if (in_est) {
      est_ids[(size_t)g * es + est_off] = c;
      if (cI) cI[(size_t)g * k2 + np + est_off] = c;
      ++est_off;
    }
  }
  __syncthreads();

  // ---- order the retrieval zone: rank = number of larger composite keys (all distinct) ----
  for (int r = tid; r < np; r += SEL_THREADS) {
    const uint32_t mine = sh_ret[r];
    int rank = 0;
    for (int i = 0; i < np; ++i) rank += (sh_ret[i] > mine);
    sh_sorted[rank] = mine;
  }
  __syncthreads();

  // ---- token layout of the retrieved clusters with the page cut-off ----
  // thread t owns ranks [t*R, t*R+R)
  const int R = (np + SEL_THREADS - 1) / SEL_THREADS;  // <= 4 for np <= 1023
  uint32_t szs[4], pgs[4];
  int32_t sts[4];
  uint32_t psum = 0, tsum = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tid * R + i;
    szs[i] = pgs[i] = 0;
    sts[i] = 0;
    if (i < R && r < np) {
      const int c = (int)(0xffffu - (sh_sorted[r] & 0xffffu));
      ret_ids[(size_t)g * np + r] = c;
      if (cI) cI[(size_t)g * k2 + r] = c;
      if (cluster_size) {
        szs[i] = (uint32_t)cluster_size[(size_t)g * nc + c];
        pgs[i] = (szs[i] + page - 1) / page;
        if (cluster_start) sts[i] = cluster_start[(size_t)g * nc + c];
      }
    }
    psum += pgs[i];
    tsum += szs[i];
  }
  if (!cluster_size) return;
  const uint64_t lay = block_excl_scan<uint64_t>((uint64_t)psum | ((uint64_t)tsum << 32), sh_scan, &tot64);
  uint32_t pg_run = (uint32_t)lay, tok_run = (uint32_t)(lay >> 32);
  // kept clusters form a prefix because the page prefix is monotone; tokens before a kept
  // cluster all belong to kept clusters
  int kept_here = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tid * R + i;
    if (i < R && r < np) {
      const bool keep = pg_run + pgs[i] <= (uint32_t)max_pages;
      if (keep) {
        ++kept_here;
        sh_off[r] = (int32_t)tok_run;
        sh_ret[r] = (uint32_t)sts[i];  // sh_ret is free again: start row per rank
        atomicMax(&sh_pages, pg_run + pgs[i]);
        atomicMax(&sh_tret, tok_run + szs[i]);
      } else {
        sh_off[r] = -1;
      }
      pg_run += pgs[i];
      tok_run += szs[i];
    }
  }
  if (kept_here) atomicAdd(&sh_nk, kept_here);
  __syncthreads();
  const int nkeep = sh_nk;
  const int32_t T_ret = (int32_t)sh_tret;
  for (int r = tid; r <= np; r += SEL_THREADS) {
    const int32_t off = (r < nkeep) ? sh_off[r] : T_ret;
    ret_tok_off[(size_t)g * (np + 1) + r] = off;
  }
  if (tid == 0) {
    meta[g * 4 + 0] = nkeep;
    meta[g * 4 + 1] = T_ret;
    meta[g * 4 + 2] = (int32_t)sh_pages;
    meta[g * 4 + 3] = 0;
  }
  if (!row_src || !cluster_start) return;
  for (int rho = tid; rho < T_ret && rho < row_src_stride; rho += SEL_THREADS) {
    // last kept cluster r with sh_off[r] <= rho  (offsets of kept clusters are non-decreasing)
    int lo = 0, hi = nkeep - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (sh_off[mid] <= rho) lo = mid; else hi = mid - 1;
    }
    row_src[(size_t)g * row_src_stride + rho] = (int32_t)sh_ret[lo] + (rho - sh_off[lo]);
  }
}

// ------------------------------------------------------------------------------------
// C entry points
// ------------------------------------------------------------------------------------
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

extern "C" size_t ri_score_select_workspace_bytes(int BG, int gs, int nc) {
  if (BG <= 0 || gs <= 0 || nc <= 0) return 0;
  const size_t ntiles = (size_t)(nc + RI_SCORE_TILE - 1) / RI_SCORE_TILE;
  return 2 * align256((size_t)BG * ntiles * gs * sizeof(float)) + align256((size_t)BG * nc * sizeof(uint16_t)) +
         align256((size_t)BG * RI_SEL_HI_BINS * sizeof(uint32_t));
}

extern "C" int ri_score_select(const void* q, const void* centroids, const uint8_t* mask,
                               const int32_t* cluster_size_i32, const int32_t* cluster_start,
                               float* logits, void* dist, int64_t* cI, int32_t* ret_ids,
                               int32_t* est_ids, int32_t* ret_tok_off, int32_t* row_src,
                               int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np,
                               int es, int page, int max_pages, float scale, void* workspace,
                               size_t workspace_bytes, ri_stream_t stream) {
  if (!q || !centroids || !logits || !ret_ids || !workspace) return RI_ERR_ARG;
  if (BG <= 0 || gs <= 0 || gs > 16 || nc <= 0 || (nc % 8) != 0) return RI_ERR_ARG;
  if (np <= 0 || np > 1023 || es < 0 || np + es > nc || nc > 65536) return RI_ERR_ARG;
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
  w += align256((size_t)BG * nc * sizeof(uint16_t));
  uint32_t* ghist = (uint32_t*)w;
  int rc = ri_launch_score(q, centroids, logits, tmax, tsum, ghist, BG, gs, nc, scale, s);
  if (rc) return rc;
  const dim3 dgrid((nc + DIST_IDS - 1) / DIST_IDS, BG);
  if (gs <= 4)
    dist_kernel<4><<<dgrid, 256, 0, s>>>(logits, tmax, tsum, mask, keys, (uint16_t*)dist, ghist, gs, nc, ntiles);
  else if (gs <= 8)
    dist_kernel<8><<<dgrid, 256, 0, s>>>(logits, tmax, tsum, mask, keys, (uint16_t*)dist, ghist, gs, nc, ntiles);
  else
    dist_kernel<16><<<dgrid, 256, 0, s>>>(logits, tmax, tsum, mask, keys, (uint16_t*)dist, ghist, gs, nc, ntiles);
  RI_HIP_CHECK_LAUNCH();
  select_kernel<<<BG, SEL_THREADS, (size_t)nc * sizeof(uint16_t) + 64, s>>>(
      keys, ghist, cluster_size_i32, cluster_start, cI, ret_ids, est_ids, ret_tok_off, row_src, row_src_stride,
      meta, nc, np, es, page, max_pages);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
