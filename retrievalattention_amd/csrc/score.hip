// Centroid scoring and cluster selection for the decode step (gfx950).
//
// score_kernel    : logits[g,j,c] = scale * <q[g,j,:], centroid[g,c,:]> on bf16 MFMA, streamed
//                   once over the centroids, plus per-256-column softmax partials.
// select_kernel   : per group, turns logits into the reference's bf16 score
//                   (sum over the query group of bf16 softmax values), then picks the
//                   retrieval zone (top np, rank order) and the estimation zone (next es)
//                   by radix select on the 16-bit score, and lays out the retrieved tokens.
// reduce/apply    : the two small kernels that complete the batch_gemm_softmax interface.
//
// Follows cache_hub/retroinfer_cache.py:569-575 and
// library/retroinfer/retroinfer_kernels/src/batch_gemm_softmax.h:222-243 (rounding pipeline).
#include "ri_common.h"

#define SCORE_TILE 256  // centroids per workgroup == width of one softmax partial
#define SEL_THREADS 1024

// ------------------------------------------------------------------------------------
// score_kernel: grid (ntiles, BG), 256 threads = 4 waves, each wave owns 64 centroids.
// MFMA 16x16x32: A = 16 centroid rows, B = query heads (columns >= gs are zero).
// Accumulator register i of lane l holds row 4*(l/16)+i, column l%16.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void score_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cent, float* __restrict__ logits,
    uint16_t* __restrict__ logits_bf16, float* __restrict__ tile_max, float* __restrict__ tile_sum,
    int gs, int nc, int ntiles, float scale) {
  const int tile = blockIdx.x;
  const int g = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15;
  const int h = lane >> 4;
  const int c0 = tile * SCORE_TILE + wave * 64;

  const uint16_t* cg = cent + (size_t)g * nc * RI_DIM;
  uint4 a[4][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = c0 + t * 16 + r;
    const bool ok = row < nc;
    const uint16_t* p = cg + (size_t)row * RI_DIM + h * 8;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) a[t][kk] = ok ? ri_ld16(p + kk * 32) : ri_zero16();
  }
  uint4 bq[4];
  {
    const uint16_t* p = q + ((size_t)g * gs + r) * RI_DIM + h * 8;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) bq[kk] = (r < gs) ? ri_ld16(p + kk * 32) : ri_zero16();
  }

  f32x4_t acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ri_as_bf16x8(a[t][kk]), ri_as_bf16x8(bq[kk]),
                                                       acc[t], 0, 0, 0);
  }

  // scale, store, and the partial row max over this lane's valid centroids
  float lmax = -INFINITY;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int cbase = c0 + t * 16 + 4 * h;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[t][i] *= scale;
      if (cbase + i < nc) lmax = fmaxf(lmax, acc[t][i]);
    }
    if (r < gs && cbase < nc) {  // nc % 4 == 0, so the four columns are valid together
      const size_t o = ((size_t)g * gs + r) * nc + cbase;
      if (logits)
        *reinterpret_cast<float4*>(logits + o) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
      if (logits_bf16) {
        uint2 pk;
        pk.x = (uint32_t)ri_f32_to_bf16(acc[t][0]) | ((uint32_t)ri_f32_to_bf16(acc[t][1]) << 16);
        pk.y = (uint32_t)ri_f32_to_bf16(acc[t][2]) | ((uint32_t)ri_f32_to_bf16(acc[t][3]) << 16);
        *reinterpret_cast<uint2*>(logits_bf16 + o) = pk;
      }
    }
  }

  __shared__ float sh_max[4][16];
  __shared__ float sh_sum[4][16];
  lmax = fmaxf(lmax, __shfl_xor(lmax, 16));
  lmax = fmaxf(lmax, __shfl_xor(lmax, 32));
  if (h == 0) sh_max[wave][r] = lmax;
  __syncthreads();
  const float tmax = fmaxf(fmaxf(sh_max[0][r], sh_max[1][r]), fmaxf(sh_max[2][r], sh_max[3][r]));
  float lsum = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int cbase = c0 + t * 16 + 4 * h;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (cbase + i < nc) lsum += __expf(acc[t][i] - tmax);
  }
  lsum += __shfl_xor(lsum, 16);
  lsum += __shfl_xor(lsum, 32);
  if (h == 0) sh_sum[wave][r] = lsum;
  __syncthreads();
  if (threadIdx.x < gs) {
    const int j = threadIdx.x;
    const float s = (sh_sum[0][j] + sh_sum[1][j]) + (sh_sum[2][j] + sh_sum[3][j]);
    const float m = fmaxf(fmaxf(sh_max[0][j], sh_max[1][j]), fmaxf(sh_max[2][j], sh_max[3][j]));
    const size_t o = ((size_t)g * ntiles + tile) * gs + j;
    tile_max[o] = m;
    tile_sum[o] = s;
  }
}

// Row statistics from the per-tile partials: one wave per row, lanes over tiles, xor-butterfly
// reductions (fixed order, so the result is reproducible).
__device__ __forceinline__ void wave_reduce_partials(const float* pm, const float* ps, int ntiles, int gs,
                                                     int j, int lane, float* m_out, float* invz_out) {
  float m = -INFINITY;
  for (int t = lane; t < ntiles; t += 64) m = fmaxf(m, pm[(size_t)t * gs + j]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  float z = 0.f;
  for (int t = lane; t < ntiles; t += 64) z += ps[(size_t)t * gs + j] * __expf(pm[(size_t)t * gs + j] - m);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) z += __shfl_xor(z, o);
  *m_out = m;
  *invz_out = 1.0f / z;
}

// batch_gemm_softmax tail: finals into slot 0 of Norm/Sum, then the bf16 softmax.
// grid = batch, block = 64 * gs (one wave per row)
__global__ void softmax_reduce_kernel(float* norm, float* sum, int ntiles, int gs) {
  const int g = blockIdx.x;
  const int j = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float m, iz;
  wave_reduce_partials(norm + (size_t)g * ntiles * gs, sum + (size_t)g * ntiles * gs, ntiles, gs, j, lane, &m,
                       &iz);
  __syncthreads();  // every row has read slot 0 before anyone overwrites it
  if (lane == 0) {
    norm[(size_t)g * ntiles * gs + j] = m;
    sum[(size_t)g * ntiles * gs + j] = iz;
  }
}

__global__ __launch_bounds__(256) void softmax_apply_kernel(const uint16_t* __restrict__ d,
                                                            const float* __restrict__ norm,
                                                            const float* __restrict__ sum,
                                                            uint16_t* __restrict__ soft, int ntiles,
                                                            int gs, int nc) {
  const int g = blockIdx.z, j = blockIdx.y;
  const float m = norm[(size_t)g * ntiles * gs + j];
  const float iz = sum[(size_t)g * ntiles * gs + j];
  const size_t base = ((size_t)g * gs + j) * nc;
  for (int c = (blockIdx.x * 256 + threadIdx.x) * 4; c < nc; c += gridDim.x * 256 * 4) {
    const uint2 v = *reinterpret_cast<const uint2*>(d + base + c);
    const uint16_t in[4] = {(uint16_t)(v.x & 0xffff), (uint16_t)(v.x >> 16), (uint16_t)(v.y & 0xffff),
                            (uint16_t)(v.y >> 16)};
    uint16_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = ri_f32_to_bf16(__expf(ri_bf16_to_f32(in[i]) - m) * iz);
    uint2 w;
    w.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
    w.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
    *reinterpret_cast<uint2*>(soft + base + c) = w;
  }
}

// ------------------------------------------------------------------------------------
// select_kernel helpers
// ------------------------------------------------------------------------------------
// exclusive prefix sum over the 1024 threads of the block; *total receives the sum
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t* sh16, uint32_t* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t n = __shfl_up(inc, d);
    if (lane >= d) inc += n;
  }
  __syncthreads();  // sh16 may still be read from a previous scan
  if (lane == 63) sh16[wave] = inc;
  __syncthreads();
  uint32_t woff = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < SEL_THREADS / 64; ++w) {
    const uint32_t s = sh16[w];
    if (w < wave) woff += s;
    tot += s;
  }
  *total = tot;
  return woff + inc - v;
}

// Histogram add that survives a degenerate distribution: when the whole wave hits one bin
// (for instance every score equal) a single lane adds the lane count.
__device__ __forceinline__ void hist_add(uint32_t* hist, uint32_t bin, bool active) {
  const uint64_t act = __ballot(active);
  if (act == 0) return;
  const uint32_t first = __shfl(bin, __ffsll((long long)act) - 1);
  const uint64_t same = __ballot(active && bin == first);
  if (same == act) {
    if ((threadIdx.x & 63) == __ffsll((long long)act) - 1) atomicAdd(&hist[first], (uint32_t)__popcll(act));
  } else if (active) {
    atomicAdd(&hist[bin], 1u);
  }
}

#define SEL_HI_BITS 11                     // first radix pass: top 11 bits of the 16-bit key
#define SEL_HI_BINS (1 << SEL_HI_BITS)     // 2048 bins, two per thread
#define SEL_LO_BITS (16 - SEL_HI_BITS)
#define SEL_LO_BINS (1 << SEL_LO_BITS)     // 32 bins

// Over the 2048-bin histogram (thread t owns bins 2t, 2t+1): for two descending ranks, the
// bin holding each and the count of entries in higher bins.  All threads call.
// out[0..1] = bin, above for rankA; out[2..3] for rankB.
__device__ __forceinline__ void find_hi_bins(const uint32_t* hist, uint32_t rankA, uint32_t rankB,
                                             uint32_t* sh16, uint32_t* out) {
  const int tid = threadIdx.x;
  const uint32_t h0 = hist[2 * tid], h1 = hist[2 * tid + 1];
  uint32_t tot;
  const uint32_t below = block_excl_scan(h0 + h1, sh16, &tot);  // entries in bins < 2t
  const uint32_t above1 = tot - below - h0 - h1;                // entries in bins > 2t+1
  const uint32_t above0 = above1 + h1;                          // entries in bins > 2t
  if (above1 <= rankA && rankA < above1 + h1) { out[0] = 2 * tid + 1; out[1] = above1; }
  if (above0 <= rankA && rankA < above0 + h0) { out[0] = 2 * tid; out[1] = above0; }
  if (above1 <= rankB && rankB < above1 + h1) { out[2] = 2 * tid + 1; out[3] = above1; }
  if (above0 <= rankB && rankB < above0 + h0) { out[2] = 2 * tid; out[3] = above0; }
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
// select_kernel: one 1024-thread workgroup per group.
// dynamic LDS: nc * 2 bytes of score keys.
// ------------------------------------------------------------------------------------
// GSM = compile-time bound on gs (4, 8 or 16): sizes the logits preload.
template <int GSM>
__global__ __launch_bounds__(SEL_THREADS) void select_kernel(
    const float* __restrict__ logits, const float* __restrict__ tile_max,
    const float* __restrict__ tile_sum, const uint8_t* __restrict__ mask,
    const int32_t* __restrict__ cluster_size, const int32_t* __restrict__ cluster_start,
    uint16_t* __restrict__ dist_out, int64_t* __restrict__ cI, int32_t* __restrict__ ret_ids,
    int32_t* __restrict__ est_ids, int32_t* __restrict__ ret_tok_off, int32_t* __restrict__ row_src,
    int row_src_stride, int32_t* __restrict__ meta, int gs, int nc, int ntiles, int np, int es,
    int page, int max_pages) {
  extern __shared__ uint16_t sh_key[];
  __shared__ float sh_m[16], sh_iz[16];
  __shared__ uint32_t hist_a[SEL_HI_BINS], hist_b[SEL_LO_BINS], hist_c[SEL_LO_BINS];
  __shared__ uint32_t sh_scan[SEL_THREADS / 64];
  __shared__ uint32_t sh_sel[12];  // hi1, above, hi2, above, lo1, above, lo2, above (+ unused tail)
  __shared__ uint32_t sh_ret[1024];
  __shared__ uint32_t sh_sorted[1024];
  __shared__ int32_t sh_off[1025];
  __shared__ uint32_t sh_cnt, sh_pages;

  const int g = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int k2 = np + es;

  // thread t owns the contiguous id range [t*E, t*E+E), E a multiple of 4 (nc % 4 == 0)
  const int E = (((nc + SEL_THREADS - 1) / SEL_THREADS) + 3) & ~3;
  const int cbeg = min(tid * E, nc);
  const int cend = min(cbeg + E, nc);

  // Issue the logits loads of the first tiles (4 ids each) before anything else: every
  // dependent step below then hides behind one memory latency instead of adding its own.
  constexpr int PRE = GSM <= 8 ? 2 : 1;
  float4 xpre[PRE][GSM];
#pragma unroll
  for (int t = 0; t < PRE; ++t)
#pragma unroll
    for (int j = 0; j < GSM; ++j)
      if (j < gs && cbeg + 4 * t < cend)
        xpre[t][j] = *reinterpret_cast<const float4*>(logits + ((size_t)g * gs + j) * nc + cbeg + 4 * t);
  uint32_t mpre[PRE];
#pragma unroll
  for (int t = 0; t < PRE; ++t)
    mpre[t] = (mask && cbeg + 4 * t < cend) ? *reinterpret_cast<const uint32_t*>(mask + (size_t)g * nc + cbeg + 4 * t) : 0u;

  if (wave < gs) {
    float m, iz;
    wave_reduce_partials(tile_max + (size_t)g * ntiles * gs, tile_sum + (size_t)g * ntiles * gs, ntiles, gs,
                         wave, lane, &m, &iz);
    if (lane == 0) { sh_m[wave] = m; sh_iz[wave] = iz; }
  }
  hist_a[2 * tid] = hist_a[2 * tid + 1] = 0;
  if (tid < SEL_LO_BINS) hist_b[tid] = hist_c[tid] = 0;
  if (tid == 0) { sh_cnt = 0; sh_pages = 0; }
  __syncthreads();

  // ---- scores: dist = bf16(sum_j bf16(exp(bf16(x_j) - m_j) / Z_j)) ----
  auto score_tile = [&](int c, const float4* x4s, uint32_t mk) {
    float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < GSM; ++j) {
      if (j < gs) {
        const float x[4] = {x4s[j].x, x4s[j].y, x4s[j].z, x4s[j].w};
        const float m = sh_m[j], iz = sh_iz[j];
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] += ri_round_bf16(__expf(ri_round_bf16(x[i]) - m) * iz);
      }
    }
    uint16_t bits[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bits[i] = ri_f32_to_bf16(d[i]);
      if ((mk >> (8 * i)) & 0xffu) bits[i] = 0xff7f;  // finfo(bfloat16).min
      const uint32_t key = ri_bf16_sort_key(bits[i]);
      sh_key[c + i] = (uint16_t)key;
      hist_add(hist_a, key >> SEL_LO_BITS, true);
    }
    if (dist_out) {
      uint2 w;
      w.x = (uint32_t)bits[0] | ((uint32_t)bits[1] << 16);
      w.y = (uint32_t)bits[2] | ((uint32_t)bits[3] << 16);
      *reinterpret_cast<uint2*>(dist_out + (size_t)g * nc + c) = w;
    }
  };
#pragma unroll
  for (int t = 0; t < PRE; ++t)
    if (cbeg + 4 * t < cend) score_tile(cbeg + 4 * t, xpre[t], mpre[t]);
  for (int c = cbeg + 4 * PRE; c < cend; c += 4) {
    float4 x4s[GSM];
#pragma unroll
    for (int j = 0; j < GSM; ++j)
      if (j < gs) x4s[j] = *reinterpret_cast<const float4*>(logits + ((size_t)g * gs + j) * nc + c);
    score_tile(c, x4s, mask ? *reinterpret_cast<const uint32_t*>(mask + (size_t)g * nc + c) : 0u);
  }
  __syncthreads();

  // ---- thresholds: T1 = key of rank np-1, T2 = key of rank k2-1 (descending) ----
  find_hi_bins(hist_a, (uint32_t)(np - 1), (uint32_t)(k2 - 1), sh_scan, sh_sel);
  __syncthreads();
  const uint32_t hi1 = sh_sel[0], hi2 = sh_sel[2];
  for (int c = cbeg; c < cbeg + E; ++c) {   // same trip count in every lane of a wave
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

  // ---- rank of tied keys by ascending id (stable: threads own ascending id ranges) ----
  uint32_t n1 = 0, n2 = 0;
  for (int c = cbeg; c < cend; ++c) {
    const uint32_t key = sh_key[c];
    n1 += (key == T1);
    n2 += (key == T2);
  }
  uint32_t tot;
  const uint32_t packed = block_excl_scan(n1 | (n2 << 16), sh_scan, &tot);
  uint32_t r1 = packed & 0xffffu, r2 = packed >> 16;

  // ---- zones ----
  uint32_t est_local = 0;
  uint64_t est_bits = 0;  // E <= 64
  for (int c = cbeg; c < cend; ++c) {
    const uint32_t key = sh_key[c];
    bool in_ret, in_est;
    if (key == T1) {
      const uint32_t pos = g1 + r1;
      in_ret = pos < (uint32_t)np;
      in_est = !in_ret && pos < (uint32_t)k2;
    } else if (key == T2) {
      in_ret = false;
      in_est = (g2 + r2) < (uint32_t)k2;
    } else {
      in_ret = key > T1;
      in_est = !in_ret && key > T2;
    }
    r1 += (key == T1);
    r2 += (key == T2);
    if (in_ret) {
      const uint32_t slot = atomicAdd(&sh_cnt, 1u);
      sh_ret[slot] = (key << 16) | (0xffffu - (uint32_t)c);
    }
    if (in_est) {
      est_bits |= 1ull << (c - cbeg);
      ++est_local;
    }
  }
  uint32_t est_off = block_excl_scan(est_local, sh_scan, &tot);  // also orders sh_ret writes
  for (int c = cbeg; c < cend; ++c) {
    if (est_bits & (1ull << (c - cbeg))) {
      est_ids[(size_t)g * es + est_off] = c;
      if (cI) cI[(size_t)g * k2 + np + est_off] = c;
      ++est_off;
    }
  }

  // ---- order the retrieval zone: rank = number of larger composite keys (all distinct) ----
  int my_c = -1;
  if (tid < np) {
    const uint32_t mine = sh_ret[tid];
    int rank = 0;
    for (int i = 0; i < np; ++i) rank += (sh_ret[i] > mine);
    sh_sorted[rank] = mine;
  }
  __syncthreads();
  if (tid < np) {
    my_c = (int)(0xffffu - (sh_sorted[tid] & 0xffffu));
    ret_ids[(size_t)g * np + tid] = my_c;
    if (cI) cI[(size_t)g * k2 + tid] = my_c;
  }

  // ---- token layout of the retrieved clusters with the page cut-off ----
  if (!cluster_size) return;
  const uint32_t sz = (tid < np) ? (uint32_t)cluster_size[(size_t)g * nc + my_c] : 0u;
  const int32_t my_start = (tid < np && cluster_start) ? cluster_start[(size_t)g * nc + my_c] : 0;
  const uint32_t pg = (sz + page - 1) / page;
  const uint32_t pg_excl = block_excl_scan(pg, sh_scan, &tot);
  // kept clusters form a prefix because the page prefix is monotone
  const bool keep = (tid < np) && (pg_excl + pg <= (uint32_t)max_pages);
  if (keep) atomicMax(&sh_pages, pg_excl + pg);
  const uint32_t tok_excl = block_excl_scan(keep ? sz : 0u, sh_scan, &tot);
  const uint32_t T_ret = tot;
  const int nk = __syncthreads_count(keep);
  if (tid <= np) {
    const int32_t off = (tid < np && keep) ? (int32_t)tok_excl : (int32_t)T_ret;
    sh_off[tid] = off;
    ret_tok_off[(size_t)g * (np + 1) + tid] = off;
  }
  if (tid < np) sh_ret[tid] = (uint32_t)my_start;  // sh_ret is free again: start row per rank
  __syncthreads();
  if (tid == 0) {
    meta[g * 4 + 0] = nk;
    meta[g * 4 + 1] = (int32_t)T_ret;
    meta[g * 4 + 2] = (int32_t)sh_pages;
    meta[g * 4 + 3] = 0;
  }
  if (!row_src || !cluster_start) return;
  for (int rho = tid; rho < (int)T_ret && rho < row_src_stride; rho += SEL_THREADS) {
    // last kept cluster r with sh_off[r] <= rho  (offsets are non-decreasing)
    int lo = 0, hi = nk - 1;
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
static int check_score_shape(int BG, int gs, int nc, int k) {
  if (BG <= 0 || gs <= 0 || gs > 16 || nc <= 0 || (nc % 8) != 0 || k != RI_DIM) return RI_ERR_ARG;
  return RI_OK;
}

extern "C" int ri_batch_gemm_softmax(const void* A, const void* B, void* D, float* Norm, float* Sum,
                                     void* Softmax, int batch_count, int m, int n, int k, float alpha,
                                     float beta, ri_stream_t stream) {
  if (!A || !B || !D || !Norm || !Sum || !Softmax || beta != 0.f) return RI_ERR_ARG;
  int rc = check_score_shape(batch_count, m, n, k);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const int ntiles = (n + SCORE_TILE - 1) / SCORE_TILE;
  // fp32 logits are not part of this interface: the partial statistics come from the fp32
  // accumulators inside the kernel, the softmax from the bf16 D, as in the reference.
  score_kernel<<<dim3(ntiles, batch_count), 256, 0, s>>>((const uint16_t*)A, (const uint16_t*)B, nullptr,
                                                         (uint16_t*)D, Norm, Sum, m, n, ntiles, alpha);
  RI_HIP_CHECK_LAUNCH();
  softmax_reduce_kernel<<<batch_count, 64 * m, 0, s>>>(Norm, Sum, ntiles, m);
  RI_HIP_CHECK_LAUNCH();
  int bx = (n + 1023) / 1024;
  if (bx > 16) bx = 16;
  softmax_apply_kernel<<<dim3(bx, m, batch_count), 256, 0, s>>>((const uint16_t*)D, Norm, Sum,
                                                                (uint16_t*)Softmax, ntiles, m, n);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" size_t ri_score_select_workspace_bytes(int BG, int gs, int nc) {
  if (BG <= 0 || gs <= 0 || nc <= 0) return 0;
  const size_t ntiles = (size_t)(nc + SCORE_TILE - 1) / SCORE_TILE;
  return 2 * (size_t)BG * ntiles * gs * sizeof(float);
}

extern "C" int ri_score_select(const void* q, const void* centroids, const uint8_t* mask,
                               const int32_t* cluster_size_i32, const int32_t* cluster_start,
                               float* logits, void* dist, int64_t* cI, int32_t* ret_ids,
                               int32_t* est_ids, int32_t* ret_tok_off, int32_t* row_src,
                               int row_src_stride, int32_t* meta, int BG, int gs, int nc, int np,
                               int es, int page, int max_pages, float scale, void* workspace,
                               size_t workspace_bytes, ri_stream_t stream) {
  if (!q || !centroids || !logits || !ret_ids || !workspace) return RI_ERR_ARG;
  int rc = check_score_shape(BG, gs, nc, RI_DIM);
  if (rc) return rc;
  if (np <= 0 || np > 1023 || es < 0 || np + es > nc || nc > 65536) return RI_ERR_ARG;
  if (es > 0 && !est_ids) return RI_ERR_ARG;
  if (cluster_size_i32 && (!ret_tok_off || !meta || page <= 0 || max_pages <= 0)) return RI_ERR_ARG;
  if (workspace_bytes < ri_score_select_workspace_bytes(BG, gs, nc)) return RI_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const int ntiles = (nc + SCORE_TILE - 1) / SCORE_TILE;
  float* tmax = (float*)workspace;
  float* tsum = tmax + (size_t)BG * ntiles * gs;
  score_kernel<<<dim3(ntiles, BG), 256, 0, s>>>((const uint16_t*)q, (const uint16_t*)centroids, logits,
                                                nullptr, tmax, tsum, gs, nc, ntiles, scale);
  RI_HIP_CHECK_LAUNCH();
#define RI_LAUNCH_SELECT(GSM)                                                                              \
  select_kernel<GSM><<<BG, SEL_THREADS, (size_t)nc * sizeof(uint16_t), s>>>(                                \
      logits, tmax, tsum, mask, cluster_size_i32, cluster_start, (uint16_t*)dist, cI, ret_ids, est_ids,     \
      ret_tok_off, row_src, row_src_stride, meta, gs, nc, ntiles, np, es, page, max_pages)
  if (gs <= 4) RI_LAUNCH_SELECT(4);
  else if (gs <= 8) RI_LAUNCH_SELECT(8);
  else RI_LAUNCH_SELECT(16);
#undef RI_LAUNCH_SELECT
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
