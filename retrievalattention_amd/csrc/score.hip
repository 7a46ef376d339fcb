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

// Row statistics from the per-tile partials, in tile order (deterministic).
__device__ __forceinline__ void reduce_partials(const float* pm, const float* ps, int ntiles, int gs,
                                                int j, float* m_out, float* invz_out) {
  float m = -INFINITY;
  for (int t = 0; t < ntiles; ++t) m = fmaxf(m, pm[(size_t)t * gs + j]);
  float z = 0.f;
  for (int t = 0; t < ntiles; ++t) z += ps[(size_t)t * gs + j] * __expf(pm[(size_t)t * gs + j] - m);
  *m_out = m;
  *invz_out = 1.0f / z;
}

// batch_gemm_softmax tail: finals into slot 0 of Norm/Sum, then the bf16 softmax.
__global__ void softmax_reduce_kernel(float* norm, float* sum, int ntiles, int gs) {
  const int g = blockIdx.x;
  const int j = threadIdx.x;
  if (j >= gs) return;
  float m, iz;
  reduce_partials(norm + (size_t)g * ntiles * gs, sum + (size_t)g * ntiles * gs, ntiles, gs, j, &m, &iz);
  norm[(size_t)g * ntiles * gs + j] = m;
  sum[(size_t)g * ntiles * gs + j] = iz;
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

// Finds the bin holding descending rank `rank` in a 256-bin histogram.
// Every thread < 256 owns one bin; exactly one thread writes the answer.
__device__ __forceinline__ void find_bin_desc(const uint32_t* hist, uint32_t rank, uint32_t* out_bin,
                                              uint32_t* out_above) {
  if (threadIdx.x < 256) {
    const int b = threadIdx.x;
    uint32_t above = 0;
    for (int k = b + 1; k < 256; ++k) above += hist[k];
    if (above <= rank && rank < above + hist[b]) {
      *out_bin = (uint32_t)b;
      *out_above = above;
    }
  }
}

// ------------------------------------------------------------------------------------
// select_kernel: one 1024-thread workgroup per group.
// dynamic LDS: nc * 2 bytes of score keys.
// ------------------------------------------------------------------------------------
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
  __shared__ uint32_t hist_a[256], hist_b[256], hist_c[256];
  __shared__ uint32_t sh_scan[SEL_THREADS / 64];
  __shared__ uint32_t sh_sel[8];  // bin1, above1, bin2, above2, lo1, abovelo1, lo2, abovelo2
  __shared__ uint32_t sh_ret[1024];
  __shared__ int32_t sh_off[1025];
  __shared__ uint32_t sh_cnt;

  const int g = blockIdx.x;
  const int tid = threadIdx.x;
  const int k2 = np + es;

  if (tid < gs)
    reduce_partials(tile_max + (size_t)g * ntiles * gs, tile_sum + (size_t)g * ntiles * gs, ntiles, gs,
                    tid, &sh_m[tid], &sh_iz[tid]);
  if (tid < 256) hist_a[tid] = hist_b[tid] = hist_c[tid] = 0;
  if (tid == 0) sh_cnt = 0;
  __syncthreads();

  // thread t owns the contiguous id range [t*E, t*E+E)
  const int E = (nc + SEL_THREADS - 1) / SEL_THREADS;
  const int cbeg = tid * E;
  const int cend = min(cbeg + E, nc);

  // ---- scores ----
  for (int c = cbeg; c < cend; ++c) {
    float d = 0.f;
    for (int j = 0; j < gs; ++j) {
      const float x = logits[((size_t)g * gs + j) * nc + c];
      const float p = __expf(ri_round_bf16(x) - sh_m[j]) * sh_iz[j];
      d += ri_round_bf16(p);
    }
    uint16_t bits = ri_f32_to_bf16(d);
    if (mask && mask[(size_t)g * nc + c]) bits = 0xff7f;  // finfo(bfloat16).min
    if (dist_out) dist_out[(size_t)g * nc + c] = bits;
    const uint32_t key = ri_bf16_sort_key(bits);
    sh_key[c] = (uint16_t)key;
    atomicAdd(&hist_a[key >> 8], 1u);
  }
  __syncthreads();

  // ---- thresholds: T1 = key of rank np-1, T2 = key of rank k2-1 (descending) ----
  find_bin_desc(hist_a, (uint32_t)(np - 1), &sh_sel[0], &sh_sel[1]);
  find_bin_desc(hist_a, (uint32_t)(k2 - 1), &sh_sel[2], &sh_sel[3]);
  __syncthreads();
  const uint32_t hi1 = sh_sel[0], hi2 = sh_sel[2];
  for (int c = cbeg; c < cend; ++c) {
    const uint32_t key = sh_key[c];
    if ((key >> 8) == hi1) atomicAdd(&hist_b[key & 255u], 1u);
    if ((key >> 8) == hi2) atomicAdd(&hist_c[key & 255u], 1u);
  }
  __syncthreads();
  find_bin_desc(hist_b, (uint32_t)(np - 1) - sh_sel[1], &sh_sel[4], &sh_sel[5]);
  find_bin_desc(hist_c, (uint32_t)(k2 - 1) - sh_sel[3], &sh_sel[6], &sh_sel[7]);
  __syncthreads();
  const uint32_t T1 = (hi1 << 8) | sh_sel[4];
  const uint32_t T2 = (hi2 << 8) | sh_sel[6];
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
  uint32_t est_off = block_excl_scan(est_local, sh_scan, &tot);
  for (int c = cbeg; c < cend; ++c) {
    if (est_bits & (1ull << (c - cbeg))) {
      est_ids[(size_t)g * es + est_off] = c;
      if (cI) cI[(size_t)g * k2 + np + est_off] = c;
      ++est_off;
    }
  }
  __syncthreads();

  // ---- sort the retrieval zone: descending composite key (score, then smaller id) ----
  int P2 = 1;
  while (P2 < np) P2 <<= 1;
  if (tid >= np && tid < P2) sh_ret[tid] = 0u;
  __syncthreads();
  for (int k = 2; k <= P2; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      if (tid < P2) {
        const int ixj = tid ^ j;
        if (ixj > tid) {
          const uint32_t a = sh_ret[tid], b = sh_ret[ixj];
          const bool desc = (tid & k) == 0;
          if (desc ? (a < b) : (a > b)) {
            sh_ret[tid] = b;
            sh_ret[ixj] = a;
          }
        }
      }
      __syncthreads();
    }
  }
  int my_c = -1;
  if (tid < np) {
    my_c = (int)(0xffffu - (sh_ret[tid] & 0xffffu));
    ret_ids[(size_t)g * np + tid] = my_c;
    if (cI) cI[(size_t)g * k2 + tid] = my_c;
  }

  // ---- token layout of the retrieved clusters with the page cut-off ----
  if (!cluster_size) return;
  const uint32_t sz = (tid < np) ? (uint32_t)cluster_size[(size_t)g * nc + my_c] : 0u;
  const uint32_t pg = (sz + page - 1) / page;
  const uint32_t pg_excl = block_excl_scan(pg, sh_scan, &tot);
  const bool keep = (tid < np) && (pg_excl + pg <= (uint32_t)max_pages);
  // kept clusters form a prefix because the page prefix is monotone
  uint32_t kept_pages;
  const uint32_t tok_excl = block_excl_scan(keep ? sz : 0u, sh_scan, &tot);
  const uint32_t T_ret = tot;
  uint32_t nkeep_tot;
  block_excl_scan(keep ? 1u : 0u, sh_scan, &nkeep_tot);
  block_excl_scan(keep ? pg : 0u, sh_scan, &kept_pages);
  if (tid <= np) {
    const int32_t off = (tid < np && keep) ? (int32_t)tok_excl : (int32_t)T_ret;
    sh_off[tid] = off;
    ret_tok_off[(size_t)g * (np + 1) + tid] = off;
  }
  if (tid == 0) {
    meta[g * 4 + 0] = (int32_t)nkeep_tot;
    meta[g * 4 + 1] = (int32_t)T_ret;
    meta[g * 4 + 2] = (int32_t)kept_pages;
    meta[g * 4 + 3] = 0;
  }
  __syncthreads();
  if (!row_src || !cluster_start) return;
  const int nk = (int)nkeep_tot;
  for (int rho = tid; rho < (int)T_ret && rho < row_src_stride; rho += SEL_THREADS) {
    // last kept cluster r with sh_off[r] <= rho  (offsets are non-decreasing)
    int lo = 0, hi = nk - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (sh_off[mid] <= rho) lo = mid; else hi = mid - 1;
    }
    const int c = (int)(0xffffu - (sh_ret[lo] & 0xffffu));
    row_src[(size_t)g * row_src_stride + rho] = cluster_start[(size_t)g * nc + c] + (rho - sh_off[lo]);
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
  softmax_reduce_kernel<<<batch_count, 64, 0, s>>>(Norm, Sum, ntiles, m);
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
  select_kernel<<<BG, SEL_THREADS, (size_t)nc * sizeof(uint16_t), s>>>(
      logits, tmax, tsum, mask, cluster_size_i32, cluster_start, (uint16_t*)dist, cI, ret_ids, est_ids,
      ret_tok_off, row_src, row_src_stride, meta, gs, nc, ntiles, np, es, page, max_pages);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
