// Centroid scoring and cluster selection for the decode step (gfx950).
//
// score_kernel    : logits[g,j,c] = scale * <q[g,j,:], centroid[g,c,:]> on bf16 MFMA, streamed
//                   once over the centroids, plus per-256-column softmax partials.
// reduce/apply    : the two small kernels that complete the batch_gemm_softmax interface.
//
// Follows cache_hub/retroinfer_cache.py:569-575 and
// library/retroinfer/retroinfer_kernels/src/batch_gemm_softmax.h:222-243 (rounding pipeline).
#include "ri_common.h"

#define SCORE_TILE RI_SCORE_TILE  // centroids per workgroup == width of one softmax partial

// ------------------------------------------------------------------------------------
// score_kernel: grid (ntiles, BG), 256 threads = 4 waves, each wave owns 64 centroids.
// MFMA 16x16x32: A = 16 centroid rows, B = query heads (columns >= gs are zero).
// Accumulator register i of lane l holds row 4*(l/16)+i, column l%16.
// ------------------------------------------------------------------------------------
// HALF: the 16-bit element type of q, cent and the 16-bit logits is IEEE half instead of bfloat16
// (batch_gemm_softmax.cu:185-197 dispatches on Half and BFloat16).
template <bool HALF>
__device__ __forceinline__ uint16_t score_f32_to_16(float f) { return ri_f32_to_e16<HALF>(f); }
template <bool HALF>
__device__ __forceinline__ float score_16_to_f32(uint16_t v) { return ri_e16_to_f32<HALF>(v); }

// TPW = 16-row centroid tiles per wave: a workgroup covers SCORE_TILE = 256 centroids with 16 / TPW waves.
// Launched with 4 (four waves, sixteen loads in flight per lane); eight waves with eight loads and sixteen with
// four were slower (29.96 and 32.1 us against 29.6 us for scoring + selection at 32 groups of 8192 centroids).
// Softmax partials of the 256 columns with one barrier: every wave reduces its own columns to a maximum and a
// sum of exponentials relative to that maximum, and after the barrier one thread per head folds the wave pairs
// (max of the maxima, sums rescaled by exp(m_w - M)).
template <bool HALF, int TPW>
__device__ __forceinline__ void score_body(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cent, float* __restrict__ logits,
    uint16_t* __restrict__ logits_bf16, float* __restrict__ tile_max, float* __restrict__ tile_sum,
    int gs, int nc, int ntiles, float scale) {
  constexpr int NWV = 16 / TPW;
  const int tile = blockIdx.x;
  const int g = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15;
  const int h = lane >> 4;
  const int c0 = tile * SCORE_TILE + wave * (16 * TPW);

  const uint16_t* cg = cent + (size_t)g * nc * RI_DIM;
  uint4 a[TPW][4];
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
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

  f32x4_t acc[TPW];
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
      acc[t] = HALF ? __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a[t][kk]),
                                                             __builtin_bit_cast(f16x8_t, bq[kk]), acc[t], 0, 0, 0)
                    : __builtin_amdgcn_mfma_f32_16x16x32_bf16(ri_as_bf16x8(a[t][kk]), ri_as_bf16x8(bq[kk]),
                                                              acc[t], 0, 0, 0);
  }

  // scale, and the wave's row maximum over its valid centroids.  The logits are stored at
  // the very end: a barrier waits for outstanding stores too.
  float lmax = -INFINITY;
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const int cbase = c0 + t * 16 + 4 * h;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[t][i] *= scale;
      if (cbase + i < nc) lmax = fmaxf(lmax, acc[t][i]);
    }
  }
  __shared__ float sh_max[NWV][16];
  __shared__ float sh_sum[NWV][16];
  lmax = fmaxf(lmax, __shfl_xor(lmax, 16));
  lmax = fmaxf(lmax, __shfl_xor(lmax, 32));
  float lsum = 0.f;
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const int cbase = c0 + t * 16 + 4 * h;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (cbase + i < nc) lsum += __expf(acc[t][i] - lmax);
  }
  lsum += __shfl_xor(lsum, 16);
  lsum += __shfl_xor(lsum, 32);
  if (h == 0) {
    sh_max[wave][r] = lmax;
    sh_sum[wave][r] = lsum;
  }
  __syncthreads();
  if ((int)threadIdx.x < gs) {
    const int j = threadIdx.x;
    float m = sh_max[0][j];
#pragma unroll
    for (int w = 1; w < NWV; ++w) m = fmaxf(m, sh_max[w][j]);
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      const float mw = sh_max[w][j];
      s += (mw == -INFINITY) ? 0.f : sh_sum[w][j] * __expf(mw - m);   // a wave past the last centroid holds nothing
    }
    const size_t o = ((size_t)g * ntiles + tile) * gs + j;
    tile_max[o] = m;
    tile_sum[o] = s;
  }
#pragma unroll
  for (int t = 0; t < TPW; ++t) {
    const int cbase = c0 + t * 16 + 4 * h;
    if (r < gs && cbase < nc) {  // nc % 4 == 0, so the four columns are valid together
      const size_t o = ((size_t)g * gs + r) * nc + cbase;
      if (logits) {
        // streaming store: the 4 MB of logits leave the cache as they are written instead of waiting, dirty,
        // for the write-back at the end of the kernel (about 1 us per step at 32 groups of 8192 centroids)
        typedef float score_f4 __attribute__((ext_vector_type(4)));
        const score_f4 val = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
        __builtin_nontemporal_store(val, reinterpret_cast<score_f4*>(logits + o));
      }
      if (logits_bf16) {
        uint2 pk;
        pk.x = (uint32_t)score_f32_to_16<HALF>(acc[t][0]) | ((uint32_t)score_f32_to_16<HALF>(acc[t][1]) << 16);
        pk.y = (uint32_t)score_f32_to_16<HALF>(acc[t][2]) | ((uint32_t)score_f32_to_16<HALF>(acc[t][3]) << 16);
        *reinterpret_cast<uint2*>(logits_bf16 + o) = pk;
      }
    }
  }
}

template <bool HALF, int TPW>
__global__ __launch_bounds__(1024 / TPW) void score_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cent, float* __restrict__ logits,
    uint16_t* __restrict__ logits16, float* __restrict__ tile_max, float* __restrict__ tile_sum,
    int gs, int nc, int ntiles, float scale) {
  score_body<HALF, TPW>(q, cent, logits, logits16, tile_max, tile_sum, gs, nc, ntiles, scale);
}

// batch_gemm_softmax tail: finals into slot 0 of Norm/Sum, then the bf16 softmax.
// grid = batch, block = 64 * gs (one wave per row)
__global__ void softmax_reduce_kernel(float* norm, float* sum, int ntiles, int gs) {
  const int g = blockIdx.x;
  const int j = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float m, iz;
  ri_wave_reduce_partials(norm + (size_t)g * ntiles * gs, sum + (size_t)g * ntiles * gs, ntiles, gs, j, lane, &m,
                       &iz);
  __syncthreads();  // every row has read slot 0 before anyone overwrites it
  if (lane == 0) {
    norm[(size_t)g * ntiles * gs + j] = m;
    sum[(size_t)g * ntiles * gs + j] = iz;
  }
}

template <bool HALF>
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
    for (int i = 0; i < 4; ++i) o[i] = score_f32_to_16<HALF>(__expf(score_16_to_f32<HALF>(in[i]) - m) * iz);
    uint2 w;
    w.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
    w.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
    *reinterpret_cast<uint2*>(soft + base + c) = w;
  }
}

// ------------------------------------------------------------------------------------
// C entry points
// ------------------------------------------------------------------------------------
static int check_score_shape(int BG, int gs, int nc, int k) {
  if (BG <= 0 || gs <= 0 || gs > 16 || nc <= 0 || (nc % 8) != 0 || k != RI_DIM) return RI_ERR_ARG;
  return RI_OK;
}

template <bool HALF>
static int batch_gemm_softmax_impl(const void* A, const void* B, void* D, float* Norm, float* Sum, void* Softmax,
                                   int batch_count, int m, int n, int k, float alpha, float beta,
                                   ri_stream_t stream) {
  if (!A || !B || !D || !Norm || !Sum || !Softmax || beta != 0.f) return RI_ERR_ARG;
  if (ri_any_misaligned16(A, B, D, Softmax)) return RI_ERR_ARG;
  int rc = check_score_shape(batch_count, m, n, k);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const int ntiles = (n + SCORE_TILE - 1) / SCORE_TILE;
  // fp32 logits are not part of this interface: the partial statistics come from the fp32
  // accumulators inside the kernel, the softmax from the 16-bit D, as in the reference.
  score_kernel<HALF, 4><<<dim3(ntiles, batch_count), 256, 0, s>>>((const uint16_t*)A, (const uint16_t*)B, nullptr,
                                                                  (uint16_t*)D, Norm, Sum, m, n, ntiles, alpha);
  RI_HIP_CHECK_LAUNCH();
  softmax_reduce_kernel<<<batch_count, 64 * m, 0, s>>>(Norm, Sum, ntiles, m);
  RI_HIP_CHECK_LAUNCH();
  int bx = (n + 1023) / 1024;
  if (bx > 16) bx = 16;
  softmax_apply_kernel<HALF><<<dim3(bx, m, batch_count), 256, 0, s>>>((const uint16_t*)D, Norm, Sum,
                                                                      (uint16_t*)Softmax, ntiles, m, n);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" int ri_batch_gemm_softmax(const void* A, const void* B, void* D, float* Norm, float* Sum,
                                     void* Softmax, int batch_count, int m, int n, int k, float alpha,
                                     float beta, ri_stream_t stream) {
  return batch_gemm_softmax_impl<false>(A, B, D, Norm, Sum, Softmax, batch_count, m, n, k, alpha, beta, stream);
}

extern "C" int ri_batch_gemm_softmax_f16(const void* A, const void* B, void* D, float* Norm, float* Sum,
                                         void* Softmax, int batch_count, int m, int n, int k, float alpha,
                                         float beta, ri_stream_t stream) {
  return batch_gemm_softmax_impl<true>(A, B, D, Norm, Sum, Softmax, batch_count, m, n, k, alpha, beta, stream);
}


// scoring pass used by the fused selection (select.hip)
int ri_launch_score(const void* q, const void* centroids, float* logits, float* tile_max, float* tile_sum,
                    int BG, int gs, int nc, float scale, bool half, hipStream_t s) {
  const int ntiles = (nc + SCORE_TILE - 1) / SCORE_TILE;
  const uint16_t *qq = (const uint16_t*)q, *cc = (const uint16_t*)centroids;
  if (half)
    score_kernel<true, 4><<<dim3(ntiles, BG), 256, 0, s>>>(qq, cc, logits, nullptr, tile_max, tile_sum, gs, nc,
                                                           ntiles, scale);
  else
    score_kernel<false, 4><<<dim3(ntiles, BG), 256, 0, s>>>(qq, cc, logits, nullptr, tile_max, tile_sum, gs, nc,
                                                            ntiles, scale);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
