// Shared device/host helpers for the gfx950 wave-index kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/retro_mi355.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define RI_DIM 128  // head dimension every kernel is specialised for

// ---- bf16 <-> fp32 (round-to-nearest-even, NaN preserved as quiet NaN) ----
__host__ __device__ __forceinline__ float ri_bf16_to_f32(uint16_t v) {
  union { uint32_t u; float f; } x;
  x.u = (uint32_t)v << 16;
  return x.f;
}
__host__ __device__ __forceinline__ uint16_t ri_f32_to_bf16(float f) {
  union { uint32_t u; float f; } x;
  x.f = f;
  if ((x.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x.u >> 16) | 0x40u);
  uint32_t r = ((x.u >> 16) & 1u) + 0x7fffu;
  return (uint16_t)((x.u + r) >> 16);
}
// fp32 value of the bf16 rounding of f
__host__ __device__ __forceinline__ float ri_round_bf16(float f) {
  return ri_bf16_to_f32(ri_f32_to_bf16(f));
}

// ---- the two 16-bit element types: bfloat16 (HALF = false) and IEEE half (HALF = true) ----
// The fused decode path, the k-means and the operators take either (the reference's operators and cache are
// generic over Half and BFloat16: batch_gemm_softmax.cu:185-197, gather_copy.cu:63-67); a kernel is
// instantiated per type and the entry points come in pairs (name, name_f16).
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));

template <bool HALF>
__host__ __device__ __forceinline__ float ri_e16_to_f32(uint16_t v) {
  if (HALF) {
#if defined(__HIP_DEVICE_COMPILE__)
    return (float)__builtin_bit_cast(_Float16, v);
#else
    // host side: plain bit arithmetic (normal, subnormal, inf/nan)
    const uint32_t s = (uint32_t)(v & 0x8000u) << 16, e = (v >> 10) & 31u, m = v & 0x3ffu;
    union { uint32_t u; float f; } x;
    if (e == 0) {
      x.f = (float)m * 5.9604644775390625e-08f;   // m * 2^-24
      x.u |= s;
    } else {
      x.u = s | (e == 31 ? 0x7f800000u : (e + 112u) << 23) | (m << 13);
    }
    return x.f;
#endif
  }
  return ri_bf16_to_f32(v);
}
// round to nearest even
template <bool HALF>
__device__ __forceinline__ uint16_t ri_f32_to_e16(float f) {
  if (HALF) return __builtin_bit_cast(uint16_t, (_Float16)f);
  return ri_f32_to_bf16(f);
}
// fp32 value of the 16-bit rounding of f
template <bool HALF>
__device__ __forceinline__ float ri_round_e16(float f) {
  return ri_e16_to_f32<HALF>(ri_f32_to_e16<HALF>(f));
}
// the two elements packed in a 32-bit word, as fp32
template <bool HALF>
__device__ __forceinline__ void ri_unpack2(uint32_t w, float& lo, float& hi) {
  if (HALF) {
    lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
    hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
  } else {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  }
}
// finfo(type).min as a bit pattern: the score of a masked (empty) cluster
template <bool HALF>
__host__ __device__ __forceinline__ uint16_t ri_e16_lowest() { return HALF ? 0xfbff : 0xff7f; }

__device__ __forceinline__ bf16x8_t ri_as_bf16x8(uint4 v) {
  return __builtin_bit_cast(bf16x8_t, v);
}
__device__ __forceinline__ uint4 ri_ld16(const void* p) {
  return *reinterpret_cast<const uint4*>(p);
}
__device__ __forceinline__ uint4 ri_zero16() { return make_uint4(0u, 0u, 0u, 0u); }

// unpack 8 bf16 packed in a uint4 into fp32
__device__ __forceinline__ void ri_unpack8(uint4 v, float* f) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

// bf16 bit pattern -> key whose unsigned order equals the float order
__host__ __device__ __forceinline__ uint32_t ri_bf16_sort_key(uint16_t b) {
  return (b & 0x8000u) ? (uint32_t)(~b & 0xffffu) : (uint32_t)(b | 0x8000u);
}

// Rows of bf16 matrices are read and written 16 bytes at a time: their base pointers must be
// 16-byte aligned (a null pointer counts as aligned: optional arguments are checked elsewhere).
static inline bool ri_misaligned16(const void* p) { return ((uintptr_t)p & 15u) != 0; }
template <typename... P>
static inline bool ri_any_misaligned16(P... p) {
  return (ri_misaligned16((const void*)p) || ...);
}

#define RI_HIP_CHECK_LAUNCH()                         \
  do {                                                \
    hipError_t e__ = hipGetLastError();               \
    if (e__ != hipSuccess) {                          \
      ri_set_last_hip_error((int)e__);                \
      return RI_ERR_LAUNCH;                           \
    }                                                 \
  } while (0)

void ri_set_last_hip_error(int e);

// ---- shared between score.hip and select.hip ----
#define RI_SCORE_TILE 256          // centroids per softmax partial
int ri_launch_score(const void* q, const void* centroids, float* logits, float* tile_max, float* tile_sum,
                    int BG, int gs, int nc, float scale, bool half, hipStream_t s);

// Row statistics from the per-256-column partials [ntiles, gs]: one wave per row, lanes over
// tiles, xor-butterfly reductions (fixed order, so the result is reproducible).
__device__ __forceinline__ void ri_wave_reduce_partials(const float* pm, const float* ps, int ntiles, int gs,
                                                        int j, int lane, float* m_out, float* invz_out) {
  // the first 64 tiles' partials are loaded together, ahead of the reductions
  const bool has0 = lane < ntiles;
  const float pm0 = has0 ? pm[(size_t)lane * gs + j] : -INFINITY;
  const float ps0 = has0 ? ps[(size_t)lane * gs + j] : 0.f;
  float m = pm0;
  for (int t = lane + 64; t < ntiles; t += 64) m = fmaxf(m, pm[(size_t)t * gs + j]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  float z = has0 ? ps0 * __expf(pm0 - m) : 0.f;
  for (int t = lane + 64; t < ntiles; t += 64) z += ps[(size_t)t * gs + j] * __expf(pm[(size_t)t * gs + j] - m);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) z += __shfl_xor(z, o);
  *m_out = m;
  *invz_out = 1.0f / z;
}

// Inclusive prefix sum over the 64 lanes of a wave with DPP row shifts and row broadcasts
// (no LDS traffic): shifts by 1, 2, 3 build sums of four neighbours, shifts by 4 and 8 finish the
// 16-lane rows, the two broadcasts carry row totals into the rows behind.
__device__ __forceinline__ uint32_t ri_wave_incl_scan(uint32_t v) {
  uint32_t r = v;
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);   // row_shr:1
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);   // row_shr:2
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x113, 0xf, 0xf, true);   // row_shr:3
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)r, 0x114, 0xf, 0xe, false);  // row_shr:4, banks 1-3
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)r, 0x118, 0xf, 0xc, false);  // row_shr:8, banks 2-3
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)r, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1, 3
  r += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)r, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2, 3
  return r;
}

