// Device code shared by the attention kernels (gfx950): the per-wave online-softmax state, the
// update for one chunk of 16 rows (softmax bookkeeping, P·V on the matrix cores) and the coherent load
// of split partials.
#pragma once
#include "ri_common.h"

// Softmax bookkeeping is spread over the four 16-lane groups of a wave: group h keeps
// NH = GS_PAD/4 heads (the MFMA hands every group four heads; with GS_PAD = 4 all groups see the
// same four, so each keeps one).  ri_head_reg(h) is the first accumulator register group h keeps,
// ri_head_of(h, i) the head held in kept slot i.
template <int GS_PAD>
__device__ __forceinline__ int ri_head_reg(int h) {
  return GS_PAD == 4 ? h : (GS_PAD == 8 ? (h >> 1) * 2 : 0);
}
template <int GS_PAD>
__device__ __forceinline__ int ri_head_of(int h, int i) {
  return (4 * h + ri_head_reg<GS_PAD>(h) + i) % GS_PAD;
}

typedef short bf16x4s_t __attribute__((ext_vector_type(4)));

#define ATT_VT_STRIDE 144  // LDS row stride of the 16 x 128 value tile in bf16 elements (288 bytes)

template <int GS_PAD>
struct WaveState {
  float m[GS_PAD / 4];
  float l[GS_PAD / 4];
  // P·V accumulators in MFMA 16x16 layout: acc[dt][i] of lane l = head 4*(l/16)+i, dim 16*dt + l%16
  f32x4_t acc[8];
};

// probability -> the 16-bit element type of the P.V operands (hardware conversion, round to nearest even)
template <bool HALF>
__device__ __forceinline__ uint16_t ri_p_to_e16(float x) {
  if (HALF) return __builtin_bit_cast(uint16_t, (_Float16)x);
  const __bf16 b = (__bf16)x;
  return __builtin_bit_cast(uint16_t, b);
}

// One chunk of 16 rows.
//   sv[NH]  scores of the heads this lane keeps for row n = lane%16 (lane group h = lane/16)
//   v[4]    value rows h, h+4, h+8, h+12 of the chunk, dims 8n..8n+7 (as loaded from memory)
// Softmax bookkeeping in fp32 per lane; P goes to LDS as bf16 [head][row], the value tile to LDS
// row-major; P·V = 8 MFMA 16x16x16 whose B operands come from LDS transpose reads
// (ds_read_b64_tr_b16: lane l of a 16-lane group receives element l%4 of the 8-byte pieces
// addressed by lanes l/4, l/4+4, l/4+8, l/4+12 — four consecutive rows of one column).
template <int GS_PAD, bool HALF>
__device__ __forceinline__ void chunk_update(WaveState<GS_PAD>& st, const float* sv, bool valid, float w,
                                             const uint4 v[4], uint16_t* vt, uint16_t* pb, float* al_sh,
                                             int lane) {
  constexpr int NH = GS_PAD / 4;
  const int n = lane & 15, h = lane >> 4;
  // value tile -> LDS
#pragma unroll
  for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(vt + (h + 4 * i) * ATT_VT_STRIDE + 8 * n) = v[i];
  float al[NH];
  bool rescale = false;
#pragma unroll
  for (int i = 0; i < NH; ++i) {
    const float s = valid ? sv[i] : -INFINITY;
    float cm = s;
    cm = fmaxf(cm, __shfl_xor(cm, 1));
    cm = fmaxf(cm, __shfl_xor(cm, 2));
    cm = fmaxf(cm, __shfl_xor(cm, 4));
    cm = fmaxf(cm, __shfl_xor(cm, 8));
    const float mn = fmaxf(st.m[i], cm);
    float p;
    if (mn == -INFINITY) {
      al[i] = 1.f;
      p = 0.f;
    } else {
      al[i] = __expf(st.m[i] - mn);  // exp(-inf) = 0 for the first chunk
      p = valid ? __expf(s - mn) : 0.f;
    }
    rescale |= (al[i] != 1.f);
    st.l[i] = st.l[i] * al[i] + w * p;
    st.m[i] = mn;
    pb[ri_head_of<GS_PAD>(h, i) * 16 + n] = ri_p_to_e16<HALF>(p);
  }
  // the running maximum rarely moves after the first chunks: rescale only when some head's did
  const bool any_rescale = __any(rescale);
  if (any_rescale && n == 0) {
#pragma unroll
    for (int i = 0; i < NH; ++i) al_sh[ri_head_of<GS_PAD>(h, i)] = al[i];
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (any_rescale) {
    const float4 a4 = *reinterpret_cast<const float4*>(al_sh + 4 * h);
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      st.acc[dt][0] *= a4.x; st.acc[dt][1] *= a4.y; st.acc[dt][2] *= a4.z; st.acc[dt][3] *= a4.w;
    }
  }
  // A operand: P[head n][rows 4h..4h+3]
  const bf16x4s_t pa = *reinterpret_cast<const bf16x4s_t*>(pb + n * 16 + 4 * h);
  const uint16_t* vsrc = vt + (4 * h + (n >> 2)) * ATT_VT_STRIDE + 4 * (n & 3);
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) {
    const bf16x4s_t vb = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (bf16x4s_t __attribute__((address_space(3)))*)(vsrc + 16 * dt));
    if (HALF)
      st.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, pa), __builtin_bit_cast(f16x4_t, vb),
                                                         st.acc[dt], 0, 0, 0);
    else
      st.acc[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa, vb, st.acc[dt], 0, 0, 0);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();  // the tile and P are rewritten by the next chunk
}

// The partials were written by other workgroups of the same launch; they are read with
// device-scope loads (which go past this compute unit's non-coherent cache lines) instead of
// an acquire fence that would drop the whole cache.
__device__ __forceinline__ float2 ri_ld_partial(const float* p) {
  const uint64_t v = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
  return make_float2(__uint_as_float((uint32_t)v), __uint_as_float((uint32_t)(v >> 32)));
}

