// Weighted flash decoding for the wave index (gfx950).
//
// One kernel serves every attention call of the decode step.  A workgroup (4 waves) takes
// one split of one group's rows; a wave walks its rows in chunks of 16:
//   * key/value rows ("KV" splits): scores = scale * q·k on bf16 MFMA 16x16x32 with the
//     query heads as the A rows and 16 key rows as the B columns, so each lane ends up with
//     the scores of one key row for four heads;
//   * estimation rows ("EST" splits): the score of a cluster is the logit already computed
//     by the scoring kernel, the "value" row is the cluster's value sum and the softmax
//     denominator is weighted by the cluster size.
// P·V runs on the vector ALU in fp32: lane (c, h) accumulates dims 8c..8c+7 over rows
// h, h+4, h+8, h+12 of each chunk, for all heads.  Splits write (max, denominator,
// numerator) partials; combine_kernel merges them (and an optional previous result) with the
// usual log-sum-exp rule.
//
// Semantics follow the weighted_flash_decoding call sites at
// cache_hub/retroinfer_cache.py:611-617 and :666-674.
#include "ri_common.h"

struct AttendParams {
  const uint16_t* q;  // [BG, gs, 128]
  // region A: rows [0, lenA) at kA/vA + (g*strideA + row)*128
  const uint16_t* kA;
  const uint16_t* vA;
  int64_t strideA;
  int lenA;
  // region B: rows [0, lenB(g)) at kB/vB + (g*strideB + src(row))*128,
  // src(row) = row_src ? row_src[g*rs_stride + row] : row
  const uint16_t* kB;
  const uint16_t* vB;
  int64_t strideB;
  const int32_t* row_src;
  int rs_stride;
  const int32_t* lenB_ptr;  // lenB(g) = lenB_ptr ? lenB_ptr[g*lenB_ptr_stride] : lenB_const
  int lenB_ptr_stride;
  int lenB_const;
  const uint16_t* weightB;  // [BG, weight_stride] bf16 per region-B row, or null
  int weight_stride;
  // estimation rows
  const int32_t* est_ids;  // [BG, es]
  const float* logits;     // [BG, gs, nc]
  const uint16_t* value_sum;  // [BG, nc, 128]
  const uint16_t* csize;      // [BG, nc] bf16
  int nc;
  int es;
  // partials
  float* part_ml;   // [BG, S, GS_PAD, 2]
  float* part_acc;  // [BG, S, GS_PAD, 128]
  int S_kv;
  int S_es;
  int gs;
  float scale;
};

template <int GS_PAD>
struct WaveState {
  float m[4];
  float l[4];
  float acc[GS_PAD][8];
};

// softmax update for one chunk: scores s[4] (this lane: row n = lane%16, heads 4*(lane/16)+i mod
// GS_PAD), validity and denominator weight; then the P·V accumulation of the four value rows
// v[4] this lane owns.  p_sh: [16][GS_PAD] floats, al_sh: [GS_PAD] floats of this wave.
template <int GS_PAD>
__device__ __forceinline__ void chunk_update(WaveState<GS_PAD>& st, const float s_in[4], bool valid, float w,
                                             const uint4 v[4], float* p_sh, float* al_sh, int lane) {
  const int n = lane & 15, h = lane >> 4;
  float p[4], al[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float s = valid ? s_in[i] : -INFINITY;
    float cm = s;
    cm = fmaxf(cm, __shfl_xor(cm, 1));
    cm = fmaxf(cm, __shfl_xor(cm, 2));
    cm = fmaxf(cm, __shfl_xor(cm, 4));
    cm = fmaxf(cm, __shfl_xor(cm, 8));
    const float mn = fmaxf(st.m[i], cm);
    if (mn == -INFINITY) {
      al[i] = 1.f;
      p[i] = 0.f;
    } else {
      al[i] = __expf(st.m[i] - mn);  // exp(-inf) = 0 for the first chunk
      p[i] = valid ? __expf(s - mn) : 0.f;
    }
    st.l[i] = st.l[i] * al[i] + w * p[i];
    st.m[i] = mn;
  }
  if (h < GS_PAD / 4) {
    *reinterpret_cast<float4*>(p_sh + n * GS_PAD + 4 * h) = make_float4(p[0], p[1], p[2], p[3]);
    if (n == 0) *reinterpret_cast<float4*>(al_sh + 4 * h) = make_float4(al[0], al[1], al[2], al[3]);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float alpha[GS_PAD];
#pragma unroll
  for (int j = 0; j < GS_PAD; j += 4) {
    const float4 a4 = *reinterpret_cast<const float4*>(al_sh + j);
    alpha[j] = a4.x; alpha[j + 1] = a4.y; alpha[j + 2] = a4.z; alpha[j + 3] = a4.w;
  }
#pragma unroll
  for (int j = 0; j < GS_PAD; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) st.acc[j][e] *= alpha[j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float vf[8];
    ri_unpack8(v[i], vf);
    const int row = h + 4 * i;
#pragma unroll
    for (int j = 0; j < GS_PAD; j += 4) {
      const float4 p4 = *reinterpret_cast<const float4*>(p_sh + row * GS_PAD + j);
      const float pj[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
#pragma unroll
        for (int e = 0; e < 8; ++e) st.acc[j + jj][e] = fmaf(pj[jj], vf[e], st.acc[j + jj][e]);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();  // p_sh is rewritten by the next chunk
}

template <int GS_PAD>
__global__ __launch_bounds__(256) void attend_kernel(AttendParams P) {
  __shared__ float sh_p[4][16 * GS_PAD];
  __shared__ float sh_al[4][GS_PAD];
  __shared__ float sh_m[4][GS_PAD];
  __shared__ float sh_l[4][GS_PAD];
  __shared__ float sh_acc[4][GS_PAD][RI_DIM];

  const int g = blockIdx.y;
  const int split = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n = lane & 15, h = lane >> 4;
  const int gs = P.gs;

  WaveState<GS_PAD> st;
#pragma unroll
  for (int i = 0; i < 4; ++i) { st.m[i] = -INFINITY; st.l[i] = 0.f; }
#pragma unroll
  for (int j = 0; j < GS_PAD; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) st.acc[j][e] = 0.f;

  float* p_sh = sh_p[wave];
  float* al_sh = sh_al[wave];

  if (split < P.S_kv) {
    // ---------------- key/value rows ----------------
    const int lenB = P.lenB_ptr ? P.lenB_ptr[(size_t)g * P.lenB_ptr_stride] : P.lenB_const;
    const int total = P.lenA + lenB;
    const int chunks = (total + 15) >> 4;
    const int nwaves = P.S_kv * 4;
    const int cpw = (chunks + nwaves - 1) / nwaves;
    const int wid = split * 4 + wave;
    const int cb = wid * cpw;
    const int ce = min(chunks, cb + cpw);

    // A operand: query heads; row m of the MFMA holds head m % GS_PAD (zero if >= gs)
    uint4 aq[4];
    {
      const int head = n % GS_PAD;
      const uint16_t* qp = P.q + ((size_t)g * gs + head) * RI_DIM + h * 8;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) aq[kk] = (head < gs) ? ri_ld16(qp + kk * 32) : ri_zero16();
    }
    const uint16_t* kA = P.kA + (size_t)g * P.strideA * RI_DIM;
    const uint16_t* vA = P.vA + (size_t)g * P.strideA * RI_DIM;
    const uint16_t* kB = P.kB + (size_t)g * P.strideB * RI_DIM;
    const uint16_t* vB = P.vB + (size_t)g * P.strideB * RI_DIM;
    const int32_t* rs = P.row_src ? P.row_src + (size_t)g * P.rs_stride : nullptr;
    const uint16_t* wB = P.weightB ? P.weightB + (size_t)g * P.weight_stride : nullptr;

    for (int c = cb; c < ce; ++c) {
      // key row of this lane
      const int row = c * 16 + n;
      const bool valid = row < total;
      const uint16_t* kp = nullptr;
      float w = 1.f;
      if (valid) {
        if (row < P.lenA) {
          kp = kA + (size_t)row * RI_DIM;
        } else {
          const int rb = row - P.lenA;
          const int src = rs ? rs[rb] : rb;
          kp = kB + (size_t)src * RI_DIM;
          if (wB) w = ri_bf16_to_f32(wB[rb]);
        }
      }
      uint4 bk[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) bk[kk] = valid ? ri_ld16(kp + kk * 32 + h * 8) : ri_zero16();
      // value rows of this lane: rows h, h+4, h+8, h+12 of the chunk, dims 8n..8n+7
      uint4 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int vr = c * 16 + h + 4 * i;
        if (vr < total) {
          const uint16_t* vp;
          if (vr < P.lenA) {
            vp = vA + (size_t)vr * RI_DIM;
          } else {
            const int rb = vr - P.lenA;
            vp = vB + (size_t)(rs ? rs[rb] : rb) * RI_DIM;
          }
          v[i] = ri_ld16(vp + n * 8);
        } else {
          v[i] = ri_zero16();
        }
      }
      f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ri_as_bf16x8(aq[kk]), ri_as_bf16x8(bk[kk]), acc, 0, 0, 0);
      const float s[4] = {acc[0] * P.scale, acc[1] * P.scale, acc[2] * P.scale, acc[3] * P.scale};
      chunk_update<GS_PAD>(st, s, valid, w, v, p_sh, al_sh, lane);
    }
  } else {
    // ---------------- estimation rows ----------------
    const int es = P.es;
    const int chunks = (es + 15) >> 4;
    const int nwaves = P.S_es * 4;
    const int cpw = (chunks + nwaves - 1) / nwaves;
    const int wid = (split - P.S_kv) * 4 + wave;
    const int cb = wid * cpw;
    const int ce = min(chunks, cb + cpw);
    const int32_t* ids = P.est_ids + (size_t)g * es;
    const uint16_t* vs = P.value_sum + (size_t)g * P.nc * RI_DIM;
    const uint16_t* cs = P.csize + (size_t)g * P.nc;

    for (int c = cb; c < ce; ++c) {
      const int row = c * 16 + n;
      const bool valid = row < es;
      float s[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      float w = 0.f;
      if (valid) {
        const int cid = ids[row];
        w = ri_bf16_to_f32(cs[cid]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int head = (4 * h + i) % GS_PAD;
          if (head < gs) s[i] = P.logits[((size_t)g * gs + head) * P.nc + cid];
        }
      }
      uint4 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int vr = c * 16 + h + 4 * i;
        v[i] = (vr < es) ? ri_ld16(vs + (size_t)ids[vr] * RI_DIM + n * 8) : ri_zero16();
      }
      chunk_update<GS_PAD>(st, s, valid, w, v, p_sh, al_sh, lane);
    }
  }

  // ---------------- wave partial -> LDS ----------------
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float l = st.l[i];
    l += __shfl_xor(l, 1);
    l += __shfl_xor(l, 2);
    l += __shfl_xor(l, 4);
    l += __shfl_xor(l, 8);
    st.l[i] = l;
  }
  if (n == 0 && h < GS_PAD / 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sh_m[wave][4 * h + i] = st.m[i];
      sh_l[wave][4 * h + i] = st.l[i];
    }
  }
#pragma unroll
  for (int j = 0; j < GS_PAD; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = st.acc[j][e];
      a += __shfl_xor(a, 16);
      a += __shfl_xor(a, 32);
      st.acc[j][e] = a;
    }
  if (h == 0) {
#pragma unroll
    for (int j = 0; j < GS_PAD; ++j) {
      float4* dst = reinterpret_cast<float4*>(&sh_acc[wave][j][n * 8]);
      dst[0] = make_float4(st.acc[j][0], st.acc[j][1], st.acc[j][2], st.acc[j][3]);
      dst[1] = make_float4(st.acc[j][4], st.acc[j][5], st.acc[j][6], st.acc[j][7]);
    }
  }
  __syncthreads();

  // ---------------- merge the four waves, write the split partial ----------------
  const int S = P.S_kv + P.S_es;
  for (int idx = threadIdx.x; idx < GS_PAD * RI_DIM; idx += 256) {
    const int j = idx / RI_DIM, d = idx % RI_DIM;
    const float M = fmaxf(fmaxf(sh_m[0][j], sh_m[1][j]), fmaxf(sh_m[2][j], sh_m[3][j]));
    float a = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = (sh_m[w][j] == -INFINITY) ? 0.f : __expf(sh_m[w][j] - M);
      a += sh_acc[w][j][d] * f;
      l += sh_l[w][j] * f;
    }
    const size_t o = ((size_t)g * S + split) * GS_PAD + j;
    P.part_acc[o * RI_DIM + d] = a;
    if (d == 0) {
      P.part_ml[o * 2] = M;
      P.part_ml[o * 2 + 1] = l;
    }
  }
}

// combine: grid (gs, BG), 128 threads (one per dim)
__global__ __launch_bounds__(128) void combine_kernel(const float* __restrict__ part_ml,
                                                      const float* __restrict__ part_acc, int S, int gs_pad,
                                                      const uint16_t* __restrict__ prev_out,
                                                      const float* __restrict__ prev_lse,
                                                      uint16_t* __restrict__ out, float* __restrict__ lse_out,
                                                      int gs, const int32_t* __restrict__ lenB_ptr,
                                                      int lenB_ptr_stride, int lenA,
                                                      int32_t* __restrict__ valid_lengths) {
  const int j = blockIdx.x, g = blockIdx.y, d = threadIdx.x;
  float M = -INFINITY;
  if (prev_lse) M = prev_lse[(size_t)g * gs + j];
  for (int s = 0; s < S; ++s) M = fmaxf(M, part_ml[(((size_t)g * S + s) * gs_pad + j) * 2]);
  float L = 0.f, A = 0.f;
  if (prev_lse) {
    const float pl = prev_lse[(size_t)g * gs + j];
    const float f = (pl == -INFINITY) ? 0.f : __expf(pl - M);
    L = f;
    A = f * ri_bf16_to_f32(prev_out[((size_t)g * gs + j) * RI_DIM + d]);
  }
  for (int s = 0; s < S; ++s) {
    const size_t o = ((size_t)g * S + s) * gs_pad + j;
    const float m = part_ml[o * 2];
    const float f = (m == -INFINITY) ? 0.f : __expf(m - M);
    L += part_ml[o * 2 + 1] * f;
    A += part_acc[o * RI_DIM + d] * f;
  }
  out[((size_t)g * gs + j) * RI_DIM + d] = ri_f32_to_bf16(A / L);
  if (d == 0) {
    if (lse_out) lse_out[(size_t)g * gs + j] = M + __logf(L);
    if (valid_lengths && j == 0)
      valid_lengths[g] = lenA + (lenB_ptr ? lenB_ptr[(size_t)g * lenB_ptr_stride] : 0);
  }
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
#define RI_MAX_SPLITS 64

static inline int gs_pad_of(int gs) { return gs <= 4 ? 4 : (gs <= 8 ? 8 : 16); }

static size_t attn_workspace_bytes(int BG, int gs) {
  if (BG <= 0 || gs <= 0 || gs > 16) return 0;
  const size_t per = (size_t)BG * RI_MAX_SPLITS * gs_pad_of(gs);
  return per * (2 + RI_DIM) * sizeof(float);
}

extern "C" size_t ri_flash_decoding_workspace_bytes(int BG, int gs) { return attn_workspace_bytes(BG, gs); }
extern "C" size_t ri_wave_attention_workspace_bytes(int BG, int gs) { return attn_workspace_bytes(BG, gs); }

static int launch_attend(AttendParams& P, int BG, int gs, hipStream_t s) {
  const int S = P.S_kv + P.S_es;
  const dim3 grid(S, BG);
  switch (gs_pad_of(gs)) {
    case 4: attend_kernel<4><<<grid, 256, 0, s>>>(P); break;
    case 8: attend_kernel<8><<<grid, 256, 0, s>>>(P); break;
    default: attend_kernel<16><<<grid, 256, 0, s>>>(P); break;
  }
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

// splits so that a wave sees about `rows_per_wave` rows, within [1, cap]
static int pick_splits(int64_t rows, int BG, int cap) {
  const int rows_per_wave = 64;
  int64_t s = (rows + 4 * rows_per_wave - 1) / (4 * rows_per_wave);
  // do not launch far more workgroups than the chip can hold at once
  const int64_t max_by_chip = (4096 + BG - 1) / BG;
  if (s > max_by_chip) s = max_by_chip;
  if (s > cap) s = cap;
  if (s < 1) s = 1;
  return (int)s;
}

extern "C" int ri_weighted_flash_decoding(const void* q, const void* k, const void* v, const void* weight,
                                          const int32_t* cache_seqlens, const void* prev_out,
                                          const float* prev_lse, void* out, float* lse_out, int BG, int gs,
                                          int S, int64_t kv_stride, float scale, void* workspace,
                                          size_t workspace_bytes, ri_stream_t stream) {
  if (!q || !k || !v || !out || !workspace) return RI_ERR_ARG;
  if (BG <= 0 || gs <= 0 || gs > 16 || S < 0 || kv_stride < S) return RI_ERR_ARG;
  if ((prev_out == nullptr) != (prev_lse == nullptr)) return RI_ERR_ARG;
  if (workspace_bytes < attn_workspace_bytes(BG, gs)) return RI_ERR_WORKSPACE;
  const int gp = gs_pad_of(gs);
  AttendParams P = {};
  P.q = (const uint16_t*)q;
  P.kA = P.kB = (const uint16_t*)k;
  P.vA = P.vB = (const uint16_t*)v;
  P.strideA = P.strideB = kv_stride;
  P.lenA = 0;
  P.lenB_ptr = cache_seqlens;
  P.lenB_ptr_stride = 1;
  P.lenB_const = S;
  P.weightB = (const uint16_t*)weight;
  P.weight_stride = S;
  P.S_kv = pick_splits(S, BG, RI_MAX_SPLITS);
  P.S_es = 0;
  P.gs = gs;
  P.scale = scale;
  P.part_ml = (float*)workspace;
  P.part_acc = P.part_ml + (size_t)BG * RI_MAX_SPLITS * gp * 2;
  hipStream_t s = (hipStream_t)stream;
  int rc = launch_attend(P, BG, gs, s);
  if (rc) return rc;
  combine_kernel<<<dim3(gs, BG), 128, 0, s>>>(P.part_ml, P.part_acc, P.S_kv, gp, (const uint16_t*)prev_out,
                                              prev_lse, (uint16_t*)out, lse_out, gs, nullptr, 0, 0, nullptr);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" int ri_wave_attention(const void* q, const void* steady_k, const void* steady_v,
                                 int64_t steady_stride, int static_len, const void* store_k,
                                 const void* store_v, int64_t store_stride, const int32_t* row_src,
                                 int row_src_stride, const int32_t* meta, const int32_t* est_ids,
                                 const float* logits, const void* value_sum, const void* cluster_size_bf16,
                                 void* out, int32_t* valid_lengths, int BG, int gs, int nc, int es,
                                 float scale, void* workspace, size_t workspace_bytes, ri_stream_t stream) {
  if (!q || !steady_k || !steady_v || !store_k || !store_v || !row_src || !meta || !out || !workspace)
    return RI_ERR_ARG;
  if (BG <= 0 || gs <= 0 || gs > 16 || static_len < 0 || static_len > steady_stride || es < 0 || nc <= 0)
    return RI_ERR_ARG;
  if (es > 0 && (!est_ids || !logits || !value_sum || !cluster_size_bf16)) return RI_ERR_ARG;
  if (workspace_bytes < attn_workspace_bytes(BG, gs)) return RI_ERR_WORKSPACE;
  const int gp = gs_pad_of(gs);
  AttendParams P = {};
  P.q = (const uint16_t*)q;
  P.kA = (const uint16_t*)steady_k;
  P.vA = (const uint16_t*)steady_v;
  P.strideA = steady_stride;
  P.lenA = static_len;
  P.kB = (const uint16_t*)store_k;
  P.vB = (const uint16_t*)store_v;
  P.strideB = store_stride;
  P.row_src = row_src;
  P.rs_stride = row_src_stride;
  P.lenB_ptr = meta + 1;
  P.lenB_ptr_stride = 4;
  P.est_ids = est_ids;
  P.logits = logits;
  P.value_sum = (const uint16_t*)value_sum;
  P.csize = (const uint16_t*)cluster_size_bf16;
  P.nc = nc;
  P.es = es;
  P.gs = gs;
  P.scale = scale;
  // the retrieved-token count is only known on the device: size the split for the row table
  // capacity scaled by the usual fill (a quarter), the estimation zone by its exact size
  const int cap_es = es > 0 ? RI_MAX_SPLITS / 2 : 0;
  P.S_es = es > 0 ? pick_splits(es, BG, cap_es) : 0;
  P.S_kv = pick_splits(static_len + row_src_stride / 4, BG, RI_MAX_SPLITS - P.S_es);
  P.part_ml = (float*)workspace;
  P.part_acc = P.part_ml + (size_t)BG * RI_MAX_SPLITS * gp * 2;
  hipStream_t s = (hipStream_t)stream;
  int rc = launch_attend(P, BG, gs, s);
  if (rc) return rc;
  combine_kernel<<<dim3(gs, BG), 128, 0, s>>>(P.part_ml, P.part_acc, P.S_kv + P.S_es, gp, nullptr, nullptr,
                                              (uint16_t*)out, nullptr, gs, meta + 1, 4, static_len,
                                              valid_lengths);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
