// Weighted flash decoding for the wave index (gfx950).
//
// One kernel serves every attention call of the decode step.  A workgroup (4 waves) takes
// one split of one group's rows; a wave owns a contiguous run of rows and walks it in batches
// of 64 rows = 4 chunks of 16.  For a batch it first fetches one row descriptor per lane
// (where the row lives), then issues every K and V load of the batch before it computes, so
// that a short kernel keeps enough bytes in flight to load HBM:
//   * key/value rows ("KV" splits): scores = scale * q·k on bf16 MFMA 16x16x32 with the
//     query heads as the A rows and 16 key rows as the B columns, so each lane ends up with
//     the scores of one key row for four heads;
//   * estimation rows ("EST" splits): the score of a cluster is the logit already computed
//     by the scoring kernel, the "value" row is the cluster's value sum and the softmax
//     denominator is weighted by the cluster size.
// P·V runs on the vector ALU in fp32: lane (c, h) accumulates dims 8c..8c+7 over rows
// h, h+4, h+8, h+12 of each chunk, for all heads.  Every workgroup writes a
// (max, denominator, numerator) partial; the workgroup that finishes last for a group merges
// the partials (and an optional previous result) with the log-sum-exp rule and writes the
// output, so the whole call is one launch.
//
// Semantics follow the weighted_flash_decoding call sites at
// cache_hub/retroinfer_cache.py:611-617 and :666-674.
#include <stdlib.h>

#include "ri_common.h"

#define ATT_FLAG_A 0x40000000  // descriptor bit: row lives in region A

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
  const int32_t* est_ids;     // [BG, es]
  const float* logits;        // [BG, gs, nc]
  const uint16_t* value_sum;  // [BG, nc, 128]
  const uint16_t* csize;      // [BG, nc] bf16
  int nc;
  int es;
  // partials and the per-group arrival counters (zero between launches)
  float* part_ml;   // [BG, S, GS_PAD, 2]
  float* part_acc;  // [BG, S, GS_PAD, 128]
  int* counters;    // [BG]
  int S_kv;
  int S_es;
  int gs;
  int fuse;  // 1: the last workgroup of a group merges; 0: a separate combine launch does
  float scale;
  // epilogue
  const uint16_t* prev_out;  // [BG, gs, 128] or null
  const float* prev_lse;     // [BG, gs] or null
  uint16_t* out;             // [BG, gs, 128]
  float* lse_out;            // [BG, gs] or null
  int32_t* valid_lengths;    // [BG] or null: lenA + lenB(g)
};

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

template <int GS_PAD>
struct WaveState {
  float m[GS_PAD / 4];
  float l[GS_PAD / 4];
  float acc[GS_PAD][8];
};

// softmax update for one chunk: scores s_in[4] (this lane: row n = lane%16, MFMA registers of
// lane group h = lane/16), validity and denominator weight; then the P·V accumulation of the
// four value rows v[4] this lane owns.  p_sh: [16][GS_PAD] floats, al_sh: [GS_PAD] floats of this wave.
template <int GS_PAD>
__device__ __forceinline__ void chunk_update(WaveState<GS_PAD>& st, const float s_in[4], bool valid, float w,
                                             const uint4 v[4], float* p_sh, float* al_sh, int lane) {
  constexpr int NH = GS_PAD / 4;
  const int n = lane & 15, h = lane >> 4;
  const int r0 = ri_head_reg<GS_PAD>(h);
  float al[NH];
  bool rescale = false;
#pragma unroll
  for (int i = 0; i < NH; ++i) {
    float sv;
    if (GS_PAD == 16) {
      sv = s_in[i];
    } else {  // pick register r0 + i without dynamic indexing
      const int r = r0 + i;
      sv = r == 0 ? s_in[0] : (r == 1 ? s_in[1] : (r == 2 ? s_in[2] : s_in[3]));
    }
    const float s = valid ? sv : -INFINITY;
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
    p_sh[n * GS_PAD + ri_head_of<GS_PAD>(h, i)] = p;
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
#pragma unroll
    for (int j = 0; j < GS_PAD; j += 4) {
      const float4 a4 = *reinterpret_cast<const float4*>(al_sh + j);
      const float alpha[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
      for (int jj = 0; jj < 4; ++jj)
#pragma unroll
        for (int e = 0; e < 8; ++e) st.acc[j + jj][e] *= alpha[jj];
    }
  }
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

// rows of a wave: the group's `total` rows are cut into `nwaves` runs of a multiple of 16 rows
__device__ __forceinline__ void wave_rows(int total, int nwaves, int wid, int* r0, int* r1) {
  int rpw = (total + nwaves - 1) / nwaves;
  rpw = (rpw + 15) & ~15;
  *r0 = min(total, wid * rpw);
  *r1 = min(total, *r0 + rpw);
}

// Merges the S split partials of group g (and the optional previous result) and writes the
// output; called by all 256 threads of one workgroup.
template <bool COHERENT>
__device__ __forceinline__ float ld_part(const float* p) {
  return COHERENT ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *p;
}

template <int GS_PAD, bool COHERENT>
__device__ __forceinline__ void combine_group(const AttendParams& P, int g, int S, int lenB) {
  const int gs = P.gs;
  for (int idx = threadIdx.x; idx < gs * (RI_DIM / 2); idx += 256) {
    const int j = idx / (RI_DIM / 2), d2 = (idx % (RI_DIM / 2)) * 2;
    const float* ml = P.part_ml + ((size_t)g * S * GS_PAD + j) * 2;
    const float* pa = P.part_acc + ((size_t)g * S * GS_PAD + j) * RI_DIM + d2;
    float M = P.prev_lse ? P.prev_lse[(size_t)g * gs + j] : -INFINITY;
#pragma unroll 8
    for (int s = 0; s < S; ++s) M = fmaxf(M, ld_part<COHERENT>(ml + (size_t)s * GS_PAD * 2));
    float L = 0.f, A0 = 0.f, A1 = 0.f;
    if (P.prev_lse) {
      const float pl = P.prev_lse[(size_t)g * gs + j];
      const float f = (pl == -INFINITY) ? 0.f : __expf(pl - M);
      const uint32_t po = *reinterpret_cast<const uint32_t*>(P.prev_out + ((size_t)g * gs + j) * RI_DIM + d2);
      L = f;
      A0 = f * __uint_as_float(po << 16);
      A1 = f * __uint_as_float(po & 0xffff0000u);
    }
#pragma unroll 8
    for (int s = 0; s < S; ++s) {
      const float m = ld_part<COHERENT>(ml + (size_t)s * GS_PAD * 2);
      const float f = (m == -INFINITY) ? 0.f : __expf(m - M);
      const float a0 = ld_part<COHERENT>(pa + (size_t)s * GS_PAD * RI_DIM);
      const float a1 = ld_part<COHERENT>(pa + (size_t)s * GS_PAD * RI_DIM + 1);
      L += ld_part<COHERENT>(ml + (size_t)s * GS_PAD * 2 + 1) * f;
      A0 += a0 * f;
      A1 += a1 * f;
    }
    const uint32_t o = (uint32_t)ri_f32_to_bf16(A0 / L) | ((uint32_t)ri_f32_to_bf16(A1 / L) << 16);
    *reinterpret_cast<uint32_t*>(P.out + ((size_t)g * gs + j) * RI_DIM + d2) = o;
    if (d2 == 0 && P.lse_out) P.lse_out[(size_t)g * gs + j] = M + __logf(L);
  }
  if (threadIdx.x == 0 && P.valid_lengths) P.valid_lengths[g] = P.lenA + lenB;
}

// CH = chunks (of 16 rows) a wave loads ahead of computing
template <int GS_PAD, int CH>
__global__ __launch_bounds__(256, 2) void attend_kernel(AttendParams P) {
  __shared__ float sh_p[4][16 * GS_PAD];
  __shared__ float sh_al[4][GS_PAD];
  __shared__ float sh_m[4][GS_PAD];
  __shared__ float sh_l[4][GS_PAD];
  __shared__ float sh_acc[4][GS_PAD][RI_DIM];
  __shared__ __attribute__((aligned(16))) uint16_t sh_q[GS_PAD][RI_DIM];
  __shared__ int sh_last;

  const int g = blockIdx.y;
  const int split = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n = lane & 15, h = lane >> 4;
  const int gs = P.gs;
  constexpr int ND = (CH * 16 + 63) / 64;  // descriptor registers per batch

  WaveState<GS_PAD> st;
#pragma unroll
  for (int i = 0; i < GS_PAD / 4; ++i) { st.m[i] = -INFINITY; st.l[i] = 0.f; }
#pragma unroll
  for (int j = 0; j < GS_PAD; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) st.acc[j][e] = 0.f;

  float* p_sh = sh_p[wave];
  float* al_sh = sh_al[wave];
  const int lenB = P.lenB_ptr ? P.lenB_ptr[(size_t)g * P.lenB_ptr_stride] : P.lenB_const;

  if (split < P.S_kv) {
    // ---------------- key/value rows ----------------
    const int total = P.lenA + lenB;
    int r0, r1;
    wave_rows(total, P.S_kv * 4, split * 4 + wave, &r0, &r1);

    // A operand: query heads through LDS (read again per chunk: registers go to the loads);
    // row m of the MFMA holds head m % GS_PAD, zero if >= gs
    for (int i = threadIdx.x; i < GS_PAD * (RI_DIM / 8); i += 256) {
      const int head = i / (RI_DIM / 8), piece = i % (RI_DIM / 8);
      *reinterpret_cast<uint4*>(&sh_q[head][piece * 8]) =
          (head < gs) ? ri_ld16(P.q + ((size_t)g * gs + head) * RI_DIM + piece * 8) : ri_zero16();
    }
    __syncthreads();
    const uint16_t* qrow = &sh_q[n % GS_PAD][h * 8];
    const uint16_t* kA = P.kA + (size_t)g * P.strideA * RI_DIM;
    const uint16_t* vA = P.vA + (size_t)g * P.strideA * RI_DIM;
    const uint16_t* kB = P.kB + (size_t)g * P.strideB * RI_DIM;
    const uint16_t* vB = P.vB + (size_t)g * P.strideB * RI_DIM;
    const int32_t* rs = P.row_src ? P.row_src + (size_t)g * P.rs_stride : nullptr;
    const uint16_t* wB = P.weightB ? P.weightB + (size_t)g * P.weight_stride : nullptr;

    for (int b0 = r0; b0 < r1; b0 += 16 * CH) {
      // descriptors, one row per lane and register: where row b0 + 64*k + lane lives (-1 = past the end)
      int desc[ND];
      float wd[ND];
#pragma unroll
      for (int k = 0; k < ND; ++k) {
        desc[k] = -1;
        wd[k] = 1.f;
        const int row = b0 + 64 * k + lane;
        if (row < r1 && 64 * k + lane < 16 * CH) {
          if (row < P.lenA) {
            desc[k] = row | ATT_FLAG_A;
          } else {
            const int rb = row - P.lenA;
            desc[k] = rs ? rs[rb] : rb;
            if (wB) wd[k] = ri_bf16_to_f32(wB[rb]);
          }
        }
      }
      const int nch = min(CH, (r1 - b0 + 15) >> 4);
      uint4 bk[CH][4], v[CH][4];
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        if (ch < nch) {
          const int dk = __shfl(desc[ch / 4], (ch % 4) * 16 + n);
          const uint16_t* kp = ((dk & ATT_FLAG_A) ? kA : kB) + (size_t)(dk & ~ATT_FLAG_A) * RI_DIM + h * 8;
#pragma unroll
          for (int kk = 0; kk < 4; ++kk) bk[ch][kk] = (dk >= 0) ? ri_ld16(kp + kk * 32) : ri_zero16();
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int dv = __shfl(desc[ch / 4], (ch % 4) * 16 + h + 4 * i);
            const uint16_t* vp = ((dv & ATT_FLAG_A) ? vA : vB) + (size_t)(dv & ~ATT_FLAG_A) * RI_DIM + n * 8;
            v[ch][i] = (dv >= 0) ? ri_ld16(vp) : ri_zero16();
          }
        }
      }
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        if (ch < nch) {
          f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kk = 0; kk < 4; ++kk)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                ri_as_bf16x8(*reinterpret_cast<const uint4*>(qrow + kk * 32)), ri_as_bf16x8(bk[ch][kk]), acc, 0, 0, 0);
          const float s[4] = {acc[0] * P.scale, acc[1] * P.scale, acc[2] * P.scale, acc[3] * P.scale};
          const bool valid = __shfl(desc[ch / 4], (ch % 4) * 16 + n) >= 0;
          const float w = __shfl(wd[ch / 4], (ch % 4) * 16 + n);
          chunk_update<GS_PAD>(st, s, valid, w, v[ch], p_sh, al_sh, lane);
        }
      }
    }
  } else {
    // ---------------- estimation rows ----------------
    const int es = P.es;
    int r0, r1;
    wave_rows(es, P.S_es * 4, (split - P.S_kv) * 4 + wave, &r0, &r1);
    const int32_t* ids = P.est_ids + (size_t)g * es;
    const uint16_t* vs = P.value_sum + (size_t)g * P.nc * RI_DIM;
    const uint16_t* cs = P.csize + (size_t)g * P.nc;
    const float* lg = P.logits + (size_t)g * gs * P.nc;

    for (int b0 = r0; b0 < r1; b0 += 16 * CH) {
      int cid[ND];
      float wd[ND];
#pragma unroll
      for (int k = 0; k < ND; ++k) {
        cid[k] = -1;
        wd[k] = 0.f;
        const int row = b0 + 64 * k + lane;
        if (row < r1 && 64 * k + lane < 16 * CH) {
          cid[k] = ids[row];
          wd[k] = ri_bf16_to_f32(cs[cid[k]]);
        }
      }
      const int nch = min(CH, (r1 - b0 + 15) >> 4);
      float sc[CH][4];
      uint4 v[CH][4];
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        if (ch < nch) {
          const int ck = __shfl(cid[ch / 4], (ch % 4) * 16 + n);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int head = (4 * h + i) % GS_PAD;
            sc[ch][i] = (ck >= 0 && head < gs) ? lg[(size_t)head * P.nc + ck] : -INFINITY;
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int cv = __shfl(cid[ch / 4], (ch % 4) * 16 + h + 4 * i);
            v[ch][i] = (cv >= 0) ? ri_ld16(vs + (size_t)cv * RI_DIM + n * 8) : ri_zero16();
          }
        }
      }
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        if (ch < nch) {
          const bool valid = __shfl(cid[ch / 4], (ch % 4) * 16 + n) >= 0;
          const float w = __shfl(wd[ch / 4], (ch % 4) * 16 + n);
          chunk_update<GS_PAD>(st, sc[ch], valid, w, v[ch], p_sh, al_sh, lane);
        }
      }
    }
  }

  // ---------------- wave partial -> LDS ----------------
#pragma unroll
  for (int i = 0; i < GS_PAD / 4; ++i) {
    float l = st.l[i];
    l += __shfl_xor(l, 1);
    l += __shfl_xor(l, 2);
    l += __shfl_xor(l, 4);
    l += __shfl_xor(l, 8);
    if (n == 0) {
      sh_m[wave][ri_head_of<GS_PAD>(h, i)] = st.m[i];
      sh_l[wave][ri_head_of<GS_PAD>(h, i)] = l;
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
    if (P.fuse) {  // device-coherent stores: another workgroup of this launch reads them
      __hip_atomic_store(&P.part_acc[o * RI_DIM + d], a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (d == 0) {
        __hip_atomic_store(&P.part_ml[o * 2], M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&P.part_ml[o * 2 + 1], l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    } else {
      P.part_acc[o * RI_DIM + d] = a;
      if (d == 0) {
        P.part_ml[o * 2] = M;
        P.part_ml[o * 2 + 1] = l;
      }
    }
  }

  // ---------------- last workgroup of the group merges all splits ----------------
  if (!P.fuse) return;
  // The partial went out with device-coherent stores; once they have completed (the barrier
  // waits for this workgroup's outstanding stores) the arrival is announced.  The last
  // workgroup to arrive reads every partial with device-coherent loads.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (threadIdx.x == 0)
    sh_last = (__hip_atomic_fetch_add(&P.counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == S - 1);
  __syncthreads();
  if (!sh_last) return;
  combine_group<GS_PAD, true>(P, g, S, lenB);
  if (threadIdx.x == 0) P.counters[g] = 0;  // ready for the next launch
}

// separate merge pass: grid (gs, BG), one wave per (group, head); lanes first cover the
// splits (statistics), then the dims (two each)
template <int GS_PAD>
__global__ __launch_bounds__(64) void combine_kernel(AttendParams P) {
  const int j = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int S = P.S_kv + P.S_es, gs = P.gs;
  const float* ml = P.part_ml + ((size_t)g * S * GS_PAD + j) * 2;
  const float* pa = P.part_acc + ((size_t)g * S * GS_PAD + j) * RI_DIM + 2 * lane;
  float2 ms = make_float2(-INFINITY, 0.f);
  if (lane < S) ms = *reinterpret_cast<const float2*>(ml + (size_t)lane * GS_PAD * 2);
  const float pl = P.prev_lse ? P.prev_lse[(size_t)g * gs + j] : -INFINITY;
  float M = fmaxf(ms.x, pl);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  const float f = (ms.x == -INFINITY) ? 0.f : __expf(ms.x - M);
  float L = ms.y * f;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) L += __shfl_xor(L, o);
  float A0 = 0.f, A1 = 0.f;
  if (P.prev_lse) {
    const float fp = (pl == -INFINITY) ? 0.f : __expf(pl - M);
    const uint32_t po = *reinterpret_cast<const uint32_t*>(P.prev_out + ((size_t)g * gs + j) * RI_DIM + 2 * lane);
    L += fp;
    A0 = fp * __uint_as_float(po << 16);
    A1 = fp * __uint_as_float(po & 0xffff0000u);
  }
#pragma unroll 8
  for (int s = 0; s < S; ++s) {
    const float fs = __shfl(f, s);
    const float2 a2 = *reinterpret_cast<const float2*>(pa + (size_t)s * GS_PAD * RI_DIM);
    A0 += a2.x * fs;
    A1 += a2.y * fs;
  }
  const uint32_t o = (uint32_t)ri_f32_to_bf16(A0 / L) | ((uint32_t)ri_f32_to_bf16(A1 / L) << 16);
  *reinterpret_cast<uint32_t*>(P.out + ((size_t)g * gs + j) * RI_DIM + 2 * lane) = o;
  if (lane == 0) {
    if (P.lse_out) P.lse_out[(size_t)g * gs + j] = M + __logf(L);
    if (P.valid_lengths && j == 0) {
      const int lenB = P.lenB_ptr ? P.lenB_ptr[(size_t)g * P.lenB_ptr_stride] : P.lenB_const;
      P.valid_lengths[g] = P.lenA + lenB;
    }
  }
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
#define RI_MAX_SPLITS 64
#define RI_MAX_GROUPS 4096  // size of the counter area at the head of the workspace

static inline int gs_pad_of(int gs) { return gs <= 4 ? 4 : (gs <= 8 ? 8 : 16); }

static size_t attn_workspace_bytes(int BG, int gs) {
  if (BG <= 0 || BG > RI_MAX_GROUPS || gs <= 0 || gs > 16) return 0;
  const size_t per = (size_t)BG * RI_MAX_SPLITS * gs_pad_of(gs);
  return RI_MAX_GROUPS * sizeof(int) + per * (2 + RI_DIM) * sizeof(float);
}

extern "C" size_t ri_flash_decoding_workspace_bytes(int BG, int gs) { return attn_workspace_bytes(BG, gs); }
extern "C" size_t ri_wave_attention_workspace_bytes(int BG, int gs) { return attn_workspace_bytes(BG, gs); }

static void carve_workspace(AttendParams& P, void* workspace, int BG, int gp) {
  P.counters = (int*)workspace;
  P.part_ml = (float*)((char*)workspace + RI_MAX_GROUPS * sizeof(int));
  P.part_acc = P.part_ml + (size_t)BG * RI_MAX_SPLITS * gp * 2;
}

static int fuse_default() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("RI_ATTN_FUSE");
    v = e ? atoi(e) : 1;
  }
  return v;
}

static int launch_attend(AttendParams& P, int BG, int gs, hipStream_t s) {
  const int S = P.S_kv + P.S_es;
  const dim3 grid(S, BG);
  P.fuse = fuse_default();
  switch (gs_pad_of(gs)) {
    case 4: attend_kernel<4, 5><<<grid, 256, 0, s>>>(P); break;
    case 8: attend_kernel<8, 4><<<grid, 256, 0, s>>>(P); break;
    default: attend_kernel<16, 2><<<grid, 256, 0, s>>>(P); break;
  }
  RI_HIP_CHECK_LAUNCH();
  if (!P.fuse) {
    switch (gs_pad_of(gs)) {
      case 4: combine_kernel<4><<<dim3(gs, BG), 64, 0, s>>>(P); break;
      case 8: combine_kernel<8><<<dim3(gs, BG), 64, 0, s>>>(P); break;
      default: combine_kernel<16><<<dim3(gs, BG), 64, 0, s>>>(P); break;
    }
    RI_HIP_CHECK_LAUNCH();
  }
  return RI_OK;
}

static inline int chunks_ahead(int gs) { return gs <= 4 ? 5 : (gs <= 8 ? 4 : 2); }

// splits so that a wave sees about one batch of rows, within [1, cap]
static int pick_splits(int64_t rows, int BG, int cap, int gs) {
  const int rows_per_wave = 16 * chunks_ahead(gs);
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
  if (BG <= 0 || BG > RI_MAX_GROUPS || gs <= 0 || gs > 16 || S < 0 || kv_stride < S) return RI_ERR_ARG;
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
  P.S_kv = pick_splits(S, BG, RI_MAX_SPLITS, gs);
  P.S_es = 0;
  P.gs = gs;
  P.scale = scale;
  P.prev_out = (const uint16_t*)prev_out;
  P.prev_lse = prev_lse;
  P.out = (uint16_t*)out;
  P.lse_out = lse_out;
  carve_workspace(P, workspace, BG, gp);
  return launch_attend(P, BG, gs, (hipStream_t)stream);
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
  if (BG <= 0 || BG > RI_MAX_GROUPS || gs <= 0 || gs > 16 || static_len < 0 || static_len > steady_stride ||
      es < 0 || nc <= 0)
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
  P.out = (uint16_t*)out;
  P.valid_lengths = valid_lengths;
  // the retrieved-token count is only known on the device: size the split for the row table
  // capacity scaled by the usual fill (a quarter), the estimation zone by its exact size
  const int cap_es = es > 0 ? RI_MAX_SPLITS / 2 : 0;
  P.S_es = es > 0 ? pick_splits(es, BG, cap_es, gs) : 0;
  P.S_kv = pick_splits(static_len + row_src_stride / 4, BG, RI_MAX_SPLITS - P.S_es, gs);
  carve_workspace(P, workspace, BG, gp);
  return launch_attend(P, BG, gs, (hipStream_t)stream);
}
