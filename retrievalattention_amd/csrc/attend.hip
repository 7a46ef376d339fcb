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
// P·V runs on the matrix cores too: the chunk's probabilities go to LDS as bf16 [head][row], the 16 x 128
// value tile row-major, and eight MFMA 16x16x16 (B operands read with LDS transpose loads) add the chunk
// to fp32 accumulators that hold, per lane, four heads of one dimension per 16-wide tile.  Every
// workgroup writes a (max, denominator, numerator) partial; the workgroup that finishes last for a group
// merges the partials (and an optional previous result) with the log-sum-exp rule and writes the
// output, so the whole call is one launch.
//
// Semantics follow the weighted_flash_decoding call sites at
// cache_hub/retroinfer_cache.py:611-617 and :666-674.
#include <stdint.h>
#include <stdlib.h>

#include <mutex>

#include "attend_common.h"
#include "ri_common.h"

#define ATT_FLAG_A 0x40000000  // descriptor bit: row lives in region A

struct AttendParams {
  const uint16_t* q;  // [BG, gs, 128]
  // region A: rows [0, lenA) at kA/vA + (g*strideA + row)*128
  const uint16_t* kA;
  const uint16_t* vA;
  int64_t strideA;
  int lenA;
  const int32_t* lenA_ptr;  // when given: lenA is read here at launch time (clamped to [0, strideA])
  // region B: rows [0, lenB(g)) at kB/vB + (g*strideB + src(row))*128,
  // src(row) = row_src ? row_src[g*rs_stride + row] : row
  const uint16_t* kB;
  const uint16_t* vB;
  int64_t strideB;
  const int32_t* row_src;
  int rs_stride;
  // with a row table: only rows whose source row lies in [src_lo, src_hi) are attended, the others are
  // skipped like padding rows (a second launch takes them, merging this one's result as its previous one)
  int src_lo, src_hi;
  // or, without a row table: rank r of np clusters covers rows [ret_off[r], ret_off[r+1]) of region B,
  // stored contiguously from row ret_start[r] (ret_off has np + 1 entries, constant from the last kept rank on)
  const int32_t* ret_off;
  const int32_t* ret_start;
  int np;
  const int32_t* lenB_ptr;  // lenB(g) = lenB_ptr ? lenB_ptr[g*lenB_ptr_stride] : lenB_const
  int lenB_ptr_stride;
  int lenB_const;
  const uint16_t* weightB;  // [BG, weight_stride] bf16 per region-B row, or null
  int weight_stride;
  // estimation rows
  const int32_t* est_ids;     // [BG, es]
  const float* logits;        // [BG, gs, nc] scores of the estimation rows, or null:
  const uint16_t* est_cent;   // [BG, nc, 128] then the scores are computed here from the centroid rows
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
  float scale;
  // epilogue
  const uint16_t* prev_out;  // [BG, gs, 128] or null
  const float* prev_lse;     // [BG, gs] or null
  uint16_t* out;             // [BG, gs, 128]
  float* lse_out;            // [BG, gs] or null
  int32_t* valid_lengths;    // [BG] or null: lenA + lenB(g)
};

// rows of a wave: the group's `total` rows are cut into `nwaves` runs of a multiple of 16 rows
__device__ __forceinline__ void wave_rows(int total, int nwaves, int wid, int* r0, int* r1) {
  int rpw = (total + nwaves - 1) / nwaves;
  rpw = (rpw + 15) & ~15;
  *r0 = min(total, wid * rpw);
  *r1 = min(total, *r0 + rpw);
}

// Merges the S split partials of group g (and the optional previous result) and writes the
// output: wave w of the calling workgroup takes heads w, w+NW, ...; lanes first cover the splits
// (statistics), then two dims each.
template <int GS_PAD, int NW, bool HALF>
__device__ __forceinline__ void combine_group(const AttendParams& P, int g, int S, int lenA, int lenB) {
  const int gs = P.gs;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int j = wave; j < gs; j += NW) {
    const float* ml = P.part_ml + ((size_t)g * S * GS_PAD + j) * 2;
    const float* pa = P.part_acc + ((size_t)g * S * GS_PAD + j) * RI_DIM + 2 * lane;
    // every load of the merge is issued up front: the statistics (one split per lane) and the
    // first CB_PRE splits' numerators; their latencies overlap instead of adding up
    constexpr int CB_PRE = 24;
    float2 ms = make_float2(-INFINITY, 0.f);
    if (lane < S) ms = ri_ld_partial(ml + (size_t)lane * GS_PAD * 2);
    float2 a2[CB_PRE];
#pragma unroll
    for (int u = 0; u < CB_PRE; ++u)
      a2[u] = (u < S) ? ri_ld_partial(pa + (size_t)u * GS_PAD * RI_DIM) : make_float2(0.f, 0.f);
    const float pl = P.prev_lse ? P.prev_lse[(size_t)g * gs + j] : -INFINITY;
    uint32_t po = 0u;
    if (P.prev_lse) po = *reinterpret_cast<const uint32_t*>(P.prev_out + ((size_t)g * gs + j) * RI_DIM + 2 * lane);
    float M = fmaxf(ms.x, pl);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
    const float f = (ms.x == -INFINITY) ? 0.f : __expf(ms.x - M);
    float L = ms.y * f;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) L += __shfl_xor(L, o);
    float A0 = 0.f, A1 = 0.f;
    if (P.prev_lse && pl != -INFINITY) {  // an empty earlier part carries no weight, whatever its output holds
      const float fp = __expf(pl - M);
      float p0, p1;
      ri_unpack2<HALF>(po, p0, p1);
      L += fp;
      A0 = fp * p0;
      A1 = fp * p1;
    }
#pragma unroll
    for (int u = 0; u < CB_PRE; ++u) {
      const float fs = __shfl(f, u);
      A0 += a2[u].x * fs;
      A1 += a2[u].y * fs;
    }
    for (int s0 = CB_PRE; s0 < S; s0 += 8) {
      float2 b2[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        b2[u] = (s0 + u < S) ? ri_ld_partial(pa + (size_t)(s0 + u) * GS_PAD * RI_DIM)
                             : make_float2(0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float fs = __shfl(f, (s0 + u) & 63);
        A0 += b2[u].x * fs;
        A1 += b2[u].y * fs;
      }
    }
    // nothing attended at all (an empty part): zeros and a log-sum-exp of -inf, not 0/0
    const bool any = L > 0.f;
    const uint32_t o = (uint32_t)ri_f32_to_e16<HALF>(any ? A0 / L : 0.f) |
                       ((uint32_t)ri_f32_to_e16<HALF>(any ? A1 / L : 0.f) << 16);
    *reinterpret_cast<uint32_t*>(P.out + ((size_t)g * gs + j) * RI_DIM + 2 * lane) = o;
    if (lane == 0 && P.lse_out) P.lse_out[(size_t)g * gs + j] = M + __logf(L);
  }
  if (threadIdx.x == 0 && P.valid_lengths) P.valid_lengths[g] = lenA + lenB;
}

#define ATT_DESC_MAX 64  // rows of one wave whose descriptors are staged in LDS at a time (32 and 128 measured slower)

// PF = chunks (of 16 rows) in flight per wave: the loads of chunk j+PF are issued before chunk j
// is computed.  Launched with PF = 1: with eight to twelve waves per compute unit one chunk ahead already
// keeps the memory system busy, and the deeper pipelines only add registers and ramp (step time at 32 groups
// of 4 heads: 52.8 us with one chunk ahead, 53.4 with two, 56.0 with three).
//
// NW = waves per workgroup (4 or 8).  The waves of a workgroup merge in LDS, so a group split over S workgroups
// hands S partials to its last arriver whatever NW is: eight-wave workgroups halve the partials (and the
// arrivals) of a launch with the same number of waves per compute unit.
// The rank tables of the retrieval zone (np + 1 token offsets, np first rows) live in dynamic LDS, sized by
// the launch, so that any number of probes the selection accepts can be attended.
// HALF: q, K, V, value sums, cluster sizes, weights and outputs are IEEE half instead of bfloat16.
template <int GS_PAD, int NW, int PF, bool HALF>
__global__ __launch_bounds__(64 * NW, GS_PAD == 16 ? 1 : 3) void attend_kernel(AttendParams P) {
  constexpr int NH = GS_PAD / 4;
  constexpr int NT = 64 * NW;
  __shared__ __attribute__((aligned(16))) uint16_t sh_vt[NW][16 * ATT_VT_STRIDE];
  __shared__ __attribute__((aligned(16))) uint16_t sh_pb[NW][16 * 16];
  __shared__ float sh_al[NW][16];
  __shared__ float sh_m[NW][GS_PAD];
  __shared__ float sh_l[NW][GS_PAD];
  // the waves' numerators for the merge: up to eight heads they are laid over the wave's own value tile (dead
  // once its rows are done), which keeps a four-wave workgroup under 40 KB of LDS (four per compute unit)
  constexpr bool ACC_OVER_VT = GS_PAD * RI_DIM * sizeof(float) <= 16 * ATT_VT_STRIDE * sizeof(uint16_t);
  __shared__ float sh_acc_own[ACC_OVER_VT ? 1 : NW][ACC_OVER_VT ? 1 : GS_PAD][RI_DIM];
  auto acc_of = [&](int w) -> float* {
    return ACC_OVER_VT ? reinterpret_cast<float*>(sh_vt[w]) : &sh_acc_own[ACC_OVER_VT ? 0 : w][0][0];
  };
  __shared__ __attribute__((aligned(16))) uint16_t sh_q[GS_PAD][RI_DIM];
  __shared__ int sh_desc[NW][ATT_DESC_MAX];
  __shared__ float sh_w[NW][ATT_DESC_MAX];
  __shared__ int sh_last;
  extern __shared__ __attribute__((aligned(16))) int sh_tab[];
  int* const sh_roff = sh_tab;              // [np + 1]
  int* const sh_rst = sh_tab + P.np + 1;    // [np]

  const int g = blockIdx.y;
  const int split = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n = lane & 15, h = lane >> 4;
  const int gs = P.gs;

  WaveState<GS_PAD> st;
#pragma unroll
  for (int i = 0; i < NH; ++i) { st.m[i] = -INFINITY; st.l[i] = 0.f; }
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) st.acc[dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  uint16_t* vt = sh_vt[wave];
  uint16_t* pb = sh_pb[wave];
  float* al_sh = sh_al[wave];
  // P rows of heads that do not exist stay zero; alpha of such heads must not scale by garbage
  for (int i = lane; i < 16 * 16 / 2; i += 64) reinterpret_cast<uint32_t*>(pb)[i] = 0u;
  if (lane < 16) al_sh[lane] = 1.f;
  int* dsc = sh_desc[wave];
  float* wsh = sh_w[wave];
  const int lenB = P.lenB_ptr ? P.lenB_ptr[(size_t)g * P.lenB_ptr_stride] : P.lenB_const;
  const int lenA_all = P.lenA_ptr ? min(max(P.lenA_ptr[0], 0), (int)P.strideA) : P.lenA;

  // Estimation rows whose scores are not handed in are key/value rows of their own: key = centroid,
  // value = value sum, weight = cluster size, located through the id list.
  const bool est_split = split >= P.S_kv;
  if (!est_split || P.est_cent) {
    // ---------------- key/value rows ----------------
    // rank tables (requested together with everything else the prologue loads: no dependent round trip)
    const bool tab = !est_split && P.ret_off != nullptr;
    // every global load of the prologue is requested before the first of them is consumed
    // (up to 1023 probes the table entries pass through registers, TAB_U per thread; longer tables are
    // staged by a plain loop after the query)
    constexpr int TAB_U = 1024 / NT;
    const bool tab_fast = tab && P.np < 1024;
    int t_off[TAB_U], t_st[TAB_U];
    if (tab_fast) {
#pragma unroll
      for (int u = 0; u < TAB_U; ++u) {
        const int i = threadIdx.x + u * NT;
        t_off[u] = (i <= P.np) ? P.ret_off[(size_t)g * (P.np + 1) + i] : 0;
        t_st[u] = (i < P.np) ? P.ret_start[(size_t)g * P.np + i] : 0;
      }
    }
    // A operand: query heads through LDS (read again per chunk: registers go to the loads);
    // row m of the MFMA holds head m % GS_PAD, zero if >= gs
    static_assert(GS_PAD * (RI_DIM / 8) <= NT, "one piece of the query per thread");
    {
      const int head = threadIdx.x / (RI_DIM / 8), piece = threadIdx.x % (RI_DIM / 8);
      uint4 qv = ri_zero16();
      if (head < gs) qv = ri_ld16(P.q + ((size_t)g * gs + head) * RI_DIM + piece * 8);
      if (head < GS_PAD) *reinterpret_cast<uint4*>(&sh_q[head][piece * 8]) = qv;
    }
    if (tab_fast) {
#pragma unroll
      for (int u = 0; u < TAB_U; ++u) {
        const int i = threadIdx.x + u * NT;
        if (i <= P.np) sh_roff[i] = t_off[u];
        if (i < P.np) sh_rst[i] = t_st[u];
      }
    } else if (tab) {
      for (int i = threadIdx.x; i <= P.np; i += NT) {
        sh_roff[i] = P.ret_off[(size_t)g * (P.np + 1) + i];
        if (i < P.np) sh_rst[i] = P.ret_start[(size_t)g * P.np + i];
      }
    }
    // (the row count is consumed only now: the loads above went out together with its load)
    const int lenA = est_split ? 0 : lenA_all;
    const int total = est_split ? P.es : lenA_all + lenB;
    int r0, r1;
    if (est_split)
      wave_rows(total, P.S_es * NW, (split - P.S_kv) * NW + wave, &r0, &r1);
    else
      wave_rows(total, P.S_kv * NW, split * NW + wave, &r0, &r1);
    const uint16_t* qrow = &sh_q[n % GS_PAD][h * 8];
    const uint16_t* kA = P.kA + (size_t)g * P.strideA * RI_DIM;
    const uint16_t* vA = P.vA + (size_t)g * P.strideA * RI_DIM;
    const uint16_t* kB = est_split ? P.est_cent + (size_t)g * P.nc * RI_DIM : P.kB + (size_t)g * P.strideB * RI_DIM;
    const uint16_t* vB = est_split ? P.value_sum + (size_t)g * P.nc * RI_DIM : P.vB + (size_t)g * P.strideB * RI_DIM;
    const int32_t* rs = est_split ? P.est_ids + (size_t)g * P.es
                                  : (P.row_src ? P.row_src + (size_t)g * P.rs_stride : nullptr);
    const uint16_t* wB = (!est_split && P.weightB) ? P.weightB + (size_t)g * P.weight_stride : nullptr;
    const uint16_t* wsrc = est_split ? P.csize + (size_t)g * P.nc : nullptr;  // weight by source row
    const int r_first = ri_head_reg<GS_PAD>(h);
    bool q_ready = false;
    if (tab) {  // the tables are searched while the rows are located
      __syncthreads();
      q_ready = true;
    }

    for (int s0 = r0; s0 < r1; s0 += ATT_DESC_MAX) {
      const int s1 = min(r1, s0 + ATT_DESC_MAX);
      // stage the descriptors of rows [s0, s1): where each row lives (-1 = padding row)
      for (int i = lane; i < ATT_DESC_MAX; i += 64) {
        const int row = s0 + i;
        int d = -1;
        float w = 1.f;
        if (row < s1) {
          if (row < lenA) {
            d = row | ATT_FLAG_A;
          } else {
            const int rb = row - lenA;
            if (tab) {
              // the last rank whose first row is <= rb (ranks of empty clusters share a first row
              // with the next rank, which is the one found)
              int lo = 0, hi = P.np;
              while (lo + 1 < hi) {
                const int mid = (lo + hi) >> 1;
                if (sh_roff[mid] <= rb) lo = mid; else hi = mid;
              }
              d = sh_rst[lo] + rb - sh_roff[lo];
            } else {
              d = rs ? rs[rb] : rb;
              if (!est_split && P.row_src && (d < P.src_lo || d >= P.src_hi)) d = -1;
            }
            if (wB) w = ri_e16_to_f32<HALF>(wB[rb]);
            if (wsrc) w = ri_e16_to_f32<HALF>(wsrc[d]);
          }
        }
        dsc[i] = d;
        wsh[i] = w;
      }
      if (!q_ready) { __syncthreads(); q_ready = true; }  // sh_q complete (also orders dsc writes)
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int nch = (s1 - s0 + 15) >> 4;
      uint4 bk[PF][4], v[PF][4];
      auto issue = [&](int slot_unused, uint4* bks, uint4* vs_, int j) {
        (void)slot_unused;
        const int dk = dsc[j * 16 + n];
        const uint16_t* kp = ((dk & ATT_FLAG_A) ? kA : kB) + (size_t)(dk & ~ATT_FLAG_A) * RI_DIM + h * 8;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) bks[kk] = (dk >= 0) ? ri_ld16(kp + kk * 32) : ri_zero16();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int dv = dsc[j * 16 + h + 4 * i];
          const uint16_t* vp = ((dv & ATT_FLAG_A) ? vA : vB) + (size_t)(dv & ~ATT_FLAG_A) * RI_DIM + n * 8;
          vs_[i] = (dv >= 0) ? ri_ld16(vp) : ri_zero16();
        }
      };
      auto compute = [&](const uint4* bks, const uint4* vs_, int j) {
        f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const uint4 qv = *reinterpret_cast<const uint4*>(qrow + kk * 32);
          acc = HALF ? __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, qv),
                                                              __builtin_bit_cast(f16x8_t, bks[kk]), acc, 0, 0, 0)
                     : __builtin_amdgcn_mfma_f32_16x16x32_bf16(ri_as_bf16x8(qv), ri_as_bf16x8(bks[kk]), acc, 0, 0, 0);
        }
        float sv[NH];
#pragma unroll
        for (int i = 0; i < NH; ++i) {
          float x;
          if (GS_PAD == 16) {
            x = acc[i];
          } else {  // register r_first + i without dynamic indexing
            const int r = r_first + i;
            x = r == 0 ? acc[0] : (r == 1 ? acc[1] : (r == 2 ? acc[2] : acc[3]));
          }
          sv[i] = x * P.scale;
        }
        const bool valid = dsc[j * 16 + n] >= 0;
        const float w = wsh[j * 16 + n];
        chunk_update<GS_PAD, HALF>(st, sv, valid, w, vs_, vt, pb, al_sh, lane);
      };
#pragma unroll
      for (int s = 0; s < PF; ++s)
        if (s < nch) issue(s, bk[s], v[s], s);
      for (int j0 = 0; j0 < nch; j0 += PF) {
#pragma unroll
        for (int s = 0; s < PF; ++s) {
          const int j = j0 + s;
          if (j < nch) {
            compute(bk[s], v[s], j);
            if (j + PF < nch) issue(s, bk[s], v[s], j + PF);
          }
        }
      }
    }
    if (!q_ready) __syncthreads();  // keep the barrier count uniform for waves without rows
  } else {
    // ---------------- estimation rows ----------------
    const int es = P.es;
    int r0, r1;
    wave_rows(es, P.S_es * NW, (split - P.S_kv) * NW + wave, &r0, &r1);
    const int32_t* ids = P.est_ids + (size_t)g * es;
    const uint16_t* vs = P.value_sum + (size_t)g * P.nc * RI_DIM;
    const uint16_t* cs = P.csize + (size_t)g * P.nc;
    const float* lg = P.logits + (size_t)g * gs * P.nc;

    for (int s0 = r0; s0 < r1; s0 += ATT_DESC_MAX) {
      const int s1 = min(r1, s0 + ATT_DESC_MAX);
      for (int i = lane; i < ATT_DESC_MAX; i += 64) {
        const int row = s0 + i;
        int d = -1;
        float w = 0.f;
        if (row < s1) {
          d = ids[row];
          w = ri_e16_to_f32<HALF>(cs[d]);
        }
        dsc[i] = d;
        wsh[i] = w;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int nch = (s1 - s0 + 15) >> 4;
      float sc[PF][NH];
      uint4 v[PF][4];
      auto issue = [&](float* scs, uint4* vs_, int j) {
        const int ck = dsc[j * 16 + n];
#pragma unroll
        for (int i = 0; i < NH; ++i) {
          const int head = ri_head_of<GS_PAD>(h, i);
          scs[i] = (ck >= 0 && head < gs) ? lg[(size_t)head * P.nc + ck] : -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int cv = dsc[j * 16 + h + 4 * i];
          vs_[i] = (cv >= 0) ? ri_ld16(vs + (size_t)cv * RI_DIM + n * 8) : ri_zero16();
        }
      };
#pragma unroll
      for (int s = 0; s < PF; ++s)
        if (s < nch) issue(sc[s], v[s], s);
      for (int j0 = 0; j0 < nch; j0 += PF) {
#pragma unroll
        for (int s = 0; s < PF; ++s) {
          const int j = j0 + s;
          if (j < nch) {
            const bool valid = dsc[j * 16 + n] >= 0;
            const float w = wsh[j * 16 + n];
            chunk_update<GS_PAD, HALF>(st, sc[s], valid, w, v[s], vt, pb, al_sh, lane);
            if (j + PF < nch) issue(sc[s], v[s], j + PF);
          }
        }
      }
    }
  }

  // ---------------- wave partial -> LDS ----------------
#pragma unroll
  for (int i = 0; i < NH; ++i) {
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
  // accumulators are already summed over rows: lane (n, h) register i holds head 4h+i, dim 16*dt+n
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int head = 4 * h + i;
    if (head < GS_PAD) {
#pragma unroll
      for (int dt = 0; dt < 8; ++dt) acc_of(wave)[head * RI_DIM + 16 * dt + n] = st.acc[dt][i];
    }
  }
  __syncthreads();

  // ---------------- merge the waves, write the split partial ----------------
  const int S = P.S_kv + P.S_es;
  for (int idx = threadIdx.x; idx < GS_PAD * RI_DIM; idx += NT) {
    const int j = idx / RI_DIM, d = idx % RI_DIM;
    float M = sh_m[0][j];
#pragma unroll
    for (int w = 1; w < NW; ++w) M = fmaxf(M, sh_m[w][j]);
    float a = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = (sh_m[w][j] == -INFINITY) ? 0.f : __expf(sh_m[w][j] - M);
      a += acc_of(w)[j * RI_DIM + d] * f;
      l += sh_l[w][j] * f;
    }
    const size_t o = ((size_t)g * S + split) * GS_PAD + j;
    // device-coherent stores: another workgroup of this launch reads them
    __hip_atomic_store(&P.part_acc[o * RI_DIM + d], a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (d == 0) {
      __hip_atomic_store(&P.part_ml[o * 2], M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&P.part_ml[o * 2 + 1], l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }

  // ---------------- last workgroup of the group merges all splits ----------------
  // Hand-off of the partials between workgroups of one launch, without fences:
  //  * the partial was written above with agent-scope atomic stores: on gfx950 those are write-through
  //    stores (sc1) that complete in the memory-side cache every compute unit shares, not in this
  //    compute unit's L1 or this chiplet's L2;
  //  * s_waitcnt(0) returns when all of this wave's stores have been acknowledged there, the barrier
  //    makes that true for the whole workgroup, and only then does one thread announce the arrival with
  //    an agent-scope atomic increment (performed at the same shared level);
  //  * the workgroup that sees the count complete reads the partials with agent-scope atomic loads
  //    (combine_group), which bypass the non-coherent cache levels.
  // So every partial is globally visible before its arrival can be counted, and the reader cannot hit a
  // stale line.  The C++ memory model would express this with a release increment and an acquire on the
  // last arriver; at agent scope those compile to a write-back and an invalidate of the whole L2, which
  // was measured at +15 us per launch (35.2 us instead of 20.0 us at the benchmark shape), while the
  // data that must be ordered is only this workgroup's own 2 KB.  The asm statement keeps the compiler
  // from moving the stores below the wait.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the partial hand-off below relies on gfx950 cache behaviour: build this file for gfx950 only"
#endif
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (threadIdx.x == 0)
    sh_last = (__hip_atomic_fetch_add(&P.counters[g], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == S - 1);
  __syncthreads();
  if (!sh_last) return;
  combine_group<GS_PAD, NW, HALF>(P, g, S, lenA_all, lenB);
  // ready for the next launch (every arrival of this launch has been counted; launches that share the
  // workspace do not overlap)
  if (threadIdx.x == 0) __hip_atomic_store(&P.counters[g], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------
#define RI_MAX_SPLITS 64
#define RI_MAX_PROBES 4096  // rank tables of a launch: (2 * np + 1) * 4 bytes of LDS (what the selection lays out)
#define RI_MAX_GROUPS 4096  // size of the counter area at the head of the workspace

static inline int gs_pad_of(int gs) { return gs <= 4 ? 4 : (gs <= 8 ? 8 : 16); }

static size_t attn_workspace_bytes(int BG, int gs) {
  if (BG <= 0 || BG > RI_MAX_GROUPS || gs <= 0 || gs > 16) return 0;
  const size_t per = (size_t)BG * RI_MAX_SPLITS * gs_pad_of(gs);
  return RI_MAX_GROUPS * sizeof(int) + per * (2 + RI_DIM) * sizeof(float);
}

extern "C" size_t ri_flash_decoding_workspace_bytes(int BG, int gs) { return attn_workspace_bytes(BG, gs); }
extern "C" size_t ri_wave_attention_workspace_bytes(int BG, int gs) { return attn_workspace_bytes(BG, gs); }

// Bytes a launch with S = S_kv + S_es splits per group really uses: the counter area, then the
// (max, denominator) pairs and the numerators of BG * S partials.
static size_t attn_scratch_used(int BG, int gp, int S) {
  return RI_MAX_GROUPS * sizeof(int) + (size_t)BG * S * gp * (2 + RI_DIM) * sizeof(float);
}

static void carve_workspace(AttendParams& P, void* workspace, int BG, int gp) {
  const int S = P.S_kv + P.S_es;
  P.counters = (int*)workspace;
  P.part_ml = (float*)((char*)workspace + RI_MAX_GROUPS * sizeof(int));
  P.part_acc = P.part_ml + (size_t)BG * S * gp * 2;
}

template <bool HALF>
static void launch_attend_t(const AttendParams& P, dim3 grid, int gp, int nw, size_t tab_bytes, hipStream_t s) {
  if (nw == 8 && gp == 4) attend_kernel<4, 8, 1, HALF><<<grid, 512, tab_bytes, s>>>(P);
  else if (nw == 8 && gp == 8) attend_kernel<8, 8, 1, HALF><<<grid, 512, tab_bytes, s>>>(P);
  else if (gp == 4) attend_kernel<4, 4, 1, HALF><<<grid, 256, tab_bytes, s>>>(P);
  else if (gp == 8) attend_kernel<8, 4, 1, HALF><<<grid, 256, tab_bytes, s>>>(P);
  else attend_kernel<16, 4, 1, HALF><<<grid, 256, tab_bytes, s>>>(P);
}

static int launch_attend(AttendParams& P, int BG, int gs, int nw, bool half, hipStream_t s) {
  const int S = P.S_kv + P.S_es;
  const dim3 grid(S, BG);
  const size_t tab_bytes = P.ret_off ? (size_t)(2 * P.np + 1) * sizeof(int) : 0;
  if (half) launch_attend_t<true>(P, grid, gs_pad_of(gs), nw, tab_bytes, s);
  else launch_attend_t<false>(P, grid, gs_pad_of(gs), nw, tab_bytes, s);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

// Waves per workgroup of a launch.  Eight for groups of up to four query heads: half the split partials and
// arrivals per group at the same number of waves per compute unit (32 groups of 4 heads over 8192 clusters:
// 18.7 against 19.3 us per launch).  Four otherwise: with eight or more heads the wave partials of an
// eight-wave workgroup take so much LDS that only one workgroup fits a compute unit (64 groups of 8 heads over
// 16384 clusters: 71 against 53 us).  RI_ATTEND_WAVES=4|8 in the environment overrides the choice for groups of
// up to eight heads (read once, for measurements).
static int attend_waves(int gs) {
  static const int forced = [] {
    const char* e = getenv("RI_ATTEND_WAVES");
    return e ? atoi(e) : 0;
  }();
  const int gp = gs_pad_of(gs);
  if (gp == 16) return 4;
  if (forced == 4 || forced == 8) return forced;
  return gp == 4 ? 8 : 4;
}

// Memory traffic of one estimation row: its value-sum row, the 32-byte sector around its cluster size, and
// either one 32-byte sector per query head around its logit or, when the scores are computed in the launch,
// its centroid row.
static int est_row_bytes(int gs, bool scored_here) { return 256 + 32 + (scored_here ? 256 : 32 * gs); }

// Split plan: about two workgroups per compute unit in total (an even load over the 256 CUs,
// all resident at once), at least 128 rows per workgroup, the budget shared between the
// key/value rows and the estimation rows in proportion to the memory traffic of a row, es_row_bytes
// against the 512 bytes of a K and a V row (the launch is bound by its traffic: weighing a key/value
// row twice an estimation row, by its arithmetic, left the estimation workgroups finishing last,
// 20.2 against 19.5 us at 32 groups of 4 heads and 60.4 against 54.9 us at 64 groups of 8).
static void plan_splits(int64_t kv_rows, int64_t es_rows, int es_row_bytes, int BG, int nw, int* S_kv, int* S_es) {
  // eight waves per compute unit while the launch is short (latency counts); twelve once every
  // wave has more than 128 rows to stream (throughput counts)
  const int64_t all_rows = (kv_rows + es_rows) * BG;
  const int target_wgs = (all_rows > 512 * 512 ? 768 : 512) * 4 / nw;
  int per_group = target_wgs / BG;
  if (per_group < 1) per_group = 1;
  if (per_group > RI_MAX_SPLITS) per_group = RI_MAX_SPLITS;
  const int64_t rows = kv_rows + es_rows;
  int64_t by_rows = (rows + 32 * nw - 1) / (32 * nw);
  if (by_rows < 1) by_rows = 1;
  if (per_group > by_rows) per_group = (int)by_rows;
  if (es_rows <= 0) {
    *S_kv = per_group;
    *S_es = 0;
    return;
  }
  if (per_group < 2) per_group = 2;
  const int64_t wk = kv_rows * 512, we = es_rows * es_row_bytes;
  int kv = (int)((wk * per_group + (wk + we) / 2) / (wk + we));
  if (kv < 1) kv = 1;
  if (kv > per_group - 1) kv = per_group - 1;
  *S_kv = kv;
  *S_es = per_group - kv;
}

static int flash_decoding_impl(const void* q, const void* k, const void* v, const void* weight,
                               const int32_t* cache_seqlens, const void* prev_out, const float* prev_lse, void* out,
                               float* lse_out, int BG, int gs, int S, int64_t kv_stride, float scale, void* workspace,
                               size_t workspace_bytes, bool half, ri_stream_t stream) {
  if (!q || !k || !v || !out || !workspace) return RI_ERR_ARG;
  if (ri_any_misaligned16(q, k, v, weight, prev_out, out, workspace)) return RI_ERR_ARG;
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
  const int nw = attend_waves(gs);
  plan_splits(S, 0, 0, BG, nw, &P.S_kv, &P.S_es);
  P.gs = gs;
  P.scale = scale;
  P.prev_out = (const uint16_t*)prev_out;
  P.prev_lse = prev_lse;
  P.out = (uint16_t*)out;
  P.lse_out = lse_out;
  carve_workspace(P, workspace, BG, gp);
  return launch_attend(P, BG, gs, nw, half, (hipStream_t)stream);
}

extern "C" int ri_weighted_flash_decoding(const void* q, const void* k, const void* v, const void* weight,
                                          const int32_t* cache_seqlens, const void* prev_out,
                                          const float* prev_lse, void* out, float* lse_out, int BG, int gs,
                                          int S, int64_t kv_stride, float scale, void* workspace,
                                          size_t workspace_bytes, ri_stream_t stream) {
  return flash_decoding_impl(q, k, v, weight, cache_seqlens, prev_out, prev_lse, out, lse_out, BG, gs, S, kv_stride,
                             scale, workspace, workspace_bytes, false, stream);
}

extern "C" int ri_weighted_flash_decoding_f16(const void* q, const void* k, const void* v, const void* weight,
                                              const int32_t* cache_seqlens, const void* prev_out,
                                              const float* prev_lse, void* out, float* lse_out, int BG, int gs,
                                              int S, int64_t kv_stride, float scale, void* workspace,
                                              size_t workspace_bytes, ri_stream_t stream) {
  return flash_decoding_impl(q, k, v, weight, cache_seqlens, prev_out, prev_lse, out, lse_out, BG, gs, S, kv_stride,
                             scale, workspace, workspace_bytes, true, stream);
}

// Shared body of ri_wave_attention and ri_wave_attention_static.  `scratch` holds the arrival
// counters and the split partials; with scratch_bytes == 0 the caller vouches for its size through
// scratch_limit (the static array) and the counters are cleared by a fill kernel first.
__global__ void attend_clear_counters_kernel(int* counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}

static int wave_attention_impl(const void* q, const void* steady_k, const void* steady_v, int64_t steady_stride,
                               int static_len, const int32_t* static_len_dev, const void* store_k,
                               const void* store_v, int64_t store_stride, const int32_t* row_src,
                               int row_src_stride, const int32_t* ret_tok_off, const int32_t* ret_start, int np,
                               const int32_t* meta, const int32_t* est_ids, const float* logits,
                               const void* est_centroids, const void* value_sum, const void* cluster_size_bf16,
                               void* out, int32_t* valid_lengths, int BG, int gs, int nc, int es, float scale,
                               void* scratch, size_t scratch_bytes, bool clear_counters, bool half, hipStream_t stream,
                               int src_lo = INT32_MIN, int src_hi = INT32_MAX, const void* prev_out = nullptr,
                               const float* prev_lse = nullptr, float* lse_out = nullptr) {
  if (!q || !steady_k || !steady_v || !store_k || !store_v || !meta || !out || !scratch) return RI_ERR_ARG;
  if ((prev_out == nullptr) != (prev_lse == nullptr) || ri_misaligned16(prev_out)) return RI_ERR_ARG;
  if (ri_any_misaligned16(q, steady_k, steady_v, store_k, store_v, value_sum, est_centroids, out, scratch))
    return RI_ERR_ARG;
  if (!row_src && (!ret_tok_off || !ret_start || np <= 0 || np > RI_MAX_PROBES)) return RI_ERR_ARG;
  if ((row_src && row_src_stride <= 0) || store_stride < 0) return RI_ERR_ARG;
  if (BG <= 0 || BG > RI_MAX_GROUPS || gs <= 0 || gs > 16 || static_len < 0 || static_len > steady_stride ||
      es < 0 || nc <= 0)
    return RI_ERR_ARG;
  if (es > 0 && (!est_ids || (!logits == !est_centroids) || !value_sum || !cluster_size_bf16)) return RI_ERR_ARG;
  const int gp = gs_pad_of(gs);
  AttendParams P = {};
  P.q = (const uint16_t*)q;
  P.kA = (const uint16_t*)steady_k;
  P.vA = (const uint16_t*)steady_v;
  P.strideA = steady_stride;
  P.lenA = static_len;
  P.lenA_ptr = static_len_dev;
  P.kB = (const uint16_t*)store_k;
  P.vB = (const uint16_t*)store_v;
  P.strideB = store_stride;
  P.row_src = row_src;
  P.rs_stride = row_src_stride;
  P.src_lo = src_lo;
  P.src_hi = src_hi;
  P.prev_out = (const uint16_t*)prev_out;
  P.prev_lse = prev_lse;
  P.lse_out = lse_out;
  if (!row_src) {
    P.ret_off = ret_tok_off;
    P.ret_start = ret_start;
    P.np = np;
  }
  P.lenB_ptr = meta + 1;
  P.lenB_ptr_stride = 4;
  P.est_ids = est_ids;
  P.logits = logits;
  P.est_cent = (const uint16_t*)est_centroids;
  P.value_sum = (const uint16_t*)value_sum;
  P.csize = (const uint16_t*)cluster_size_bf16;
  P.nc = nc;
  P.es = es;
  P.gs = gs;
  P.scale = scale;
  P.out = (uint16_t*)out;
  P.valid_lengths = valid_lengths;
  // the retrieved-token count is only known on the device: size the split for the row table
  // capacity scaled by the usual fill (a quarter) or for 16 tokens per rank, the estimation zone by
  // its exact size
  const int nw = attend_waves(gs);
  plan_splits(static_len + (row_src ? row_src_stride / 4 : np * 16), es, est_row_bytes(gs, est_centroids != nullptr), BG,
              nw, &P.S_kv, &P.S_es);
  if (scratch_bytes < attn_scratch_used(BG, gp, P.S_kv + P.S_es)) return RI_ERR_WORKSPACE;
  carve_workspace(P, scratch, BG, gp);
  if (clear_counters) {
    attend_clear_counters_kernel<<<(BG + 255) / 256, 256, 0, stream>>>(P.counters, BG);
    RI_HIP_CHECK_LAUNCH();
  }
  return launch_attend(P, BG, gs, nw, half, stream);
}

// Clears the arrival counters at the head of an attention workspace with a small kernel on `stream` (no
// memset: the call can be captured).  Every attention launch leaves its counters at zero, so this is only
// needed after a launch that did not run to its end (a fault, a device reset): its groups' counters may be
// left non-zero, and later launches on that workspace would then never see a last arrival and write nothing.
extern "C" int ri_attention_workspace_reset(void* workspace, size_t workspace_bytes, ri_stream_t stream) {
  if (!workspace || ri_misaligned16(workspace)) return RI_ERR_ARG;
  if (workspace_bytes < RI_MAX_GROUPS * sizeof(int)) return RI_ERR_WORKSPACE;
  attend_clear_counters_kernel<<<(RI_MAX_GROUPS + 255) / 256, 256, 0, (hipStream_t)stream>>>((int*)workspace,
                                                                                             RI_MAX_GROUPS);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

static int ri_wave_attention_any(const void* q, const void* steady_k, const void* steady_v,
                                 int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                 const void* store_k,
                                 const void* store_v, int64_t store_stride, const int32_t* row_src,
                                 int row_src_stride, const int32_t* ret_tok_off, const int32_t* ret_start, int np,
                                 const int32_t* meta, const int32_t* est_ids,
                                 const float* logits, const void* est_centroids, const void* value_sum,
                                 const void* cluster_size_bf16, void* out, int32_t* valid_lengths, int BG, int gs,
                                 int nc, int es, float scale, void* workspace, size_t workspace_bytes,
                                 ri_stream_t stream, bool half) {
  if (workspace && workspace_bytes < attn_workspace_bytes(BG, gs)) return RI_ERR_WORKSPACE;
  return wave_attention_impl(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v,
                             store_stride, row_src, row_src_stride, ret_tok_off, ret_start, np, meta, est_ids, logits,
                             est_centroids, value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale,
                             workspace, workspace_bytes, false, half, (hipStream_t)stream);
}

extern "C" int ri_wave_attention(const void* q, const void* steady_k, const void* steady_v,
                                 int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                 const void* store_k,
                                 const void* store_v, int64_t store_stride, const int32_t* row_src,
                                 int row_src_stride, const int32_t* ret_tok_off, const int32_t* ret_start, int np,
                                 const int32_t* meta, const int32_t* est_ids,
                                 const float* logits, const void* est_centroids, const void* value_sum,
                                 const void* cluster_size_bf16, void* out, int32_t* valid_lengths, int BG, int gs,
                                 int nc, int es, float scale, void* workspace, size_t workspace_bytes,
                                 ri_stream_t stream) {
  return ri_wave_attention_any(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v, store_stride, row_src, row_src_stride, ret_tok_off, ret_start, np, meta, est_ids, logits, est_centroids, value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale, workspace, workspace_bytes, stream, false);
}

extern "C" int ri_wave_attention_f16(const void* q, const void* steady_k, const void* steady_v,
                                 int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                 const void* store_k,
                                 const void* store_v, int64_t store_stride, const int32_t* row_src,
                                 int row_src_stride, const int32_t* ret_tok_off, const int32_t* ret_start, int np,
                                 const int32_t* meta, const int32_t* est_ids,
                                 const float* logits, const void* est_centroids, const void* value_sum,
                                 const void* cluster_size_bf16, void* out, int32_t* valid_lengths, int BG, int gs,
                                 int nc, int es, float scale, void* workspace, size_t workspace_bytes,
                                 ri_stream_t stream) {
  return ri_wave_attention_any(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v, store_stride, row_src, row_src_stride, ret_tok_off, ret_start, np, meta, est_ids, logits, est_centroids, value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale, workspace, workspace_bytes, stream, true);
}

// Part of a wave attention: the steady zone and estimation zone as asked for, and of the rows of the row
// table only those whose source row lies in [src_row_lo, src_row_hi); an earlier part's result comes in
// as (prev_out, prev_lse) and this part's log-sum-exp goes out, so that two launches over disjoint row
// windows give the attention over all rows.  Used with a host-resident store: the rows already in the
// block cache are attended while the missed blocks are still being staged, and the staged rows follow.
static int ri_wave_attention_part_any(const void* q, const void* steady_k, const void* steady_v,
                                      int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                      const void* store_k, const void* store_v, int64_t store_stride,
                                      const int32_t* row_src, int row_src_stride, int src_row_lo, int src_row_hi,
                                      const int32_t* meta, const int32_t* est_ids, const float* logits,
                                      const void* value_sum, const void* cluster_size_bf16, const void* prev_out,
                                      const float* prev_lse, void* out, float* lse_out, int32_t* valid_lengths,
                                      int BG, int gs, int nc, int es, float scale, void* workspace,
                                      size_t workspace_bytes, ri_stream_t stream, bool half) {
  if (!row_src || src_row_lo > src_row_hi) return RI_ERR_ARG;   // an empty window attends none of the table's rows
  if (workspace && workspace_bytes < attn_workspace_bytes(BG, gs)) return RI_ERR_WORKSPACE;
  // a part that leaves the steady zone out must not pick its length up from the device either
  if (static_len == 0) static_len_dev = nullptr;
  return wave_attention_impl(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v,
                             store_stride, row_src, row_src_stride, nullptr, nullptr, 0, meta, est_ids, logits, nullptr,
                             value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale, workspace,
                             workspace_bytes, false, half, (hipStream_t)stream, src_row_lo, src_row_hi, prev_out, prev_lse,
                             lse_out);
}

extern "C" int ri_wave_attention_part(const void* q, const void* steady_k, const void* steady_v,
                                      int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                      const void* store_k, const void* store_v, int64_t store_stride,
                                      const int32_t* row_src, int row_src_stride, int src_row_lo, int src_row_hi,
                                      const int32_t* meta, const int32_t* est_ids, const float* logits,
                                      const void* value_sum, const void* cluster_size_bf16, const void* prev_out,
                                      const float* prev_lse, void* out, float* lse_out, int32_t* valid_lengths,
                                      int BG, int gs, int nc, int es, float scale, void* workspace,
                                      size_t workspace_bytes, ri_stream_t stream) {
  return ri_wave_attention_part_any(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v, store_stride, row_src, row_src_stride, src_row_lo, src_row_hi, meta, est_ids, logits, value_sum, cluster_size_bf16, prev_out, prev_lse, out, lse_out, valid_lengths, BG, gs, nc, es, scale, workspace, workspace_bytes, stream, false);
}

extern "C" int ri_wave_attention_part_f16(const void* q, const void* steady_k, const void* steady_v,
                                      int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                      const void* store_k, const void* store_v, int64_t store_stride,
                                      const int32_t* row_src, int row_src_stride, int src_row_lo, int src_row_hi,
                                      const int32_t* meta, const int32_t* est_ids, const float* logits,
                                      const void* value_sum, const void* cluster_size_bf16, const void* prev_out,
                                      const float* prev_lse, void* out, float* lse_out, int32_t* valid_lengths,
                                      int BG, int gs, int nc, int es, float scale, void* workspace,
                                      size_t workspace_bytes, ri_stream_t stream) {
  return ri_wave_attention_part_any(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v, store_stride, row_src, row_src_stride, src_row_lo, src_row_hi, meta, est_ids, logits, value_sum, cluster_size_bf16, prev_out, prev_lse, out, lse_out, valid_lengths, BG, gs, nc, es, scale, workspace, workspace_bytes, stream, true);
}

// ------------------------------------------------------------------------------------
// The same attention for callers that cannot allocate (code under stream capture, serving loops,
// harnesses that forbid hipMalloc): arrival counters and split partials live in a static device
// array of RI_STATIC_SCRATCH_BYTES that every GPU holds from the moment the library is loaded.
// Its address is looked up once per device; host code only ever uses that address.
// ------------------------------------------------------------------------------------
#define RI_STATIC_SCRATCH_BYTES (8u << 20)
#define RI_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[RI_STATIC_SCRATCH_BYTES];
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[RI_MAX_DEVICES] = {};

// device address of this GPU's copy of `scratch` (looked up on the first call on the device)
static int static_scratch_ptr(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { ri_set_last_hip_error((int)e); return RI_ERR_LAUNCH; }
  if (dev < 0 || dev >= RI_MAX_DEVICES) return RI_ERR_ARG;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) { ri_set_last_hip_error((int)e); return RI_ERR_LAUNCH; }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return RI_OK;
}

// (also looks the array's address up on the current device, so that a caller who asks for the size before
// capturing a stream has the first-call work behind it: the look-up can load the code object)
extern "C" size_t ri_wave_attention_static_scratch_bytes(void) {
  void* ptr = nullptr;
  (void)static_scratch_ptr(&ptr);
  return RI_STATIC_SCRATCH_BYTES;
}

static int ri_wave_attention_static_any(const void* q, const void* steady_k, const void* steady_v,
                                        int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                        const void* store_k, const void* store_v, int64_t store_stride,
                                        const int32_t* row_src, int row_src_stride, const int32_t* ret_tok_off,
                                        const int32_t* ret_start, int np, const int32_t* meta,
                                        const int32_t* est_ids, const float* logits, const void* est_centroids,
                                        const void* value_sum, const void* cluster_size_bf16, void* out,
                                        int32_t* valid_lengths, int BG, int gs, int nc, int es, float scale,
                                        ri_stream_t stream, bool half) {
  void* ptr = nullptr;
  const int rc = static_scratch_ptr(&ptr);
  if (rc) return rc;
  // the array keeps what the previous call left: the counters are cleared by a kernel on the caller's
  // stream (a fill kernel, not a memset, so that the call can be captured into a graph)
  return wave_attention_impl(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v,
                             store_stride, row_src, row_src_stride, ret_tok_off, ret_start, np, meta, est_ids, logits,
                             est_centroids, value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale, ptr,
                             RI_STATIC_SCRATCH_BYTES, true, half, (hipStream_t)stream);
}

extern "C" int ri_wave_attention_static(const void* q, const void* steady_k, const void* steady_v,
                                        int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                        const void* store_k, const void* store_v, int64_t store_stride,
                                        const int32_t* row_src, int row_src_stride, const int32_t* ret_tok_off,
                                        const int32_t* ret_start, int np, const int32_t* meta,
                                        const int32_t* est_ids, const float* logits, const void* est_centroids,
                                        const void* value_sum, const void* cluster_size_bf16, void* out,
                                        int32_t* valid_lengths, int BG, int gs, int nc, int es, float scale,
                                        ri_stream_t stream) {
  return ri_wave_attention_static_any(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v, store_stride, row_src, row_src_stride, ret_tok_off, ret_start, np, meta, est_ids, logits, est_centroids, value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale, stream, false);
}

extern "C" int ri_wave_attention_static_f16(const void* q, const void* steady_k, const void* steady_v,
                                        int64_t steady_stride, int static_len, const int32_t* static_len_dev,
                                        const void* store_k, const void* store_v, int64_t store_stride,
                                        const int32_t* row_src, int row_src_stride, const int32_t* ret_tok_off,
                                        const int32_t* ret_start, int np, const int32_t* meta,
                                        const int32_t* est_ids, const float* logits, const void* est_centroids,
                                        const void* value_sum, const void* cluster_size_bf16, void* out,
                                        int32_t* valid_lengths, int BG, int gs, int nc, int es, float scale,
                                        ri_stream_t stream) {
  return ri_wave_attention_static_any(q, steady_k, steady_v, steady_stride, static_len, static_len_dev, store_k, store_v, store_stride, row_src, row_src_stride, ret_tok_off, ret_start, np, meta, est_ids, logits, est_centroids, value_sum, cluster_size_bf16, out, valid_lengths, BG, gs, nc, es, scale, stream, true);
}

static int ri_buffer_attention_any(const void* q, const void* buf_k, const void* buf_v, int64_t buf_stride,
                                   const int32_t* cache_seqlens, int max_len, const int32_t* est_ids,
                                   const float* logits, const void* value_sum, const void* cluster_size_bf16,
                                   void* out, int BG, int gs, int nc, int es, float scale, void* workspace,
                                   size_t workspace_bytes, ri_stream_t stream, bool half) {
  if (!q || !buf_k || !buf_v || !cache_seqlens || !out || !workspace) return RI_ERR_ARG;
  if (ri_any_misaligned16(q, buf_k, buf_v, value_sum, out, workspace)) return RI_ERR_ARG;
  if (BG <= 0 || BG > RI_MAX_GROUPS || gs <= 0 || gs > 16 || max_len <= 0 || max_len > buf_stride || es < 0 ||
      nc <= 0)
    return RI_ERR_ARG;
  if (es > 0 && (!est_ids || !logits || !value_sum || !cluster_size_bf16)) return RI_ERR_ARG;
  if (workspace_bytes < attn_workspace_bytes(BG, gs)) return RI_ERR_WORKSPACE;
  const int gp = gs_pad_of(gs);
  AttendParams P = {};
  P.q = (const uint16_t*)q;
  P.kA = P.kB = (const uint16_t*)buf_k;
  P.vA = P.vB = (const uint16_t*)buf_v;
  P.strideA = P.strideB = buf_stride;
  P.lenA = 0;
  P.lenB_ptr = cache_seqlens;
  P.lenB_ptr_stride = 1;
  P.lenB_const = max_len;
  P.est_ids = est_ids;
  P.logits = logits;
  P.value_sum = (const uint16_t*)value_sum;
  P.csize = (const uint16_t*)cluster_size_bf16;
  P.nc = nc;
  P.es = es;
  P.gs = gs;
  P.scale = scale;
  P.out = (uint16_t*)out;
  // the valid lengths are only known on the device: size the split for a quarter of the buffer
  const int nw = attend_waves(gs);
  plan_splits(max_len / 4 + 64, es, est_row_bytes(gs, false), BG, nw, &P.S_kv, &P.S_es);
  carve_workspace(P, workspace, BG, gp);
  return launch_attend(P, BG, gs, nw, half, (hipStream_t)stream);
}

extern "C" int ri_buffer_attention(const void* q, const void* buf_k, const void* buf_v, int64_t buf_stride,
                                   const int32_t* cache_seqlens, int max_len, const int32_t* est_ids,
                                   const float* logits, const void* value_sum, const void* cluster_size_bf16,
                                   void* out, int BG, int gs, int nc, int es, float scale, void* workspace,
                                   size_t workspace_bytes, ri_stream_t stream) {
  return ri_buffer_attention_any(q, buf_k, buf_v, buf_stride, cache_seqlens, max_len, est_ids, logits, value_sum, cluster_size_bf16, out, BG, gs, nc, es, scale, workspace, workspace_bytes, stream, false);
}

extern "C" int ri_buffer_attention_f16(const void* q, const void* buf_k, const void* buf_v, int64_t buf_stride,
                                   const int32_t* cache_seqlens, int max_len, const int32_t* est_ids,
                                   const float* logits, const void* value_sum, const void* cluster_size_bf16,
                                   void* out, int BG, int gs, int nc, int es, float scale, void* workspace,
                                   size_t workspace_bytes, ri_stream_t stream) {
  return ri_buffer_attention_any(q, buf_k, buf_v, buf_stride, cache_seqlens, max_len, est_ids, logits, value_sum, cluster_size_bf16, out, BG, gs, nc, es, scale, workspace, workspace_bytes, stream, true);
}

