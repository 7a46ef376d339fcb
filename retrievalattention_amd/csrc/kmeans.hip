// Prefill k-means kernels (gfx950): inner-product assignment on bf16 MFMA, deterministic
// inverted lists, and list-ordered segmented reductions for centroid and value sums.
// Restates cache_hub/kmeans.py (assign :6-49, update :52-80, reverse index :128-173,
// index add :176-221) with a fixed summation order instead of fp32 atomics.
#include "ri_common.h"

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* km_lds_ptr;
typedef const __attribute__((address_space(1))) void* km_glb_ptr;

#define KM_WAVES 4        // waves per workgroup sharing one centroid tile
// The assignment kernel comes in two tilings (KM_TT 32-token MFMA columns per wave held in registers,
// KM_CT centroid rows per LDS tile):
//   4 x 128  long centroid loops (more than KM_WIDE_MIN_NC centroids per problem): most reuse of every LDS read,
//            256 VGPRs and 64 KiB of LDS, two workgroups per CU;
//   2 x 32   short loops (the segmented iterations: 512 centroids per problem): the load of the tokens in
//            front of the loop is a large part of the kernel, and 126 VGPRs / 16 KiB let four workgroups per
//            CU overlap one's loads with the others' MFMAs.
// Measured with 8 x 131072 tokens: 512 centroids per problem 125.6 against 135.4 us, 1024: 228 against 252,
// 2048: 433 against 457, 4096: 836 against 845, 8192: 1639 against 1611 us.
#define KM_WIDE_MIN_NC 4096

// 16 bytes per lane from global memory straight into LDS: lane l lands at lds_base + 16 l
// (lds_base: byte address inside the workgroup's LDS, the same in every lane).  The wait for the
// data is the caller's (s_waitcnt vmcnt): issued as inline assembly so that LDS reads of other
// buffers are not made to wait for it.
__device__ __forceinline__ void km_lds_dma16(const void* g, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(lds_base) : "memory", "m0");
}

// first data row of problem p: problems are `seg` consecutive N-row slices of each head
__device__ __forceinline__ size_t km_row0(int p, int seg, int64_t head_rows, int N) {
  return (size_t)(p / seg) * (size_t)head_rows + (size_t)(p % seg) * (size_t)N;
}

// ------------------------------------------------------------------------------------
// assign: grid (ceil(N / (KM_WAVES * 32 * KM_TT)), P), KM_WAVES waves; a wave keeps KM_TT columns of 32
// tokens in registers for the whole kernel (KM_TT independent accumulator chains).  Centroid
// tiles of KM_CT rows go through two LDS buffers shared by all waves of the workgroup: the next
// tile is requested from global memory straight into the other buffer (no registers, no LDS
// stores) before the MFMAs of the current one, one wait and one barrier per tile.  (On the full-size
// pass 4 token columns x 4 waves measured fastest against 2x4, 2x8, 2x12, 3x8, and 128-row tiles
// against 64 and 256, with clocks warmed up and runs interleaved.)
// MFMA 32x32x16: A = centroid rows, B = token columns; accumulator i of lane l is
// row (i/4)*8 + (l/32)*4 + i%4, column l%32.  nc is a multiple of 32; the last tile may hold
// fewer sub-tiles.
// ------------------------------------------------------------------------------------
// HALF: keys and centroids are IEEE half instead of bfloat16.
template <int KM_TT, int KM_CT, bool HALF>
__global__ __launch_bounds__(KM_WAVES * 64) void km_assign_kernel(const uint16_t* __restrict__ data,
                                                                  const uint16_t* __restrict__ cent,
                                                                  int32_t* __restrict__ assign, int N, int nc,
                                                                  int seg, int64_t head_rows) {
  static_assert(KM_CT % (4 * KM_WAVES) == 0 && KM_CT % 32 == 0, "a tile is whole 1 KiB wave loads and whole sub-tiles");
  constexpr int KM_WG_TOKENS = KM_WAVES * 32 * KM_TT;
  __shared__ __attribute__((aligned(1024))) uint16_t sh_c[2][KM_CT][RI_DIM];
  const int p = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, hh = lane >> 5;
  const int t0 = blockIdx.x * KM_WG_TOKENS + wave * (32 * KM_TT);
  const uint16_t* dp = data + km_row0(p, seg, head_rows, N) * RI_DIM;
  const uint16_t* cp = cent + (size_t)p * nc * RI_DIM;

  // A tile goes from global memory straight into LDS, 16 bytes per lane and 1 KiB (four rows)
  // per wave instruction: lane l lands at byte l * 16 of the instruction's LDS window, and which
  // global piece it fetches is free, so the 16-byte pieces of row w are stored at piece ^ (w & 15):
  // the 16 lanes of a ds_read_b128 phase then hit 16 different piece positions (all 64 banks once).
  const int ld_row = lane >> 4, ld_piece = lane & 15;
  const uint32_t sh_base = (uint32_t)(uintptr_t)(km_lds_ptr)&sh_c[0][0][0];
  auto tile_load = [&](int ct, int buf) {
#pragma unroll
    for (int u = 0; u < KM_CT / 4 / KM_WAVES; ++u) {
      const int row4 = (wave + u * KM_WAVES) * 4;      // first of the four rows of this instruction
      const int row = row4 + ld_row;
      if (ct + row4 < nc) {  // uniform: nc is a multiple of 32
        const uint16_t* g = cp + (size_t)(ct + row) * RI_DIM + ((ld_piece ^ (row & 15)) * 8);
        km_lds_dma16(g, __builtin_amdgcn_readfirstlane(sh_base + (uint32_t)((buf * KM_CT + row4) * RI_DIM * 2)));
      }
    }
  };
  tile_load(0, 0);
  uint4 b[KM_TT][8];
#pragma unroll
  for (int tt = 0; tt < KM_TT; ++tt) {
    const int tok = t0 + tt * 32 + r;
    const uint16_t* q = dp + (size_t)tok * RI_DIM + hh * 8;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) b[tt][kk] = (tok < N) ? ri_ld16(q + kk * 16) : ri_zero16();
  }
  // (the token registers are consumed here so that the compiler's own wait for their loads sits
  // in front of the loop and not inside it, where it would also wait for the tile in flight)
#pragma unroll
  for (int tt = 0; tt < KM_TT; ++tt)
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) asm volatile("" : : "v"(b[tt][kk].x));
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  float best[KM_TT];
  int bidx[KM_TT];
#pragma unroll
  for (int tt = 0; tt < KM_TT; ++tt) {
    best[tt] = -INFINITY;
    bidx[tt] = 0;
  }
  int buf = 0;
  for (int ct = 0; ct < nc; ct += KM_CT, buf ^= 1) {
    const int nxt = ct + KM_CT;
    if (nxt < nc) tile_load(nxt, buf ^ 1);
#pragma unroll
    for (int half = 0; half < KM_CT / 32; ++half) {
      if (ct + half * 32 < nc) {  // uniform: only the last tile can lack sub-tiles
        f32x16_t acc[KM_TT];
#pragma unroll
        for (int tt = 0; tt < KM_TT; ++tt)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[tt][i] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
          const uint4 a = *reinterpret_cast<const uint4*>(&sh_c[buf][half * 32 + r][((kk * 2 + hh) ^ (r & 15)) * 8]);
#pragma unroll
          for (int tt = 0; tt < KM_TT; ++tt)
            acc[tt] = HALF ? __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                                    __builtin_bit_cast(f16x8_t, b[tt][kk]), acc[tt], 0, 0, 0)
                           : __builtin_amdgcn_mfma_f32_32x32x16_bf16(ri_as_bf16x8(a), ri_as_bf16x8(b[tt][kk]), acc[tt], 0,
                                                                     0, 0);
        }
        // argmax epilogue: the lane's 16 scores are in ascending row order, so the first score
        // equal to their maximum is the lowest row; the index search only runs when some lane
        // of the wave improves on its best (about half of the sub-tiles of a full-size pass)
#pragma unroll
        for (int tt = 0; tt < KM_TT; ++tt) {
          float m = acc[tt][0];
#pragma unroll
          for (int i = 1; i < 16; ++i) m = fmaxf(m, acc[tt][i]);
          const bool upd = m > best[tt];
          if (__builtin_amdgcn_ballot_w64(upd) != 0ull) {
            int sel = 15;
#pragma unroll
            for (int i = 14; i >= 0; --i) sel = (acc[tt][i] == m) ? i : sel;
            if (upd) {
              best[tt] = m;
              bidx[tt] = ct + half * 32 + (sel >> 2) * 8 + hh * 4 + (sel & 3);
            }
          }
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
#pragma unroll
  for (int tt = 0; tt < KM_TT; ++tt) {
    const float ob = __shfl_xor(best[tt], 32);
    const int oi = __shfl_xor(bidx[tt], 32);
    if (ob > best[tt] || (ob == best[tt] && oi < bidx[tt])) {
      best[tt] = ob;
      bidx[tt] = oi;
    }
    const int tok = t0 + tt * 32 + r;
    if (hh == 0 && tok < N) assign[(size_t)p * N + tok] = bidx[tt];
  }
}

// ------------------------------------------------------------------------------------
// inverted lists
// ------------------------------------------------------------------------------------
// Inverted lists are a stable sort of the token ids by cluster id: one or two least-significant-
// digit counting passes of at most 9 bits.  A pass is three launches: per-chunk digit histograms
// (one wave per chunk of KM_SORT_CHUNK tokens, wave-private LDS counters), an exclusive scan of
// the [digit][chunk] table per problem, and a scatter in which every wave walks its chunk in
// token order, ranks equal digits inside each 64-token round with ballots and keeps running
// positions in LDS.  Stability makes every list ascending without any per-list sort, and no
// global atomics are involved, so the result does not depend on scheduling.
#define KM_SORT_CHUNK 1024
#define KM_SORT_ROUNDS (KM_SORT_CHUNK / 64)
#define KM_SORT_MAX_BINS 512

__device__ __forceinline__ void km_wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// chunk_hist[p][digit][chunk] = tokens of the chunk whose key has that digit
__global__ __launch_bounds__(256) void km_sort_hist_kernel(const int32_t* __restrict__ keys,
                                                           int32_t* __restrict__ chunk_hist, int N, int nchunks,
                                                           int shift, int bits) {
  __shared__ int32_t sh[4][KM_SORT_MAX_BINS];
  const int p = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = blockIdx.x * 4 + wave;
  const int bins = 1 << bits;
  if (chunk >= nchunks) return;
  int32_t* h = sh[wave];
  for (int b = lane; b < bins; b += 64) h[b] = 0;
  km_wave_lds_sync();
  const int base = chunk * KM_SORT_CHUNK;
  int32_t k[KM_SORT_ROUNDS];
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r) {
    const int i = base + r * 64 + lane;
    k[r] = (i < N) ? keys[(size_t)p * N + i] : -1;
  }
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r)
    if (base + r * 64 + lane < N) atomicAdd(&h[(k[r] >> shift) & (bins - 1)], 1);
  km_wave_lds_sync();
  for (int b = lane; b < bins; b += 64) chunk_hist[((size_t)p * bins + b) * nchunks + chunk] = h[b];
}

// in-place exclusive prefix sum over the n = bins * nchunks entries of each problem.
// When the digit of this pass is the whole cluster id (offsets != nullptr), the scanned entry of
// (digit c, chunk 0) is where list c starts: the CSR offsets and the counts are written here.
__global__ __launch_bounds__(1024) void km_sort_scan_kernel(int32_t* __restrict__ chunk_hist, int n,
                                                            int32_t* __restrict__ offsets,
                                                            int32_t* __restrict__ counts, int nchunks, int nc,
                                                            int N) {
  __shared__ int32_t sh_w[16];
  __shared__ int32_t sh_carry;
  int32_t* a = chunk_hist + (size_t)blockIdx.x * n;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) sh_carry = 0;
  __syncthreads();
  for (int base = 0; base < n; base += 4096) {
    const int i0 = base + threadIdx.x * 4;
    int32_t v[4], run = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      v[u] = (i0 + u < n) ? a[i0 + u] : 0;
      run += v[u];
    }
    int32_t inc = run;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t o = __shfl_up(inc, d);
      if (lane >= d) inc += o;
    }
    if (lane == 63) sh_w[wave] = inc;
    __syncthreads();
    int32_t woff = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int32_t x = sh_w[w];
      if (w < wave) woff += x;
      tot += x;
    }
    int32_t ex = sh_carry + woff + inc - run;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (i0 + u < n) a[i0 + u] = ex;
      ex += v[u];
    }
    __syncthreads();
    if (threadIdx.x == 0) sh_carry += tot;
    __syncthreads();
  }
  if (!offsets) return;
  // (the barrier above made the scanned table visible to the whole workgroup)
  int32_t* off = offsets + (size_t)blockIdx.x * (nc + 1);
  for (int c = threadIdx.x; c <= nc; c += 1024) {
    const int32_t lo = (c < nc) ? a[(size_t)c * nchunks] : N;
    off[c] = lo;
    if (c < nc) {
      const int32_t hi = (c + 1 < nc) ? a[(size_t)(c + 1) * nchunks] : N;
      counts[(size_t)blockIdx.x * nc + c] = hi - lo;
    }
  }
}

// toks == nullptr: token id = position (first pass); out_keys == nullptr: last pass
__global__ __launch_bounds__(256) void km_sort_scatter_kernel(const int32_t* __restrict__ keys,
                                                              const int32_t* __restrict__ toks,
                                                              const int32_t* __restrict__ chunk_hist,
                                                              int32_t* __restrict__ out_keys,
                                                              int32_t* __restrict__ out_toks, int N, int nchunks,
                                                              int shift, int bits) {
  __shared__ int32_t sh[4][KM_SORT_MAX_BINS];
  const int p = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = blockIdx.x * 4 + wave;
  const int bins = 1 << bits;
  if (chunk >= nchunks) return;
  int32_t* run = sh[wave];
  for (int b = lane; b < bins; b += 64) run[b] = chunk_hist[((size_t)p * bins + b) * nchunks + chunk];
  const int base = chunk * KM_SORT_CHUNK;
  int32_t k[KM_SORT_ROUNDS], t[KM_SORT_ROUNDS];
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r) {
    const int i = base + r * 64 + lane;
    k[r] = (i < N) ? keys[(size_t)p * N + i] : 0;
    t[r] = (i < N && toks) ? toks[(size_t)p * N + i] : i;
  }
  km_wave_lds_sync();
  const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r) {
    const bool valid = base + r * 64 + lane < N;
    const int bin = (k[r] >> shift) & (bins - 1);
    uint64_t peers = __ballot(valid);  // lanes of this round with the same digit
    for (int b = 0; b < bits; ++b) {
      const bool bit = (bin >> b) & 1;
      const uint64_t m = __ballot(valid && bit);
      peers &= bit ? m : ~m;
    }
    const int start = run[bin];
    km_wave_lds_sync();  // every lane has read the running position before the leader advances it
    if (valid) {
      const int pos = start + __popcll(peers & below);
      if (lane == 63 - __clzll((long long)peers)) run[bin] = start + __popcll(peers);
      out_toks[(size_t)p * N + pos] = t[r];
      if (out_keys) out_keys[(size_t)p * N + pos] = k[r];
    }
    km_wave_lds_sync();
  }
}

// The three launches above in one, for problems that fit one workgroup (at most KM_SMALL_MAX tokens,
// cluster ids of at most 9 bits: a segment of the segmented iterations): sixteen waves take
// consecutive chunks of the problem's tokens, count their digits into wave-private LDS rows, the
// workgroup scans the [digit][wave] table in LDS, and every wave scatters its chunk as
// km_sort_scatter_kernel does.  Same stable order, hence the same lists; the digit table never
// leaves LDS.  Writes offsets and counts like the one-pass scan.
#define KM_SMALL_WAVES 16
#define KM_SMALL_MAX (KM_SMALL_WAVES * KM_SORT_CHUNK)

__global__ __launch_bounds__(KM_SMALL_WAVES * 64) void km_sort_small_kernel(const int32_t* __restrict__ keys,
                                                                           int32_t* __restrict__ offsets,
                                                                           int32_t* __restrict__ counts,
                                                                           int32_t* __restrict__ members, int N,
                                                                           int nc, int bits) {
  __shared__ int32_t sh[KM_SMALL_WAVES][KM_SORT_MAX_BINS];
  __shared__ int32_t sh_w[KM_SMALL_WAVES];
  const int p = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int bins = 1 << bits;
  const int rounds = (N + KM_SMALL_WAVES * 64 - 1) / (KM_SMALL_WAVES * 64);   // 64-token rounds per wave
  const int base = wave * rounds * 64;
  int32_t* run = sh[wave];
  for (int b = lane; b < bins; b += 64) run[b] = 0;
  km_wave_lds_sync();
  int32_t k[KM_SORT_ROUNDS];
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r) {
    const int i = base + r * 64 + lane;
    k[r] = (r < rounds && i < N) ? (keys[(size_t)p * N + i] & (bins - 1)) : -1;
  }
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r)
    if (k[r] >= 0) atomicAdd(&run[k[r]], 1);
  __syncthreads();
  // exclusive scan in (digit, wave) order: thread t owns digit t / 2, waves 8 (t % 2) .. + 7
  {
    const int t = threadIdx.x, bin = t >> 1, w0 = (t & 1) * 8;
    int32_t v[8], tot = 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      v[u] = (bin < bins) ? sh[w0 + u][bin] : 0;
      tot += v[u];
    }
    int32_t inc = tot;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t o = __shfl_up(inc, d);
      if (lane >= d) inc += o;
    }
    if (lane == 63) sh_w[wave] = inc;
    const int32_t pair = tot + __shfl_down(tot, 1);   // even t: the digit's count over all waves
    __syncthreads();
    int32_t ex = inc - tot;
#pragma unroll
    for (int w = 0; w < KM_SMALL_WAVES; ++w)
      if (w < wave) ex += sh_w[w];
    if ((t & 1) == 0 && bin < nc) {
      offsets[(size_t)p * (nc + 1) + bin] = ex;
      counts[(size_t)p * nc + bin] = pair;
    }
    if (t == 0) offsets[(size_t)p * (nc + 1) + nc] = N;
    if (bin < bins) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        sh[w0 + u][bin] = ex;
        ex += v[u];
      }
    }
  }
  __syncthreads();
  const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
  for (int r = 0; r < KM_SORT_ROUNDS; ++r) {
    if (r < rounds) {   // uniform
      const bool valid = k[r] >= 0;
      const int bin = valid ? k[r] : 0;
      uint64_t peers = __ballot(valid);  // lanes of this round with the same digit
      for (int b = 0; b < bits; ++b) {
        const bool bit = (bin >> b) & 1;
        const uint64_t m = __ballot(valid && bit);
        peers &= bit ? m : ~m;
      }
      const int start = run[bin];
      km_wave_lds_sync();  // every lane has read the running position before the leader advances it
      if (valid) {
        const int pos = start + __popcll(peers & below);
        if (lane == 63 - __clzll((long long)peers)) run[bin] = start + __popcll(peers);
        members[(size_t)p * N + pos] = base + r * 64 + lane;
      }
      km_wave_lds_sync();
    }
  }
}

// CSR offsets from the sorted members: position i starts every cluster in (key[i-1], key[i]]
__global__ __launch_bounds__(256) void km_bounds_kernel(const int32_t* __restrict__ assign,
                                                        const int32_t* __restrict__ members,
                                                        int32_t* __restrict__ offsets, int N, int nc) {
  const int p = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  const int32_t* as = assign + (size_t)p * N;
  const int32_t* mem = members + (size_t)p * N;
  int32_t* off = offsets + (size_t)p * (nc + 1);
  const int c = min(max(as[mem[i]], 0), nc - 1);
  const int cprev = (i > 0) ? min(max(as[mem[i - 1]], 0), nc - 1) : -1;
  for (int k = cprev + 1; k <= c; ++k) off[k] = i;
  if (i == N - 1)
    for (int k = c + 1; k <= nc; ++k) off[k] = N;
}

__global__ __launch_bounds__(256) void km_counts_kernel(const int32_t* __restrict__ offsets,
                                                        int32_t* __restrict__ counts, int nc) {
  const int p = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c < nc) counts[(size_t)p * nc + c] = offsets[(size_t)p * (nc + 1) + c + 1] - offsets[(size_t)p * (nc + 1) + c];
}

// ------------------------------------------------------------------------------------
// list-ordered reductions.  A list is summed in blocks of KM_BLK rows: inside a block one fp32
// add per row in list order starting from +0, then the block sums are added in block order
// starting from block 0's.  One wave per block, lane l owns dims 2l and 2l+1.  Lists of at
// most KM_BLK rows (nearly all of them) are finished by their own wave.  A longer list (the first
// Lloyd iterations produce a few huge ones) is split into its blocks, which other waves of the same
// launch sum in parallel, and a second, small launch adds the block sums in order.
//
// Which wave sums which block needs no queue and no counter: block j of a long list that starts at
// list offset o owns slot 2 * (o / KM_BLK) + j of its problem.  Two long lists never share a slot (a
// list of more than KM_BLK rows ends at least as many whole blocks later as it has blocks beyond its
// first), slots stay below km_item_cap(N), and the owner of a slot, if it has one, is the last
// cluster whose offset is below KM_BLK * (slot / 2 + 1): every later list starts at or after the
// owner's end, which is not.  A wave given a slot finds that cluster by a 64-way search of the
// offsets and leaves when the cluster is short or has fewer blocks.
// ------------------------------------------------------------------------------------
#define KM_BLK 256

// Rows k0 .. k1-1 of a list added in list order.  Sixteen rows per round: the lanes fetch the round's
// member ids with one load, the ids are broadcast from the lanes, and the sixteen row loads are all
// in flight before the first add; a short last round adds +0 for its missing rows, which changes no
// sum.  (Two dependent round trips per sixteen rows instead of two per row for a list's tail.)
template <bool HALF>
__device__ __forceinline__ void km_sum_rows(const uint32_t* __restrict__ rp, const int32_t* __restrict__ mem, int k0,
                                            int k1, float& s0, float& s1) {
  const int lane = threadIdx.x & 63;
  for (int k = k0; k < k1; k += 16) {
    const int n = min(16, k1 - k);
    const int id = (lane < n) ? mem[k + lane] : 0;
    uint32_t v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int r = __builtin_amdgcn_readlane(id, j);
      v[j] = (j < n) ? rp[(size_t)r * (RI_DIM / 2)] : 0u;
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      float x0, x1;
      ri_unpack2<HALF>(v[j], x0, x1);   // a missing row reads as the word 0 = (+0, +0) in either type
      s0 += x0;
      s1 += x1;
    }
  }
}

template <bool MEAN, bool HALF>
__device__ __forceinline__ void km_finish(float s0, float s1, int count, int normalize, uint32_t* op) {
  if (MEAN) {
    const float cnt = (float)count;
    s0 = s0 / cnt;
    s1 = s1 / cnt;
    if (normalize) {
      float sq = s0 * s0 + s1 * s1;  // two roundings: built without fp contraction
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
      const float nrm = sqrtf(sq);
      s0 = s0 / nrm;
      s1 = s1 / nrm;
    }
  }
  *op = (uint32_t)ri_f32_to_e16<HALF>(s0) | ((uint32_t)ri_f32_to_e16<HALF>(s1) << 16);
}

// slots of one problem: the last list starts below N and a slot index is at most 2 (N / KM_BLK) + 1
static inline int km_item_cap(int N) { return 2 * (N / KM_BLK) + 2; }

// The long list that owns `slot`, found by the whole wave: returns its cluster (or -1), its length
// in s, its list offset in o and the block of it that the slot stands for in j.
// off[0 .. nc] ascending, off[0] = 0.
__device__ __forceinline__ int km_slot_owner(const int32_t* __restrict__ off, int nc, int slot, int& s, int& o,
                                             int& j) {
  const int lane = threadIdx.x & 63;
  const int limit = KM_BLK * (slot / 2 + 1);
  // last index in [0, nc) whose offset is below limit: narrow [lo, lo + len) 64 ways per round
  int lo = 0, len = nc;
  while (len > 1) {
    const int stride = (len + 63) / 64;
    const int i = lo + lane * stride;
    const bool below = (i < lo + len) && off[i] < limit;
    const int k = __popcll(__ballot(below));   // probes are ascending: the first k are below (k >= 1)
    const int nlo = lo + (k - 1) * stride;
    len = min(stride, lo + len - nlo);
    lo = nlo;
  }
  o = off[lo];
  s = off[lo + 1] - o;
  j = slot - 2 * (o / KM_BLK);
  if (s <= KM_BLK || j < 0 || j >= (s + KM_BLK - 1) / KM_BLK) return -1;
  return lo;
}

// grid (item workgroups + ceil(nc / 4), P), four waves each.  The first item_wgs workgroups take
// one slot per wave (blocks of long lists, their fp32 sums go to partial[p][slot]); the others one
// cluster per wave.
template <bool MEAN, bool HALF>
__global__ __launch_bounds__(256) void km_reduce_kernel(const uint16_t* __restrict__ rows,
                                                        const int32_t* __restrict__ counts,
                                                        const int32_t* __restrict__ offsets,
                                                        const int32_t* __restrict__ members,
                                                        uint16_t* __restrict__ out, float2* __restrict__ partial,
                                                        int item_wgs, int cap, int N, int nc, int seg,
                                                        int64_t head_rows, int normalize) {
  const int p = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int32_t* off = offsets + (size_t)p * (nc + 1);
  const uint32_t* rp = reinterpret_cast<const uint32_t*>(rows + km_row0(p, seg, head_rows, N) * RI_DIM) + lane;
  if ((int)blockIdx.x < item_wgs) {
    const int slot = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (slot >= cap) return;
    int s, o, j;
    if (km_slot_owner(off, nc, slot, s, o, j) < 0) return;
    float s0 = 0.f, s1 = 0.f;
    km_sum_rows<HALF>(rp, members + (size_t)p * N + o, j * KM_BLK, min(s, (j + 1) * KM_BLK), s0, s1);
    partial[((size_t)p * cap + slot) * 64 + lane] = make_float2(s0, s1);
    return;
  }
  const int c = ((int)blockIdx.x - item_wgs) * 4 + (threadIdx.x >> 6);
  if (c >= nc) return;
  const int s = counts[(size_t)p * nc + c];
  uint32_t* op = reinterpret_cast<uint32_t*>(out + ((size_t)p * nc + c) * RI_DIM) + lane;
  if (s == 0) {
    if (!MEAN) *op = 0u;  // empty cluster: zero value sum; the centroid is left untouched
    return;
  }
  if (s > KM_BLK) return;  // summed by the slot waves, finished by km_reduce_fold_kernel
  float s0 = 0.f, s1 = 0.f;
  km_sum_rows<HALF>(rp, members + (size_t)p * N + off[c], 0, s, s0, s1);
  km_finish<MEAN, HALF>(s0, s1, s, normalize, op);
}

// grid (item workgroups, P): the wave of a long list's first slot adds the block sums in block
// order and finishes the cluster
template <bool MEAN, bool HALF>
__global__ __launch_bounds__(256) void km_reduce_fold_kernel(const int32_t* __restrict__ offsets,
                                                             const float2* __restrict__ partial,
                                                             uint16_t* __restrict__ out, int cap, int nc,
                                                             int normalize) {
  const int p = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int slot = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (slot >= cap) return;
  int s, o, j;
  const int c = km_slot_owner(offsets + (size_t)p * (nc + 1), nc, slot, s, o, j);
  if (c < 0 || j != 0) return;
  const int nb = (s + KM_BLK - 1) / KM_BLK;
  const float2* pp = partial + ((size_t)p * cap + slot) * 64 + lane;
  float2 t = pp[0];
  int b = 1;
  for (; b + 4 <= nb; b += 4) {
    float2 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = pp[(size_t)(b + u) * 64];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      t.x += v[u].x;
      t.y += v[u].y;
    }
  }
  for (; b < nb; ++b) {
    const float2 v = pp[(size_t)b * 64];
    t.x += v.x;
    t.y += v.y;
  }
  uint32_t* op = reinterpret_cast<uint32_t*>(out + ((size_t)p * nc + c) * RI_DIM) + lane;
  km_finish<MEAN, HALF>(t.x, t.y, s, normalize, op);
}

// out[p, i, :] = in[p, members[p, i], :]; 16 lanes per row
__global__ __launch_bounds__(256) void km_permute_kernel(const uint4* __restrict__ in,
                                                         const int32_t* __restrict__ members,
                                                         uint4* __restrict__ out, int N, int64_t in_stride,
                                                         int64_t out_stride) {
  const int p = blockIdx.y;
  const int i = blockIdx.x * 16 + (threadIdx.x >> 4);
  const int piece = threadIdx.x & 15;
  if (i >= N) return;
  const int32_t src = members[(size_t)p * N + i];
  out[((size_t)p * out_stride + i) * 16 + piece] = in[((size_t)p * in_stride + src) * 16 + piece];
}

// ------------------------------------------------------------------------------------
// C entry points
// ------------------------------------------------------------------------------------
static int km_check(int P, int N, int nc) {
  if (P <= 0 || N <= 0 || nc <= 0 || P > 65535) return RI_ERR_ARG;
  return RI_OK;
}

static int km_sort_chunks(int N) { return (N + KM_SORT_CHUNK - 1) / KM_SORT_CHUNK; }

// digit widths of the list sort: one pass when the cluster ids fit 9 bits, else two of about half each
static void km_sort_bits(int nc, int& lo_bits, int& hi_bits) {
  int total_bits = 1;
  while ((1 << total_bits) < nc) ++total_bits;
  lo_bits = total_bits <= 9 ? total_bits : (total_bits + 1) / 2;
  hi_bits = total_bits - lo_bits;
}

static int km_assign_args(const void* data, const void* centroids, const int32_t* assign, int P, int N, int nc,
                          int seg) {
  if (!data || !centroids || !assign) return RI_ERR_ARG;
  if (ri_any_misaligned16(data, centroids)) return RI_ERR_ARG;
  int rc = km_check(P, N, nc);
  if (rc) return rc;
  if (nc % 32 != 0 || seg <= 0 || P % seg != 0) return RI_ERR_ARG;
  return RI_OK;
}

template <bool HALF>
static int km_assign(const void* data, const void* centroids, int32_t* assign, int P, int N, int nc, int seg,
                     int64_t head_rows, ri_stream_t stream) {
  int rc = km_assign_args(data, centroids, assign, P, N, nc, seg);
  if (rc) return rc;
  if (nc > KM_WIDE_MIN_NC) {
    constexpr int wg_tokens = KM_WAVES * 32 * 4;
    km_assign_kernel<4, 128, HALF><<<dim3((N + wg_tokens - 1) / wg_tokens, P), KM_WAVES * 64, 0, (hipStream_t)stream>>>(
        (const uint16_t*)data, (const uint16_t*)centroids, assign, N, nc, seg, head_rows);
  } else {
    constexpr int wg_tokens = KM_WAVES * 32 * 2;
    km_assign_kernel<2, 32, HALF><<<dim3((N + wg_tokens - 1) / wg_tokens, P), KM_WAVES * 64, 0, (hipStream_t)stream>>>(
        (const uint16_t*)data, (const uint16_t*)centroids, assign, N, nc, seg, head_rows);
  }
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" int ri_kmeans_assign(const void* data, const void* centroids, int32_t* assign, int P, int N,
                                int nc, int seg, int64_t head_rows, ri_stream_t stream) {
  return km_assign<false>(data, centroids, assign, P, N, nc, seg, head_rows, stream);
}

extern "C" int ri_kmeans_assign_f16(const void* data, const void* centroids, int32_t* assign, int P, int N,
                                    int nc, int seg, int64_t head_rows, ri_stream_t stream) {
  return km_assign<true>(data, centroids, assign, P, N, nc, seg, head_rows, stream);
}

extern "C" size_t ri_kmeans_workspace_bytes(int P, int N, int nc) {
  if (P <= 0 || N <= 0 || nc <= 0) return 0;
  // digit table [P, 512, chunks] + one (key, token) staging pair [P, N] for the two-pass case
  return ((size_t)P * KM_SORT_MAX_BINS * km_sort_chunks(N) + 2 * (size_t)P * N) * sizeof(int32_t);
}

static int km_build_lists(const int32_t* assign, int32_t* counts, int32_t* offsets, int32_t* members, int P, int N,
                          int nc, void* workspace, hipStream_t s) {
  const int nchunks = km_sort_chunks(N);
  int32_t* chunk_hist = (int32_t*)workspace;
  int32_t* tmp_key = chunk_hist + (size_t)P * KM_SORT_MAX_BINS * nchunks;
  int32_t* tmp_tok = tmp_key + (size_t)P * N;
  int lo_bits, hi_bits;
  km_sort_bits(nc, lo_bits, hi_bits);
  if (hi_bits == 0 && N <= KM_SMALL_MAX) {
    km_sort_small_kernel<<<P, KM_SMALL_WAVES * 64, 0, s>>>(assign, offsets, counts, members, N, nc, lo_bits);
    RI_HIP_CHECK_LAUNCH();
    return RI_OK;
  }
  const dim3 cgrid((nchunks + 3) / 4, P);
  // pass over the low digit (the only one when the ids fit 9 bits)
  km_sort_hist_kernel<<<cgrid, 256, 0, s>>>(assign, chunk_hist, N, nchunks, 0, lo_bits);
  RI_HIP_CHECK_LAUNCH();
  // one pass and no cluster id beyond nc: the scan itself yields offsets and counts
  const bool direct = hi_bits == 0;
  km_sort_scan_kernel<<<P, 1024, 0, s>>>(chunk_hist, (1 << lo_bits) * nchunks, direct ? offsets : nullptr,
                                         direct ? counts : nullptr, nchunks, nc, N);
  RI_HIP_CHECK_LAUNCH();
  km_sort_scatter_kernel<<<cgrid, 256, 0, s>>>(assign, nullptr, chunk_hist, hi_bits ? tmp_key : nullptr,
                                               hi_bits ? tmp_tok : members, N, nchunks, 0, lo_bits);
  RI_HIP_CHECK_LAUNCH();
  if (hi_bits) {
    km_sort_hist_kernel<<<cgrid, 256, 0, s>>>(tmp_key, chunk_hist, N, nchunks, lo_bits, hi_bits);
    RI_HIP_CHECK_LAUNCH();
    km_sort_scan_kernel<<<P, 1024, 0, s>>>(chunk_hist, (1 << hi_bits) * nchunks, nullptr, nullptr, nchunks, nc, N);
    RI_HIP_CHECK_LAUNCH();
    km_sort_scatter_kernel<<<cgrid, 256, 0, s>>>(tmp_key, tmp_tok, chunk_hist, nullptr, members, N, nchunks,
                                                 lo_bits, hi_bits);
    RI_HIP_CHECK_LAUNCH();
  }
  if (!direct) {
    km_bounds_kernel<<<dim3((N + 255) / 256, P), 256, 0, s>>>(assign, members, offsets, N, nc);
    RI_HIP_CHECK_LAUNCH();
    km_counts_kernel<<<dim3((nc + 255) / 256, P), 256, 0, s>>>(offsets, counts, nc);
    RI_HIP_CHECK_LAUNCH();
  }
  return RI_OK;
}

static int km_lists_args(const int32_t* assign, const int32_t* counts, const int32_t* offsets, const int32_t* members,
                         int P, int N, int nc, const void* workspace, size_t workspace_bytes) {
  if (!assign || !counts || !offsets || !members || !workspace) return RI_ERR_ARG;
  int rc = km_check(P, N, nc);
  if (rc) return rc;
  if (nc > (1 << 18)) return RI_ERR_ARG;  // two passes of at most 9 bits
  if (workspace_bytes < ri_kmeans_workspace_bytes(P, N, nc)) return RI_ERR_WORKSPACE;
  return RI_OK;
}

extern "C" int ri_kmeans_build_lists(const int32_t* assign, int32_t* counts, int32_t* offsets,
                                     int32_t* members, int P, int N, int nc, void* workspace,
                                     size_t workspace_bytes, ri_stream_t stream) {
  int rc = km_lists_args(assign, counts, offsets, members, P, N, nc, workspace, workspace_bytes);
  if (rc) return rc;
  return km_build_lists(assign, counts, offsets, members, P, N, nc, workspace, (hipStream_t)stream);
}

extern "C" size_t ri_kmeans_reduce_workspace_bytes(int P, int N, int nc) {
  if (P <= 0 || N <= 0 || nc <= 0) return 0;
  // partial [P, cap, 128] fp32
  return (size_t)P * (size_t)km_item_cap(N) * RI_DIM * sizeof(float) + 256;
}

template <bool MEAN, bool HALF>
static int km_reduce(const void* rows, const int32_t* counts, const int32_t* offsets, const int32_t* members,
                     void* out, int P, int N, int nc, int seg, int64_t head_rows, int normalize, void* workspace,
                     size_t workspace_bytes, hipStream_t s) {
  if (workspace_bytes < ri_kmeans_reduce_workspace_bytes(P, N, nc)) return RI_ERR_WORKSPACE;
  const int cap = km_item_cap(N);
  float2* partial = (float2*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  const int item_wgs = (cap + 3) / 4;
  if ((long long)item_wgs + (nc + 3) / 4 > 0x7fffffffLL) return RI_ERR_ARG;
  km_reduce_kernel<MEAN, HALF><<<dim3(item_wgs + (nc + 3) / 4, P), 256, 0, s>>>(
      (const uint16_t*)rows, counts, offsets, members, (uint16_t*)out, partial, item_wgs, cap, N, nc, seg, head_rows,
      normalize);
  RI_HIP_CHECK_LAUNCH();
  km_reduce_fold_kernel<MEAN, HALF><<<dim3(item_wgs, P), 256, 0, s>>>(offsets, partial, (uint16_t*)out, cap, nc,
                                                                      normalize);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

template <bool HALF>
static int km_update(const void* data, const int32_t* counts, const int32_t* offsets, const int32_t* members,
                     void* centroids, int P, int N, int nc, int seg, int64_t head_rows, int normalize, void* workspace,
                     size_t workspace_bytes, ri_stream_t stream) {
  if (!data || !counts || !offsets || !members || !centroids || !workspace) return RI_ERR_ARG;
  if (ri_any_misaligned16(data, centroids, workspace)) return RI_ERR_ARG;
  int rc = km_check(P, N, nc);
  if (rc) return rc;
  if (seg <= 0 || P % seg != 0) return RI_ERR_ARG;
  return km_reduce<true, HALF>(data, counts, offsets, members, centroids, P, N, nc, seg, head_rows, normalize,
                               workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int ri_kmeans_update(const void* data, const int32_t* counts, const int32_t* offsets,
                                const int32_t* members, void* centroids, int P, int N, int nc, int seg,
                                int64_t head_rows, int normalize, void* workspace, size_t workspace_bytes,
                                ri_stream_t stream) {
  return km_update<false>(data, counts, offsets, members, centroids, P, N, nc, seg, head_rows, normalize, workspace,
                          workspace_bytes, stream);
}

extern "C" int ri_kmeans_update_f16(const void* data, const int32_t* counts, const int32_t* offsets,
                                    const int32_t* members, void* centroids, int P, int N, int nc, int seg,
                                    int64_t head_rows, int normalize, void* workspace, size_t workspace_bytes,
                                    ri_stream_t stream) {
  return km_update<true>(data, counts, offsets, members, centroids, P, N, nc, seg, head_rows, normalize, workspace,
                         workspace_bytes, stream);
}

template <bool HALF>
static int km_value_sum(const void* values, const int32_t* counts, const int32_t* offsets, const int32_t* members,
                        void* value_sum, int P, int N, int nc, void* workspace, size_t workspace_bytes,
                        ri_stream_t stream) {
  if (!values || !counts || !offsets || !members || !value_sum || !workspace) return RI_ERR_ARG;
  if (ri_any_misaligned16(values, value_sum, workspace)) return RI_ERR_ARG;
  int rc = km_check(P, N, nc);
  if (rc) return rc;
  return km_reduce<false, HALF>(values, counts, offsets, members, value_sum, P, N, nc, 1, (int64_t)N, 0, workspace,
                                workspace_bytes, (hipStream_t)stream);
}

extern "C" int ri_kmeans_value_sum(const void* values, const int32_t* counts, const int32_t* offsets,
                                   const int32_t* members, void* value_sum, int P, int N, int nc, void* workspace,
                                   size_t workspace_bytes, ri_stream_t stream) {
  return km_value_sum<false>(values, counts, offsets, members, value_sum, P, N, nc, workspace, workspace_bytes, stream);
}

extern "C" int ri_kmeans_value_sum_f16(const void* values, const int32_t* counts, const int32_t* offsets,
                                       const int32_t* members, void* value_sum, int P, int N, int nc, void* workspace,
                                       size_t workspace_bytes, ri_stream_t stream) {
  return km_value_sum<true>(values, counts, offsets, members, value_sum, P, N, nc, workspace, workspace_bytes, stream);
}

extern "C" int ri_permute_rows(const void* in, const int32_t* members, void* out, int P, int N,
                               int64_t in_stride_rows, int64_t out_stride_rows, ri_stream_t stream) {
  if (!in || !members || !out || P <= 0 || N <= 0 || P > 65535 || in_stride_rows < N || out_stride_rows < N)
    return RI_ERR_ARG;
  if (ri_any_misaligned16(in, out)) return RI_ERR_ARG;
  km_permute_kernel<<<dim3((N + 15) / 16, P), 256, 0, (hipStream_t)stream>>>(
      (const uint4*)in, members, (uint4*)out, N, in_stride_rows, out_stride_rows);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
