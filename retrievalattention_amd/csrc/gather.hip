// Wave-buffer copy kernels (gfx950): 128-bit accesses, 16 lanes per 256-byte vector, so a
// 64-wide wave moves four vectors per instruction.  Semantics follow
// library/retroinfer/retroinfer_kernels/src/copy_kernel.cuh and gather_copy.cu; the index
// arrays may live in pinned host memory, as in the reference.
#include "ri_common.h"

#define PAGE 8                       // vectors per cache block (reference CHUNK_SIZE)
#define VEC_U4 (RI_DIM * 2 / 16)     // 16-byte pieces per vector

// dst[g, i] = src[g, idx[g, copy_start + i]]; grid (ceil(copy_num/16), groups), 256 threads
__global__ __launch_bounds__(256) void gather_vectors_kernel(
    const uint4* __restrict__ src_k, uint4* __restrict__ dst_k, const uint4* __restrict__ src_v,
    uint4* __restrict__ dst_v, const uint16_t* __restrict__ src_m, uint16_t* __restrict__ dst_m,
    const int64_t* __restrict__ idx, int data_length, int buffer_length, int index_size, int copy_start,
    int copy_num) {
  const int g = blockIdx.y;
  const int i = blockIdx.x * 16 + (threadIdx.x >> 4);
  const int piece = threadIdx.x & 15;
  if (i >= copy_num) return;
  const int64_t s = idx[(size_t)g * index_size + copy_start + i];
  const size_t so = ((size_t)g * data_length + s) * VEC_U4 + piece;
  const size_t dofs = ((size_t)g * buffer_length + i) * VEC_U4 + piece;
  dst_k[dofs] = src_k[so];
  dst_v[dofs] = src_v[so];
  if (piece == 0) dst_m[(size_t)g * buffer_length + i] = src_m[(size_t)g * data_length + s];
}

// One item = up to 8 consecutive vectors; half a workgroup (128 threads) moves one item.
__device__ __forceinline__ void copy_item(const uint4* __restrict__ sk, uint4* __restrict__ dk,
                                          const uint4* __restrict__ sv, uint4* __restrict__ dv, size_t src_vec,
                                          size_t dst_vec, int nvec, int t128) {
  const int vec = t128 >> 4, piece = t128 & 15;
  if (vec < nvec) {
    const size_t so = (src_vec + vec) * VEC_U4 + piece;
    const size_t d = (dst_vec + vec) * VEC_U4 + piece;
    dk[d] = sk[so];
    dv[d] = sv[so];
  }
}

// grid (X, groups).  Items of a group: ceil(copy1/8) pieces of src1, then the src2 blocks, then
// the src3 blocks; workgroup x takes item pairs x, x+X, ...
__global__ __launch_bounds__(256) void concat_gather_kernel(
    const uint4* __restrict__ k1, const uint4* __restrict__ k2, const uint4* __restrict__ k3,
    uint4* __restrict__ kd, const uint4* __restrict__ v1, const uint4* __restrict__ v2,
    const uint4* __restrict__ v3, uint4* __restrict__ vd, const int32_t* __restrict__ off2,
    const int32_t* __restrict__ sizes2, const int32_t* __restrict__ dst2, const int32_t* __restrict__ num2,
    const int32_t* __restrict__ off3, const int32_t* __restrict__ sizes3, const int32_t* __restrict__ dst3,
    const int32_t* __restrict__ num3, int32_t* __restrict__ valid_lengths, int len1, int len2, int len3,
    int buffer_length, int offset_length, int copy1) {
  const int g = blockIdx.y;
  const int n2 = num2[g], n3 = num3[g];
  const size_t ib = (size_t)g * offset_length;
  const int total2 = n2 ? dst2[ib + n2 - 1] + sizes2[ib + n2 - 1] : 0;
  const int items1 = (copy1 + PAGE - 1) / PAGE;
  const int items = items1 + n2 + n3;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    const int total3 = n3 ? dst3[ib + n3 - 1] + sizes3[ib + n3 - 1] : 0;
    valid_lengths[g] = copy1 + total2 + total3;
  }
  const int half = threadIdx.x >> 7, t128 = threadIdx.x & 127;
  const size_t dbase = (size_t)g * buffer_length;
  for (int it = blockIdx.x * 2 + half; it < items; it += gridDim.x * 2) {
    if (it < items1) {
      const int v0 = it * PAGE;
      copy_item(k1, kd, v1, vd, (size_t)g * len1 + v0, dbase + v0, min(PAGE, copy1 - v0), t128);
    } else if (it < items1 + n2) {
      const int j = it - items1;
      copy_item(k2, kd, v2, vd, (size_t)g * len2 + off2[ib + j], dbase + copy1 + dst2[ib + j], sizes2[ib + j],
                t128);
    } else {
      const int j = it - items1 - n2;
      copy_item(k3, kd, v3, vd, ((size_t)g * len3 + off3[ib + j]) * PAGE, dbase + copy1 + total2 + dst3[ib + j],
                sizes3[ib + j], t128);
    }
  }
}

// grid (X, groups): cache[g, dst_block[j], 0:sizes[j]] = src[g, start + src_off[j] : +sizes[j]]
__global__ __launch_bounds__(256) void scatter_kernel(const uint4* __restrict__ ks, uint4* __restrict__ kc,
                                                      const uint4* __restrict__ vs, uint4* __restrict__ vc,
                                                      const int32_t* __restrict__ src_off,
                                                      const int32_t* __restrict__ sizes,
                                                      const int32_t* __restrict__ dst_block,
                                                      const int32_t* __restrict__ num, int data_length,
                                                      int buffer_length, int offset_length, int start) {
  const int g = blockIdx.y;
  const int n = num[g];
  const size_t ib = (size_t)g * offset_length;
  const int half = threadIdx.x >> 7, t128 = threadIdx.x & 127;
  for (int j = blockIdx.x * 2 + half; j < n; j += gridDim.x * 2)
    copy_item(ks, kc, vs, vc, (size_t)g * data_length + start + src_off[ib + j],
              ((size_t)g * buffer_length + dst_block[ib + j]) * PAGE, sizes[ib + j], t128);
}

extern "C" int ri_gather_copy_vectors(const void* src_keys, void* dst_keys, const void* src_values,
                                      void* dst_values, const void* src_meta, void* dst_meta,
                                      const int64_t* idx, int groups, int data_length, int buffer_length,
                                      int index_size, int copy_start, int copy_num, ri_stream_t stream) {
  if (!src_keys || !dst_keys || !src_values || !dst_values || !src_meta || !dst_meta || !idx) return RI_ERR_ARG;
  if (ri_any_misaligned16(src_keys, dst_keys, src_values, dst_values)) return RI_ERR_ARG;
  if (groups <= 0 || copy_num < 0 || copy_start < 0 || copy_start + copy_num > index_size ||
      copy_num > buffer_length)
    return RI_ERR_ARG;
  if (copy_num == 0) return RI_OK;
  gather_vectors_kernel<<<dim3((copy_num + 15) / 16, groups), 256, 0, (hipStream_t)stream>>>(
      (const uint4*)src_keys, (uint4*)dst_keys, (const uint4*)src_values, (uint4*)dst_values,
      (const uint16_t*)src_meta, (uint16_t*)dst_meta, idx, data_length, buffer_length, index_size, copy_start,
      copy_num);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" int ri_gather_copy_and_concat(const void* k1, const void* k2, const void* k3, void* kdst,
                                         const void* v1, const void* v2, const void* v3, void* vdst,
                                         const int32_t* off2, const int32_t* sizes2, const int32_t* dst2,
                                         const int32_t* num2, const int32_t* off3, const int32_t* sizes3,
                                         const int32_t* dst3, const int32_t* num3, int32_t* valid_lengths,
                                         int groups, int data_length1, int data_length2, int data_length3,
                                         int buffer_length, int offset_length, int copy_vectors1,
                                         ri_stream_t stream) {
  if (!k1 || !k2 || !k3 || !kdst || !v1 || !v2 || !v3 || !vdst || !off2 || !sizes2 || !dst2 || !num2 ||
      !off3 || !sizes3 || !dst3 || !num3 || !valid_lengths)
    return RI_ERR_ARG;
  if (ri_any_misaligned16(k1, k2, k3, kdst, v1, v2, v3, vdst)) return RI_ERR_ARG;
  if (groups <= 0 || copy_vectors1 < 0 || copy_vectors1 > data_length1 || copy_vectors1 > buffer_length ||
      offset_length <= 0)
    return RI_ERR_ARG;
  int x = (copy_vectors1 / PAGE + 2 * offset_length) / 8 + 1;
  if (x > 64) x = 64;
  concat_gather_kernel<<<dim3(x, groups), 256, 0, (hipStream_t)stream>>>(
      (const uint4*)k1, (const uint4*)k2, (const uint4*)k3, (uint4*)kdst, (const uint4*)v1, (const uint4*)v2,
      (const uint4*)v3, (uint4*)vdst, off2, sizes2, dst2, num2, off3, sizes3, dst3, num3, valid_lengths,
      data_length1, data_length2, data_length3, buffer_length, offset_length, copy_vectors1);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" int ri_gather_copy_and_scatter(const void* ksrc, void* kcache, const void* vsrc, void* vcache,
                                          const int32_t* src_off, const int32_t* sizes,
                                          const int32_t* dst_block, const int32_t* num, int groups,
                                          int data_length, int buffer_length, int offset_length,
                                          int s_copy_start, ri_stream_t stream) {
  if (!ksrc || !kcache || !vsrc || !vcache || !src_off || !sizes || !dst_block || !num) return RI_ERR_ARG;
  if (ri_any_misaligned16(ksrc, kcache, vsrc, vcache)) return RI_ERR_ARG;
  if (groups <= 0 || offset_length <= 0 || s_copy_start < 0) return RI_ERR_ARG;
  int x = offset_length / 8 + 1;
  if (x > 32) x = 32;
  scatter_kernel<<<dim3(x, groups), 256, 0, (hipStream_t)stream>>>(
      (const uint4*)ksrc, (uint4*)kcache, (const uint4*)vsrc, (uint4*)vcache, src_off, sizes, dst_block, num,
      data_length, buffer_length, offset_length, s_copy_start);
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}
