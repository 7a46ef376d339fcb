// A decode step through the C ABI from a plain HIP program: no Python, no torch.  This is what a
// cgo / JNI / pybind caller of include/retro_mi355.h does: device buffers of its own, ri_score_select, then
// ri_wave_attention (and the no-allocation variant), status codes checked.  The result of every group is
// compared with a direct fp64 evaluation of the same step on the host (cache_hub/retroinfer_cache.py:598-674:
// exact attention over the steady zone and the retrieved clusters, merged with the estimation zone), using
// the zones and logits the library reported.
// Built by `python -m retrievalattention_amd.build` into tests/capi_decode_step; run by tests/test_gpu_capi.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "retro_mi355.h"

#define HIP_OK(x)                                                                          \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      std::fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);  \
      return 2;                                                                            \
    }                                                                                      \
  } while (0)
#define RI_OK_(x)                                                                          \
  do {                                                                                     \
    int rc_ = (x);                                                                         \
    if (rc_ != 0) {                                                                        \
      std::fprintf(stderr, "%s at line %d\n", ri_status_string(rc_), __LINE__);            \
      return 3;                                                                            \
    }                                                                                      \
  } while (0)

static uint64_t rng_state = 0x243f6a8885a308d3ULL;
static double uniform() {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return ((rng_state >> 11) + 0.5) / 9007199254740992.0;
}
static float normal() { return (float)(std::sqrt(-2.0 * std::log(uniform())) * std::cos(6.283185307179586 * uniform())); }
static uint16_t to_bf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static double from_bf16(uint16_t b) {
  const uint32_t u = (uint32_t)b << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

template <typename T>
static T* to_device(const std::vector<T>& h) {
  T* d = nullptr;
  if (hipMalloc((void**)&d, h.size() * sizeof(T) + 16) != hipSuccess) return nullptr;
  if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return d;
}
template <typename T>
static T* device_zeros(size_t n) {
  T* d = nullptr;
  if (hipMalloc((void**)&d, n * sizeof(T) + 16) != hipSuccess) return nullptr;
  if (hipMemset(d, 0, n * sizeof(T)) != hipSuccess) return nullptr;
  return d;
}

int main() {
  const int BG = 6, gs = 4, D = 128, nc = 512, np = 9, es = 118, page = 8, max_pages = 72;
  const int static_len = 69, steady_stride = 80;
  const float scale = 1.0f / std::sqrt((float)D);
  if (ri_abi_version() < 6) return 4;

  // clusters of 8..24 tokens (one of them empty), K/V rows, centroids, value sums
  std::vector<int32_t> size((size_t)BG * nc), start((size_t)BG * nc);
  std::vector<uint8_t> mask((size_t)BG * nc);
  int64_t rows = 0;
  for (int g = 0; g < BG; ++g) {
    int64_t run = 0;
    for (int c = 0; c < nc; ++c) {
      const int s = (c == 17) ? 0 : 8 + (int)(uniform() * 17);
      size[(size_t)g * nc + c] = s;
      start[(size_t)g * nc + c] = (int32_t)run;
      mask[(size_t)g * nc + c] = s == 0;
      run += s;
    }
    rows = run > rows ? run : rows;
  }
  auto fill = [&](size_t n, float sc) {
    std::vector<uint16_t> v(n);
    for (auto& x : v) x = to_bf16(sc * normal());
    return v;
  };
  const std::vector<uint16_t> q = fill((size_t)BG * gs * D, 1.f), cent = fill((size_t)BG * nc * D, 1.5f),
                              vsum = fill((size_t)BG * nc * D, 4.f), sk = fill((size_t)BG * rows * D, 1.f),
                              sv = fill((size_t)BG * rows * D, 1.f), stk = fill((size_t)BG * steady_stride * D, 1.f),
                              stv = fill((size_t)BG * steady_stride * D, 1.f);
  std::vector<uint16_t> csize((size_t)BG * nc);
  for (size_t i = 0; i < csize.size(); ++i) csize[i] = to_bf16((float)size[i]);

  uint16_t *d_q = to_device(q), *d_cent = to_device(cent), *d_vsum = to_device(vsum), *d_sk = to_device(sk),
           *d_sv = to_device(sv), *d_stk = to_device(stk), *d_stv = to_device(stv), *d_csize = to_device(csize);
  int32_t *d_size = to_device(size), *d_start = to_device(start);
  uint8_t* d_mask = to_device(mask);
  float* d_logits = device_zeros<float>((size_t)BG * gs * nc);
  int32_t *d_ret = device_zeros<int32_t>((size_t)BG * np), *d_est = device_zeros<int32_t>((size_t)BG * es),
          *d_off = device_zeros<int32_t>((size_t)BG * (np + 1)), *d_rst = device_zeros<int32_t>((size_t)BG * np),
          *d_meta = device_zeros<int32_t>((size_t)BG * 4), *d_vl = device_zeros<int32_t>(BG);
  uint16_t *d_out = device_zeros<uint16_t>((size_t)BG * gs * D), *d_out2 = device_zeros<uint16_t>((size_t)BG * gs * D);
  const size_t ws1 = ri_score_select_workspace_bytes(BG, gs, nc), ws2 = ri_wave_attention_workspace_bytes(BG, gs);
  uint8_t *d_ws1 = device_zeros<uint8_t>(ws1), *d_ws2 = device_zeros<uint8_t>(ws2);   // zeroed once, as the header asks
  if (!d_q || !d_cent || !d_vsum || !d_sk || !d_sv || !d_stk || !d_stv || !d_csize || !d_size || !d_start || !d_mask ||
      !d_logits || !d_ret || !d_est || !d_off || !d_rst || !d_meta || !d_vl || !d_out || !d_out2 || !d_ws1 || !d_ws2)
    return 2;

  hipStream_t s;
  HIP_OK(hipStreamCreate(&s));
  // bad arguments come back as status codes, before anything is launched
  if (ri_score_select(d_q, d_cent, d_mask, d_size, d_start, d_logits, nullptr, nullptr, d_ret, d_est, d_off, d_rst, nullptr,
                      0, d_meta, BG, gs, nc, 5000, es, page, max_pages, scale, d_ws1, ws1, s) == 0)
    return 5;
  if (ri_score_select(d_q, d_cent, d_mask, d_size, d_start, d_logits, nullptr, nullptr, d_ret, d_est, d_off, d_rst, nullptr,
                      0, d_meta, BG, gs, nc, np, es, page, max_pages, scale, d_ws1, ws1 / 2, s) == 0)
    return 5;
  for (int rep = 0; rep < 2; ++rep) {   // twice on the same workspaces: they are left ready for the next call
    RI_OK_(ri_score_select(d_q, d_cent, d_mask, d_size, d_start, d_logits, nullptr, nullptr, d_ret, d_est, d_off, d_rst,
                           nullptr, 0, d_meta, BG, gs, nc, np, es, page, max_pages, scale, d_ws1, ws1, s));
    RI_OK_(ri_wave_attention(d_q, d_stk, d_stv, steady_stride, static_len, nullptr, d_sk, d_sv, rows, nullptr, 0, d_off,
                             d_rst, np, d_meta, d_est, d_logits, nullptr, d_vsum, d_csize, d_out, d_vl, BG, gs, nc, es,
                             scale, d_ws2, ws2, s));
  }
  RI_OK_(ri_wave_attention_static(d_q, d_stk, d_stv, steady_stride, static_len, nullptr, d_sk, d_sv, rows, nullptr, 0,
                                  d_off, d_rst, np, d_meta, d_est, d_logits, nullptr, d_vsum, d_csize, d_out2, d_vl, BG,
                                  gs, nc, es, scale, s));
  HIP_OK(hipStreamSynchronize(s));

  std::vector<uint16_t> out((size_t)BG * gs * D), out2(out.size());
  std::vector<float> logits((size_t)BG * gs * nc);
  std::vector<int32_t> ret((size_t)BG * np), est((size_t)BG * es), meta((size_t)BG * 4), vl(BG);
  HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(out2.data(), d_out2, out2.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(logits.data(), d_logits, logits.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(ret.data(), d_ret, ret.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(est.data(), d_est, est.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(meta.data(), d_meta, meta.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(vl.data(), d_vl, vl.size() * 4, hipMemcpyDeviceToHost));
  if (std::memcmp(out.data(), out2.data(), out.size() * 2) != 0) {
    std::fprintf(stderr, "the no-allocation entry point differs from the workspace one\n");
    return 6;
  }

  double max_abs = 0.0, sum_abs = 0.0;
  for (int g = 0; g < BG; ++g) {
    const int kept = meta[g * 4 + 0];
    int tokens = 0;
    for (int r = 0; r < kept; ++r) tokens += size[(size_t)g * nc + ret[(size_t)g * np + r]];
    if (kept != np || meta[g * 4 + 1] != tokens || vl[g] != static_len + tokens) {
      std::fprintf(stderr, "group %d: layout mismatch (%d kept, %d tokens, valid length %d)\n", g, kept, meta[g * 4 + 1], vl[g]);
      return 7;
    }
    for (int j = 0; j < gs; ++j) {
      const uint16_t* qj = &q[((size_t)g * gs + j) * D];
      // scores of every attended row: steady zone, retrieved clusters (exact), estimation zone (from the logits)
      std::vector<double> sc, wt;
      std::vector<const uint16_t*> val;
      auto add_row = [&](const uint16_t* k, const uint16_t* v) {
        double d = 0;
        for (int i = 0; i < D; ++i) d += from_bf16(qj[i]) * from_bf16(k[i]);
        sc.push_back(d * scale);
        wt.push_back(1.0);
        val.push_back(v);
      };
      for (int t = 0; t < static_len; ++t) add_row(&stk[((size_t)g * steady_stride + t) * D], &stv[((size_t)g * steady_stride + t) * D]);
      for (int r = 0; r < kept; ++r) {
        const int c = ret[(size_t)g * np + r];
        for (int t = 0; t < size[(size_t)g * nc + c]; ++t) {
          const size_t row = (size_t)g * rows + start[(size_t)g * nc + c] + t;
          add_row(&sk[row * D], &sv[row * D]);
        }
      }
      for (int e = 0; e < es; ++e) {
        const int c = est[(size_t)g * es + e];
        sc.push_back(logits[((size_t)g * gs + j) * nc + c]);
        wt.push_back(from_bf16(csize[(size_t)g * nc + c]));   // the denominator counts every token of the cluster
        val.push_back(&vsum[((size_t)g * nc + c) * D]);       // the numerator takes the cluster's value sum
      }
      double m = -1e300, den = 0;
      for (double x : sc) m = x > m ? x : m;
      std::vector<double> num(D, 0.0);
      for (size_t i = 0; i < sc.size(); ++i) {
        const double p = std::exp(sc[i] - m);
        den += p * wt[i];
        for (int d = 0; d < D; ++d) num[d] += p * from_bf16(val[i][d]);
      }
      for (int d = 0; d < D; ++d) {
        const double diff = std::fabs(num[d] / den - from_bf16(out[((size_t)g * gs + j) * D + d]));
        max_abs = diff > max_abs ? diff : max_abs;
        sum_abs += diff;
      }
    }
  }
  const double mean_abs = sum_abs / ((double)BG * gs * D);
  std::printf("decode step through the C ABI: max-abs %.3e, mean-abs %.3e against the host evaluation\n", max_abs, mean_abs);
  if (!(max_abs <= 2e-2 && mean_abs <= 2e-3)) return 8;   // the tolerance of the path's bf16 outputs
  HIP_OK(hipStreamDestroy(s));
  std::printf("ok\n");
  return 0;
}
