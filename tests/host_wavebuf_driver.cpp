// Stand-alone driver of the host wave buffer (csrc/wavebuf.cpp) for sanitizer builds: a random workload over
// every entry point — pool creation, index and K/V registration, construction per batch, many access/update
// steps with the update running behind the caller, a decode-time update_kv, destruction — with the
// block cache invariants checked along the way.  tests/test_wavebuf_sanitizers.py compiles this file together
// with wavebuf.cpp under -fsanitize=thread and -fsanitize=address,undefined and runs it (host code only).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>

#include "retro_mi355.h"

#define REQUIRE(x)                                                   \
  do {                                                               \
    if (!(x)) {                                                      \
      std::fprintf(stderr, "check failed at line %d: %s\n", __LINE__, #x); \
      return 1;                                                      \
    }                                                                \
  } while (0)

static uint64_t rng_state = 0x9e3779b97f4a7c15ULL;
static uint32_t rnd() {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return (uint32_t)(rng_state >> 16);
}

int main(int argc, char** argv) {
  const int threads = argc > 1 ? std::atoi(argv[1]) : 4;
  const int B = 2, H = 3, BG = B * H, dim = 128, block = 8;
  const int nc = 40, extra = 8, final_nc = nc + extra, nprobe = 6, buffer_size = 48, capacity = 20;
  const int n_tokens = 700, out_len = 1024, in_len = 800, steps = 300;

  ri_threadpool* pool = ri_threadpool_create(threads);
  REQUIRE(pool != nullptr);
  ri_wavebuf* wb = ri_wavebuf_create(B, H, dim, nprobe, block, nc, final_nc, buffer_size, capacity, threads, pool);
  REQUIRE(wb != nullptr);
  REQUIRE(ri_wavebuf_batch_access(wb) != 0);   // nothing registered yet: an error, not a crash

  std::vector<int32_t> lists[12];
  for (int i = 0; i < 12; ++i) lists[i].assign((i % 4 == 3) ? BG : (size_t)BG * buffer_size, 0);
  std::vector<int64_t> searched((size_t)BG * nprobe, 0);
  REQUIRE(ri_wavebuf_set_indices(wb, lists[0].data(), lists[1].data(), lists[2].data(), lists[3].data(), lists[4].data(),
                                 lists[5].data(), lists[6].data(), lists[7].data(), lists[8].data(), lists[9].data(),
                                 lists[10].data(), lists[11].data(), searched.data()) == 0);
  std::vector<uint16_t> ivf_k((size_t)BG * out_len * dim, 0), ivf_v((size_t)BG * out_len * dim, 0);
  std::vector<uint16_t> in_k((size_t)H * in_len * dim), in_v((size_t)H * in_len * dim);
  REQUIRE(ri_wavebuf_set_kv(wb, ivf_k.data(), ivf_v.data(), out_len, in_k.data(), in_v.data(), in_len) == 0);

  // construction: a random clustering per sequence; row r of the input carries its own index in element 0
  std::vector<int32_t> sizes_all((size_t)BG * final_nc, 0);
  for (int b = 0; b < B; ++b) {
    for (size_t i = 0; i < in_k.size(); ++i) {
      in_k[i] = (uint16_t)((i / dim) % in_len);
      in_v[i] = (uint16_t)(((i / dim) % in_len) ^ 0x5555);
    }
    std::vector<int32_t> assign((size_t)H * n_tokens), sizes((size_t)H * nc, 0);
    for (int h = 0; h < H; ++h)
      for (int t = 0; t < n_tokens; ++t) {
        int c = (int)(rnd() % nc);
        if (c == 7) c = 8;   // one cluster stays empty
        assign[(size_t)h * n_tokens + t] = c;
        ++sizes[(size_t)h * nc + c];
      }
    int mx = 1;
    for (int32_t s : sizes) mx = s > mx ? s : mx;
    std::vector<int32_t> cl((size_t)H * nc * mx, 0), fill((size_t)H * nc, 0);
    for (int h = 0; h < H; ++h)
      for (int t = 0; t < n_tokens; ++t) {
        const int c = assign[(size_t)h * n_tokens + t];
        cl[((size_t)h * nc + c) * mx + fill[(size_t)h * nc + c]++] = t;
      }
    REQUIRE(ri_wavebuf_async_construction(wb, cl.data(), sizes.data(), mx, b) == 0);
    REQUIRE(ri_wavebuf_construction_sync(wb) == 0);
    for (int h = 0; h < H; ++h) {
      const int g = b * H + h;
      int row = 0;
      for (int c = 0; c < nc; ++c) {
        sizes_all[(size_t)g * final_nc + c] = sizes[(size_t)h * nc + c];
        for (int i = 0; i < sizes[(size_t)h * nc + c]; ++i, ++row) {
          const int tok = cl[((size_t)h * nc + c) * mx + i];
          REQUIRE(ivf_k[((size_t)g * out_len + row) * dim] == (uint16_t)tok);
          REQUIRE(ivf_v[((size_t)g * out_len + row) * dim + dim - 1] == (uint16_t)(tok ^ 0x5555));
        }
      }
    }
  }

  int ncl = nc;
  long hits = 0, misses = 0;
  for (int step = 0; step < steps; ++step) {
    if (step == steps / 2) {   // decode-time growth: eight new clusters of 1..6 tokens behind the prompt's
      const int un = 40;
      std::vector<uint16_t> uk((size_t)BG * un * dim, 7), uv((size_t)BG * un * dim, 9);
      std::vector<int32_t> usz((size_t)BG * extra), ucl((size_t)BG * extra * 6, 0);
      for (int g = 0; g < BG; ++g) {
        int t = 0;
        for (int c = 0; c < extra; ++c) {
          const int s = 1 + (int)(rnd() % 6);
          usz[(size_t)g * extra + c] = (t + s <= un) ? s : 0;
          for (int i = 0; i < usz[(size_t)g * extra + c]; ++i) ucl[((size_t)g * extra + c) * 6 + i] = t++;
          sizes_all[(size_t)g * final_nc + nc + c] = usz[(size_t)g * extra + c];
        }
      }
      REQUIRE(ri_wavebuf_sync(wb) == 0);
      REQUIRE(ri_wavebuf_update_kv(wb, uk.data(), uv.data(), un, ucl.data(), usz.data(), extra, 6) == 0);
      ncl = final_nc;
    }
    for (int g = 0; g < BG; ++g) {
      std::set<int> used;
      for (int r = 0; r < nprobe; ++r) {
        int c;
        do {   // a hot set of twelve clusters plus the long tail
          const int range = (rnd() % 3) ? 12 : ncl;
          c = (int)(rnd() % range);
        } while (used.count(c));
        used.insert(c);
        searched[(size_t)g * nprobe + r] = c;
      }
    }
    REQUIRE(ri_wavebuf_batch_access(wb) == 0);
    // the lists of this step are complete here; the cache update still runs on the workers
    for (int g = 0; g < BG; ++g) {
      const int nh = lists[3][g], nm = lists[7][g];
      REQUIRE(nh >= 0 && nm >= 0 && nh + nm <= buffer_size);
      int blocks = 0;
      for (int r = 0; r < nprobe; ++r)
        blocks += (sizes_all[(size_t)g * final_nc + searched[(size_t)g * nprobe + r]] + block - 1) / block;
      REQUIRE(nh + nm == blocks);   // buffer_size is large enough here: nothing is cut off
      std::set<int> ids;
      for (int i = 0; i < nh; ++i) {
        const int id = lists[0][(size_t)g * buffer_size + i];
        REQUIRE(id >= 0 && id < capacity && ids.insert(id).second);
      }
      hits += nh;
      misses += nm;
    }
    if (step % 3 != 2) REQUIRE(ri_wavebuf_sync(wb) == 0);   // sometimes the next access finds the update still running
    for (int g = 0; g < BG && step % 3 != 2; ++g) {
      const int nu = lists[11][g];
      REQUIRE(nu >= 0 && nu <= capacity);
      std::set<int> ids;
      for (int i = 0; i < nu; ++i) {
        const int id = lists[10][(size_t)g * buffer_size + i];
        REQUIRE(id >= 0 && id < capacity && ids.insert(id).second);
      }
    }
  }
  REQUIRE(ri_wavebuf_sync(wb) == 0);
  REQUIRE(hits > 0 && misses > 0);
  REQUIRE(ri_wavebuf_overflow_events(wb) == 0);
  ri_wavebuf_destroy(wb);
  ri_threadpool_destroy(pool);
  std::printf("ok: %ld block hits, %ld block misses over %d steps\n", hits, misses, steps);
  return 0;
}
