// Host side of the wave buffer: a small worker pool, the per-group LRU manager of the GPU
// block cache, and the re-organisation of K/V rows into cluster-contiguous host arrays.
// Behaviour follows library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp
// (descriptors :513-542, organise :545-567, access :190-257, update :102-188) and
// thread_pool.hpp; the data structures are this library's own: the LRU order is an
// index-linked list over cluster ids and free blocks are a stack, which makes the block ids
// handed out deterministic.
#include <sched.h>

#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

#include "../../include/retro_mi355.h"

namespace {

class WorkerPool {
 public:
  // first_core >= 0: worker i runs on core first_core + i only (thread_pool.hpp:18-23, 65-66 pins worker i
  // to core i); a core the process may not use leaves that worker unpinned
  explicit WorkerPool(int n, int first_core = -1) {
    if (n <= 0) n = (int)std::thread::hardware_concurrency();
    if (n <= 0) n = 1;
    for (int i = 0; i < n; ++i)
      workers_.emplace_back([this, i, first_core] {
        if (first_core >= 0) {
          cpu_set_t set;
          CPU_ZERO(&set);
          CPU_SET((first_core + i) % CPU_SETSIZE, &set);
          if (sched_setaffinity(0, sizeof(set), &set) == 0) pinned_.fetch_add(1);
        }
        ready_.fetch_add(1);
        loop();
      });
    while (ready_.load() < n) std::this_thread::yield();
  }
  int pinned() const { return pinned_.load(); }
  ~WorkerPool() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      stop_ = true;
    }
    cv_job_.notify_all();
    for (auto& t : workers_) t.join();
  }
  // enqueue a batch of jobs under one lock so that wait() cannot observe a partial batch
  void submit(std::vector<std::function<void()>> jobs) {
    {
      std::lock_guard<std::mutex> lk(mu_);
      pending_ += (int)jobs.size();
      for (auto& j : jobs) queue_.push_back(std::move(j));
    }
    cv_job_.notify_all();
  }
  void wait() {
    std::unique_lock<std::mutex> lk(mu_);
    cv_done_.wait(lk, [this] { return pending_ == 0; });
  }
  int size() const { return (int)workers_.size(); }

 private:
  std::atomic<int> pinned_{0}, ready_{0};
  void loop() {
    for (;;) {
      std::function<void()> job;
      {
        std::unique_lock<std::mutex> lk(mu_);
        cv_job_.wait(lk, [this] { return stop_ || !queue_.empty(); });
        if (stop_ && queue_.empty()) return;
        job = std::move(queue_.front());
        queue_.pop_front();
      }
      job();
      {
        std::lock_guard<std::mutex> lk(mu_);
        if (--pending_ == 0) cv_done_.notify_all();
      }
    }
  }
  std::mutex mu_;
  std::condition_variable cv_job_, cv_done_;
  std::deque<std::function<void()>> queue_;
  std::vector<std::thread> workers_;
  int pending_ = 0;
  bool stop_ = false;
};

// One group's view of the block cache.
struct GroupCache {
  int capacity = 0;
  int ncl = 0;  // clusters known so far
  // per cluster
  std::vector<int32_t> start, nblk, last, blk_off;
  std::vector<uint8_t> resident;
  std::vector<int32_t> lru_prev, lru_next;  // -1 terminated
  std::vector<int32_t> blk_ids;             // blk_off[c] .. +nblk[c]
  int32_t lru_head = -1, lru_tail = -1;     // head = most recent
  std::vector<int32_t> free_blocks;         // stack; top = back
  std::vector<int32_t> hit_keys, miss_keys;

  void init(int cap, int max_clusters) {
    capacity = cap;
    start.assign(max_clusters, 0);
    nblk.assign(max_clusters, 0);
    last.assign(max_clusters, 0);
    blk_off.assign(max_clusters, 0);
    resident.assign(max_clusters, 0);
    lru_prev.assign(max_clusters, -1);
    lru_next.assign(max_clusters, -1);
    free_blocks.resize(cap);
    for (int i = 0; i < cap; ++i) free_blocks[i] = cap - 1 - i;  // pops 0, 1, 2, ...
  }
  // append `n` clusters with the given sizes, laid out from row `row0`; returns the end row
  int64_t add_clusters(const int32_t* sizes, int n, int64_t row0, int block) {
    int64_t row = row0;
    size_t boff = blk_ids.size();
    for (int i = 0; i < n; ++i) {
      const int c = ncl + i;
      const int sz = sizes[i];
      start[c] = (int32_t)row;
      nblk[c] = (sz + block - 1) / block;
      last[c] = sz == 0 ? 0 : (sz % block == 0 ? block : sz % block);
      blk_off[c] = (int32_t)boff;
      resident[c] = 0;
      boff += (size_t)nblk[c];
      row += sz;
    }
    blk_ids.resize(boff, -1);
    ncl += n;
    return row;
  }
  void reset_clusters() {
    ncl = 0;
    blk_ids.clear();
  }
  void lru_unlink(int c) {
    const int p = lru_prev[c], n = lru_next[c];
    if (p >= 0) lru_next[p] = n; else lru_head = n;
    if (n >= 0) lru_prev[n] = p; else lru_tail = p;
  }
  void lru_push_front(int c) {
    lru_prev[c] = -1;
    lru_next[c] = lru_head;
    if (lru_head >= 0) lru_prev[lru_head] = c; else lru_tail = c;
    lru_head = c;
  }
  void evict_tail() {
    const int c = lru_tail;
    if (c < 0) return;
    lru_unlink(c);
    for (int j = nblk[c] - 1; j >= 0; --j) free_blocks.push_back(blk_ids[blk_off[c] + j]);
    resident[c] = 0;
  }
};

}  // namespace

struct ri_threadpool {
  WorkerPool pool;
  explicit ri_threadpool(int n, int first_core = -1) : pool(n, first_core) {}
};

struct ri_wavebuf {
  int batch_size, group_num, BG, dim, nprobe, block, n_centroids, final_n_centroids, buffer_size, capacity;
  int jobs, groups_per_job;
  WorkerPool* pool;
  std::vector<GroupCache> caches;
  std::vector<int64_t> seq_len;  // rows used in the cluster store, per group
  std::atomic<int64_t> overflow{0};
  // registered host arrays
  int32_t *hit_ids = nullptr, *hit_sizes = nullptr, *hit_cumsum = nullptr, *hit_nums = nullptr;
  int32_t *miss_ids = nullptr, *miss_sizes = nullptr, *miss_cumsum = nullptr, *miss_nums = nullptr;
  int32_t *upd_buf = nullptr, *upd_sizes = nullptr, *upd_cache = nullptr, *upd_nums = nullptr;
  int64_t* searched = nullptr;
  uint16_t *ivf_k = nullptr, *ivf_v = nullptr, *in_k = nullptr, *in_v = nullptr;
  int64_t out_len = 0, in_len = 0;

  void organize(int g, const uint16_t* keys, const uint16_t* vals, int64_t in_rows, const int32_t* lists,
                const int32_t* sizes, int n, int64_t max_cs, int64_t row0) {
    uint16_t* dk = ivf_k + (size_t)g * out_len * dim;
    uint16_t* dv = ivf_v + (size_t)g * out_len * dim;
    const size_t row_bytes = (size_t)dim * sizeof(uint16_t);
    int64_t row = row0;
    (void)in_rows;
    for (int c = 0; c < n; ++c) {
      const int32_t* ids = lists + (size_t)c * max_cs;
      for (int j = 0; j < sizes[c]; ++j, ++row) {
        std::memcpy(dk + (size_t)row * dim, keys + (size_t)ids[j] * dim, row_bytes);
        std::memcpy(dv + (size_t)row * dim, vals + (size_t)ids[j] * dim, row_bytes);
      }
    }
  }

  void access_group(int g) {
    GroupCache& gc = caches[g];
    int32_t* hi = hit_ids + (size_t)g * buffer_size;
    int32_t* hs = hit_sizes + (size_t)g * buffer_size;
    int32_t* hc = hit_cumsum + (size_t)g * buffer_size;
    int32_t* mi = miss_ids + (size_t)g * buffer_size;
    int32_t* ms = miss_sizes + (size_t)g * buffer_size;
    int32_t* mc = miss_cumsum + (size_t)g * buffer_size;
    const int64_t* ids = searched + (size_t)g * nprobe;
    gc.hit_keys.clear();
    gc.miss_keys.clear();
    int nh = 0, nm = 0, hsum = 0, msum = 0, pages = 0;
    for (int i = 0; i < nprobe; ++i) {
      const int c = (int)ids[i];
      if (c < 0 || c >= gc.ncl) continue;
      const int nb = gc.nblk[c];
      pages += nb;
      if (pages > buffer_size) {  // the rest of the probe list does not fit the execution buffer
        overflow.fetch_add(1, std::memory_order_relaxed);
        break;
      }
      if (nb == 0) continue;  // empty cluster: nothing to fetch
      if (!gc.resident[c]) {
        gc.miss_keys.push_back(c);
        int row = gc.start[c];
        for (int j = 0; j < nb; ++j) {
          const int sz = (j == nb - 1) ? gc.last[c] : block;
          mi[nm] = row; ms[nm] = sz; mc[nm] = msum;
          row += block; msum += sz; ++nm;
        }
      } else {
        gc.hit_keys.push_back(c);
        for (int j = 0; j < nb; ++j) {
          const int sz = (j == nb - 1) ? gc.last[c] : block;
          hi[nh] = gc.blk_ids[gc.blk_off[c] + j]; hs[nh] = sz; hc[nh] = hsum;
          hsum += sz; ++nh;
        }
      }
    }
    hit_nums[g] = nh;
    miss_nums[g] = nm;
  }

  void update_group(int g) {
    GroupCache& gc = caches[g];
    int32_t* ub = upd_buf + (size_t)g * buffer_size;
    int32_t* us = upd_sizes + (size_t)g * buffer_size;
    int32_t* uc = upd_cache + (size_t)g * buffer_size;
    // hits: most recent last touched = rank 0
    for (int i = (int)gc.hit_keys.size() - 1; i >= 0; --i) {
      const int c = gc.hit_keys[i];
      gc.lru_unlink(c);
      gc.lru_push_front(c);
    }
    // admit a prefix of the misses that fits the whole cache
    int admit = 0, need = 0;
    for (int c : gc.miss_keys) {
      if (need + gc.nblk[c] > gc.capacity) break;
      need += gc.nblk[c];
      ++admit;
    }
    int nu = 0, usum = 0;
    if (admit > 0) {
      while ((int)gc.free_blocks.size() < need && gc.lru_tail >= 0) gc.evict_tail();
      for (int i = 0; i < admit; ++i) {
        const int c = gc.miss_keys[i];
        gc.resident[c] = 1;
        for (int j = 0; j < gc.nblk[c]; ++j) {
          const int id = gc.free_blocks.back();
          gc.free_blocks.pop_back();
          gc.blk_ids[gc.blk_off[c] + j] = id;
          const int sz = (j == gc.nblk[c] - 1) ? gc.last[c] : block;
          uc[nu] = id; us[nu] = sz; ub[nu] = usum;
          usum += sz; ++nu;
        }
        gc.lru_push_front(c);
      }
    }
    upd_nums[g] = nu;
    gc.hit_keys.clear();
    gc.miss_keys.clear();
  }

  template <class F>
  std::vector<std::function<void()>> per_group_jobs(F f) {
    std::vector<std::function<void()>> v;
    for (int j = 0; j < jobs; ++j) {
      const int b = j * groups_per_job, e = std::min(BG, b + groups_per_job);
      v.emplace_back([this, b, e, f] { for (int g = b; g < e; ++g) (this->*f)(g); });
    }
    return v;
  }
};

extern "C" {

ri_threadpool* ri_threadpool_create(int num_threads) { return new ri_threadpool(num_threads); }
ri_threadpool* ri_threadpool_create_pinned(int num_threads, int first_core) {
  if (first_core < 0) return nullptr;
  return new ri_threadpool(num_threads, first_core);
}
int ri_threadpool_pinned_workers(const ri_threadpool* pool) { return pool ? pool->pool.pinned() : 0; }
void ri_threadpool_destroy(ri_threadpool* pool) { delete pool; }

ri_wavebuf* ri_wavebuf_create(int batch_size, int group_num, int dim, int nprobe, int block_size,
                              int n_centroids, int final_n_centroids, int buffer_size, int capacity,
                              int threads, ri_threadpool* pool) {
  if (!pool || batch_size <= 0 || group_num <= 0 || dim <= 0 || nprobe <= 0 || block_size <= 0 ||
      n_centroids <= 0 || final_n_centroids < n_centroids || buffer_size <= 0 || capacity < 0 || threads <= 0)
    return nullptr;
  ri_wavebuf* wb = new ri_wavebuf();
  wb->batch_size = batch_size; wb->group_num = group_num; wb->BG = batch_size * group_num; wb->dim = dim;
  wb->nprobe = nprobe; wb->block = block_size; wb->n_centroids = n_centroids;
  wb->final_n_centroids = final_n_centroids; wb->buffer_size = buffer_size; wb->capacity = capacity;
  wb->pool = &pool->pool;
  // at least two groups per job (wave_buffer_cpu.cpp:334-336)
  wb->jobs = std::min(threads, (wb->BG + 1) / 2);
  if (wb->jobs < 1) wb->jobs = 1;
  wb->groups_per_job = (wb->BG + wb->jobs - 1) / wb->jobs;
  wb->caches.resize(wb->BG);
  for (auto& c : wb->caches) c.init(capacity, final_n_centroids);
  wb->seq_len.assign(wb->BG, 0);
  return wb;
}

void ri_wavebuf_destroy(ri_wavebuf* wb) {
  if (!wb) return;
  wb->pool->wait();
  delete wb;
}

int ri_wavebuf_set_indices(ri_wavebuf* wb, int32_t* hit_ids, int32_t* hit_sizes, int32_t* hit_cumsum,
                           int32_t* hit_nums, int32_t* miss_ids, int32_t* miss_sizes, int32_t* miss_cumsum,
                           int32_t* miss_nums, int32_t* update_buffer_indices, int32_t* update_sizes,
                           int32_t* update_cache_indices, int32_t* update_nums, int64_t* searched_clusters) {
  if (!wb || !hit_ids || !hit_sizes || !hit_cumsum || !hit_nums || !miss_ids || !miss_sizes || !miss_cumsum ||
      !miss_nums || !update_buffer_indices || !update_sizes || !update_cache_indices || !update_nums ||
      !searched_clusters)
    return RI_ERR_ARG;
  wb->hit_ids = hit_ids; wb->hit_sizes = hit_sizes; wb->hit_cumsum = hit_cumsum; wb->hit_nums = hit_nums;
  wb->miss_ids = miss_ids; wb->miss_sizes = miss_sizes; wb->miss_cumsum = miss_cumsum; wb->miss_nums = miss_nums;
  wb->upd_buf = update_buffer_indices; wb->upd_sizes = update_sizes; wb->upd_cache = update_cache_indices;
  wb->upd_nums = update_nums; wb->searched = searched_clusters;
  return RI_OK;
}

int ri_wavebuf_set_kv(ri_wavebuf* wb, void* ivf_keys, void* ivf_values, int64_t output_seq_length,
                      void* input_keys, void* input_values, int64_t input_seq_length) {
  if (!wb || !ivf_keys || !ivf_values || output_seq_length <= 0) return RI_ERR_ARG;
  wb->ivf_k = (uint16_t*)ivf_keys; wb->ivf_v = (uint16_t*)ivf_values; wb->out_len = output_seq_length;
  wb->in_k = (uint16_t*)input_keys; wb->in_v = (uint16_t*)input_values; wb->in_len = input_seq_length;
  return RI_OK;
}

int ri_wavebuf_async_construction(ri_wavebuf* wb, const int32_t* clusters, const int32_t* cluster_size,
                                  int64_t max_cluster_size, int batch_idx) {
  if (!wb || !clusters || !cluster_size || batch_idx < 0 || batch_idx >= wb->batch_size) return RI_ERR_ARG;
  if (!wb->ivf_k || !wb->in_k) return RI_ERR_STATE;
  const int H = wb->group_num, nc = wb->n_centroids;
  // descriptors first (cheap, on the caller), then one copy job per KV head
  int64_t len0 = -1;
  for (int h = 0; h < H; ++h) {
    GroupCache& gc = wb->caches[batch_idx * H + h];
    gc.reset_clusters();
    const int64_t len = gc.add_clusters(cluster_size + (size_t)h * nc, nc, 0, wb->block);
    if (len0 < 0) len0 = len;
    if (len != len0 || len > wb->in_len || len > wb->out_len) return RI_ERR_ARG;
    wb->seq_len[batch_idx * H + h] = len;
  }
  std::vector<std::function<void()>> jobs;
  for (int h = 0; h < H; ++h) {
    jobs.emplace_back([wb, h, H, nc, clusters, cluster_size, max_cluster_size, batch_idx] {
      wb->organize(batch_idx * H + h, wb->in_k + (size_t)h * wb->in_len * wb->dim,
                   wb->in_v + (size_t)h * wb->in_len * wb->dim, wb->in_len,
                   clusters + (size_t)h * nc * max_cluster_size, cluster_size + (size_t)h * nc, nc,
                   max_cluster_size, 0);
    });
  }
  wb->pool->submit(std::move(jobs));
  return RI_OK;
}

int ri_wavebuf_construction_sync(ri_wavebuf* wb) {
  if (!wb) return RI_ERR_ARG;
  wb->pool->wait();
  return RI_OK;
}

int ri_wavebuf_update_kv(ri_wavebuf* wb, void* update_keys, void* update_values, int64_t update_seq_length,
                         const int32_t* clusters, const int32_t* cluster_size, int update_n_centroids,
                         int64_t max_cluster_size) {
  if (!wb || !update_keys || !update_values || !clusters || !cluster_size || update_n_centroids <= 0)
    return RI_ERR_ARG;
  if (!wb->ivf_k) return RI_ERR_STATE;
  wb->pool->wait();
  const int n = update_n_centroids;
  for (int g = 0; g < wb->BG; ++g)
    if (wb->caches[g].ncl + n > wb->final_n_centroids) return RI_ERR_ARG;
  std::vector<std::function<void()>> jobs;
  for (int j = 0; j < wb->jobs; ++j) {
    const int b = j * wb->groups_per_job, e = std::min(wb->BG, b + wb->groups_per_job);
    jobs.emplace_back([=] {
      for (int g = b; g < e; ++g) {
        const int64_t row0 = wb->seq_len[g];
        const int32_t* sz = cluster_size + (size_t)g * n;
        const int64_t end = wb->caches[g].add_clusters(sz, n, row0, wb->block);
        if (end > wb->out_len) continue;  // no room: descriptors exist but rows are not copied
        wb->organize(g, (const uint16_t*)update_keys + (size_t)g * update_seq_length * wb->dim,
                     (const uint16_t*)update_values + (size_t)g * update_seq_length * wb->dim, update_seq_length,
                     clusters + (size_t)g * n * max_cluster_size, sz, n, max_cluster_size, row0);
        wb->seq_len[g] = end;
      }
    });
  }
  wb->pool->submit(std::move(jobs));
  wb->pool->wait();
  return RI_OK;
}

int ri_wavebuf_batch_access(ri_wavebuf* wb) {
  if (!wb) return RI_ERR_ARG;
  if (!wb->hit_ids || !wb->searched) return RI_ERR_STATE;
  wb->pool->wait();
  wb->pool->submit(wb->per_group_jobs(&ri_wavebuf::access_group));
  wb->pool->wait();
  // the LRU update runs behind the caller's back until ri_wavebuf_sync()
  wb->pool->submit(wb->per_group_jobs(&ri_wavebuf::update_group));
  return RI_OK;
}

int ri_wavebuf_sync(ri_wavebuf* wb) {
  if (!wb) return RI_ERR_ARG;
  wb->pool->wait();
  return RI_OK;
}

int64_t ri_wavebuf_overflow_events(const ri_wavebuf* wb) { return wb ? wb->overflow.load() : 0; }

}  // extern "C"
