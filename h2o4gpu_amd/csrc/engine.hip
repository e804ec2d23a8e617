// Host side of the gfx950 k-means engine: the resident-data handle, the Lloyd
// loop, seeding, and the C entry points h2o4gpu's bindings call.
//
// Replaces src/gpu/kmeans/kmeans_h2o4gpu.cu (kmeans_fit :617-815,
// kmeans_predict :817-889, kmeans_transform :891-975, kmeans_init :572-607, the
// exported symbols :1060-1097) and the loop of src/gpu/kmeans/kmeans_impl.h
// :109-232. One device, one stream, no global state: calls on different handles
// are independent.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <csignal>
#include <cstdarg>
#include <cstdlib>
#include <condition_variable>
#include <cstring>
#include <ctime>
#include <limits>
#include <map>
#include <tuple>
#include <memory>
#include <mutex>
#include <new>
#include <numeric>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include <unistd.h>

#include "kmeans_common.h"

namespace kmhip {

// ---------------------------------------------------------------------------
// logging (format of src/common/logger.cpp:16-33)
// ---------------------------------------------------------------------------
void log_msg(int verbose, int level, const char *fmt, ...) {
  if (!(verbose > LOG_NOTHING && level <= verbose)) return;
  static const char *names[] = {"NOTHING", "FATAL", "ERROR", "INFO",
                                "WARN",    "DEBUG", "VERBOSE"};
  time_t now = time(nullptr);
  struct tm tmv;
  localtime_r(&now, &tmv);
  char buf[16];
  buf[strftime(buf, sizeof(buf), "%H:%M:%S", &tmv)] = '\0';
  fprintf(stderr, "%s %-5s kmeans_hip: ", buf, names[(level / 100) % 7]);
  va_list args;
  va_start(args, fmt);
  vfprintf(stderr, fmt, args);
  va_end(args);
  fprintf(stderr, "\n");
}

// Set by SIGINT/SIGTERM when the handlers are installed; the loop then finishes
// the current iteration, relabels once and returns normally
// (kmeans_h2o4gpu.cu:565-570, kmeans_impl.h:114,210-215). The reference
// installs the handlers on every call and never restores them; here they are
// installed only when H2O4GPU_KMEANS_SIGNALS=1 is set in the environment.
static volatile std::sig_atomic_t g_stop_flag = 0;
static void on_signal(int sig) {
  (void)sig;
  g_stop_flag = 1;
}
static void maybe_install_signal_handlers() {
  const char *e = getenv("H2O4GPU_KMEANS_SIGNALS");
  if (e && e[0] == '1') {
    std::signal(SIGINT, on_signal);
    std::signal(SIGTERM, on_signal);
  }
}

// The first k entries of
//     std::vector<int> v(n); std::iota(...); std::shuffle(v.begin(), v.end(),
//                                                        std::default_random_engine(seed));
// (the reference's random-row start, kmeans_h2o4gpu.cu:662-669) without shuffling n entries.
// libstdc++'s shuffle walks i = 1 .. n-1 and swaps v[i] with v[j_i], j_i uniform in [0, i];
// when step i runs, v[i] still holds i, so an entry below k changes only at steps with
// j_i < k, where it receives i. Only those steps touch memory; what remains per step is
// the generator (minstd_rand0: x <- 16807 x mod 2^31-1) and the acceptance test of
// uniform_int_distribution's two-division fallback, with the quotient urngrange / (i+1)
// carried along instead of recomputed. Below 46341 rows libstdc++ takes a different path
// (two swaps per draw) and the plain call is used; it is cheap there.
// 10M rows: 25 ms instead of 190 ms (the plain shuffle is bound by its random swaps).
static void first_rows_of_shuffle(int64_t n, int k, unsigned seed, int *out) {
  const uint64_t M = 2147483647ull;    // minstd_rand0 modulus
  const uint64_t R = M - 2;            // max() - min() of the engine
  if ((uint64_t)n <= R / (uint64_t)n || n < 2 * (int64_t)k + 2) {
    std::vector<int> v((size_t)n);
    std::iota(v.begin(), v.end(), 0);
    std::shuffle(v.begin(), v.end(), std::default_random_engine(seed));
    std::copy(v.begin(), v.begin() + k, out);
    return;
  }
  uint64_t x = seed % M;
  if (x == 0) x = 1;
  auto next = [&]() -> uint64_t {  // one step of the generator, value in [1, M-1]
    const uint64_t p = x * 16807ull;
    uint64_t r = (p & M) + (p >> 31);
    if (r >= M) r -= M;
    x = r;
    return r;
  };
  std::vector<int> a((size_t)k);
  std::iota(a.begin(), a.end(), 0);
  // steps inside the first k entries: ordinary swaps
  for (int64_t i = 1; i < k; i++) {
    const uint64_t ue = (uint64_t)i + 1, scaling = R / ue, past = ue * scaling;
    uint64_t ret;
    do ret = next() - 1; while (ret >= past);
    std::swap(a[(size_t)i], a[(size_t)(ret / scaling)]);
  }
  // steps i >= k: v[i] == i arrives at entry j when j < k
  uint64_t scaling = R / ((uint64_t)k + 1);
  uint64_t hold_until = R / scaling;  // largest i+1 with this quotient
  for (int64_t i = k; i < n; i++) {
    const uint64_t ue = (uint64_t)i + 1;
    if (ue > hold_until) {
      scaling = R / ue;
      hold_until = R / scaling;
    }
    const uint64_t past = ue * scaling;
    uint64_t ret;
    do ret = next() - 1; while (ret >= past);
    if (ret < (uint64_t)k * scaling) a[(size_t)(ret / scaling)] = (int)i;
  }
  std::copy(a.begin(), a.end(), out);
}

// (kernel, device) -> largest dynamic-LDS size granted so far
static std::mutex g_lds_mu;
static std::map<std::pair<const void *, int>, size_t> g_lds_granted;
int ensure_dynamic_lds(const void *kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return 0;  // within the default limit
  int dev = 0;
  KM_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_lds_mu);
  size_t &granted = g_lds_granted[std::make_pair(kernel, dev)];
  if (granted >= bytes) return 0;
  KM_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  granted = bytes;
  return 0;
}
// (kernel, device, dynamic LDS) -> workgroups of `block` threads one CU holds at once
static std::map<std::tuple<const void *, int, size_t>, int> g_resident;
int resident_blocks_per_cu(const void *kernel, int block, size_t lds) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 1;
  std::lock_guard<std::mutex> lock(g_lds_mu);
  auto key = std::make_tuple(kernel, dev, lds);
  auto it = g_resident.find(key);
  if (it != g_resident.end()) return it->second;
  int nb = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel, block, lds) != hipSuccess || nb < 1) {
    (void)hipGetLastError();
    nb = 1;
  }
  g_resident[key] = nb;
  return nb;
}
void forget_dynamic_lds(int dev) {
  std::lock_guard<std::mutex> lock(g_lds_mu);
  for (auto it = g_lds_granted.begin(); it != g_lds_granted.end();) {
    if (it->first.second == dev) it = g_lds_granted.erase(it);
    else ++it;
  }
  for (auto it = g_resident.begin(); it != g_resident.end();) {
    if (std::get<1>(it->first) == dev) it = g_resident.erase(it);
    else ++it;
  }
}

static int visible_devices() {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

}  // namespace kmhip

using namespace kmhip;

// ---------------------------------------------------------------------------
// the handle
// ---------------------------------------------------------------------------
struct h2o4gpu_kmeans_handle {
  int elem_size = 0;
  int64_t n = 0;
  int d = 0;
  int k = 0;  // rows of the model; a stacked handle holds sets * kps of them
  // stacked restarts: `sets` independent centroid sets of kset centroids each, every set
  // padded to kps model rows; cur_set is the set the per-set calls address
  int sets = 1, kset = 0, kps = 0, cur_set = 0;
  std::vector<int> set_iterations;
  int dev = 0;
  int verbose = 0;
  int num_cu = 0;
  hipStream_t stream = nullptr;
  int opt_assign = ASSIGN_AUTO;
  int opt_fuse = 1;  // 1: use the fused assign+accumulate kernel where the shape allows
  int opt_buckets = 1;  // 1: bucketed centroid sums where the sums do not fit LDS
  int opt_exact = 0;    // 1: float32 MFMA argmin on the float distances, not on 16-ulp keys
  int opt_split = 0;    // 6 or 9: float32 matrix-core kernels as that many bfloat16 products per feature pair
  int opt_transform_buffers = 2;  // sets of device buffers of a transform in several batches
  int opt_seed_matrix = 1;  // k-means||: distances between candidates as one matrix (0: a kernel per pick)
  int opt_tiled_direct = 1;  // tiled kernels: operands by direct-to-LDS loads where the shape allows
  int opt_transform_batch_mb = 4096;  // device buffer of transform_host's output, per batch of rows
  int last_variant = ASSIGN_AUTO;

  // profiling
  bool prof_on = false;
  struct Pending {
    std::string name;
    hipEvent_t a, b;
  };
  std::vector<Pending> pending;
  std::vector<hipEvent_t> pool;
  std::map<std::string, std::pair<int, double>> prof;
  hipEvent_t t0 = nullptr, t1 = nullptr;

  virtual ~h2o4gpu_kmeans_handle() {}
  virtual int set_data_host(const void *X) = 0;
  virtual int set_data_device(const void *dX) = 0;
  virtual int set_centroids_host(const void *C) = 0;
  virtual int init_random_rows(int seed) = 0;
  virtual int start_from_rows(const int *rows) = 0;  // centroids = the given k rows of the data
  virtual int init_plusplus(int seed) = 0;
  virtual int init_parallel(int seed) = 0;
  std::vector<int> last_seed_rows;
  // what the last k-means|| run found: data row of every candidate in the order found,
  // candidates added and sum of minimum costs per round, rows per nearest candidate (empty
  // when there were at most k candidates), candidate index of each final centre (-1: zero row)
  struct ParallelSeedInfo {
    std::vector<int> cand_rows;
    int round_count[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    double phi[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    std::vector<double> weights;
    std::vector<int> chosen;
  } seed_info;
  virtual int fit(int max_iterations, double threshold, int *iters) = 0;
  virtual int assign() = 0;
  virtual int update(double *shift2) = 0;
  virtual int set_labels_host(const int *labels) = 0;
  virtual int iterate(int steps) = 0;
  virtual int get_centroids(void *C) = 0;
  virtual int get_labels(int *labels) = 0;
  virtual int get_counts(int *counts) = 0;
  virtual int get_min_distances(void *m) = 0;
  virtual int inertia(double *out) = 0;
  virtual int predict_host(size_t rows, const void *X, int *labels) = 0;
  virtual int transform_host(size_t rows, const void *X, void *dist) = 0;
  virtual int transform_resident(void *d_dist) = 0;
  virtual int release() = 0;
  int kk() const { return sets > 1 ? kset : k; }  // centroids of one set

  hipEvent_t get_event() {
    if (!pool.empty()) {
      hipEvent_t e = pool.back();
      pool.pop_back();
      return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
  }
  void prof_begin(const char *name) {
    if (!prof_on) return;
    Pending p;
    p.name = name;
    p.a = get_event();
    p.b = get_event();
    if (p.a) (void)hipEventRecord(p.a, stream);
    pending.push_back(p);
  }
  void prof_end() {
    if (!prof_on || pending.empty()) return;
    if (pending.back().b) (void)hipEventRecord(pending.back().b, stream);
  }
  int prof_resolve() {
    if (pending.empty()) return 0;
    KM_HIP_TRY(hipStreamSynchronize(stream));
    for (auto &p : pending) {
      float ms = 0;
      if (p.a && p.b && hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
        auto &acc = prof[p.name];
        acc.first += 1;
        acc.second += ms;
      }
      if (p.a) pool.push_back(p.a);
      if (p.b) pool.push_back(p.b);
    }
    pending.clear();
    return 0;
  }
  void prof_free() {
    for (auto &p : pending) {
      if (p.a) (void)hipEventDestroy(p.a);
      if (p.b) (void)hipEventDestroy(p.b);
    }
    pending.clear();
    for (auto e : pool) (void)hipEventDestroy(e);
    pool.clear();
    if (t0) (void)hipEventDestroy(t0);
    if (t1) (void)hipEventDestroy(t1);
    t0 = t1 = nullptr;
  }
};

namespace kmhip {

// ---------------------------------------------------------------------------
// Host-to-device upload of a large pageable buffer through two pinned staging
// buffers: a few host threads copy chunk i+1 into one buffer while the DMA engine
// drains chunk i from the other. The entry points receive ordinary malloc'ed /
// numpy memory (src/gpu/kmeans/kmeans_h2o4gpu.h:24-42 copies it on the host first
// and then uploads it from pageable memory in one call).
// The buffers are allocated once per process and device and kept; uploads of
// different handles take turns.
// ---------------------------------------------------------------------------
struct StagingPool {
  // 1.28 GB of rows: 16 to 64 MB chunks all reach 52 GB/s, 8 MB 50, 4 MB 44 (the DMA alone: 56.7)
  static constexpr size_t CHUNK = 16u << 20;
  static constexpr int MAX_DEV = 64;
  std::mutex mu;
  void *buf[MAX_DEV][2] = {};
  hipEvent_t done[MAX_DEV][2] = {};
  // The staged copies run on a stream of the pool's own, which lives as long as the events
  // recorded on it. (Recorded on a handle's stream, an event outlived the stream: after some
  // 12,000 handles created and destroyed in one process, hipEventSynchronize on such an event
  // failed with "operation not permitted on an event last recorded in a capturing stream".)
  hipStream_t xfer[MAX_DEV] = {};
  bool broken[MAX_DEV] = {};

  // Host copies run on a small set of worker threads that are created once and then wait
  // for work: a staged transfer makes one such copy per chunk, which is no place to start
  // and join threads. The caller holds
  // mu, so there is one job at a time. The workers are never joined (they sleep until the
  // process ends); the state they share lives on the heap for that reason.
  struct Workers {
    std::mutex m;
    std::condition_variable wake, done;
    std::vector<std::thread> threads;
    long generation = 0;
    int pending = 0;
    int parts = 0;
    char *dst = nullptr;
    const char *src = nullptr;
    size_t bytes = 0, per = 0;
    // width != 0: src is the stretch [base, base + bytes) of a dense [rows][width] byte matrix
    // and dst the start of a matrix of the same rows `pitch` bytes apart
    size_t width = 0, pitch = 0, base = 0;
    pid_t owner = 0;
  };
  Workers *workers = nullptr;

  static void copy_bytes(char *dst, const char *src, size_t lo, size_t len, size_t width, size_t pitch,
                         size_t base) {
    if (width == 0) {
      memcpy(dst + lo, src + lo, len);
      return;
    }
    const char *s = src + lo;
    for (size_t f = base + lo, end = base + lo + len; f < end;) {
      const size_t row = f / width, col = f - row * width;
      const size_t run = std::min(width - col, end - f);
      memcpy(dst + row * pitch + col, s, run);
      s += run;
      f += run;
    }
  }
  static void copy_part(Workers *w, int part) {
    const size_t lo = w->per * (size_t)part;
    if (lo < w->bytes) copy_bytes(w->dst, w->src, lo, std::min(w->per, w->bytes - lo), w->width, w->pitch, w->base);
  }
  static void worker_main(Workers *w, int index) {
    long seen = 0;
    for (;;) {
      {
        std::unique_lock<std::mutex> lock(w->m);
        w->wake.wait(lock, [&] { return w->generation != seen; });
        seen = w->generation;
      }
      if (index < w->parts) copy_part(w, index);
      std::lock_guard<std::mutex> lock(w->m);
      if (--w->pending == 0) w->done.notify_one();
    }
  }
  void parallel_copy(char *dst, const char *src, size_t bytes, int threads, size_t width = 0, size_t pitch = 0,
                     size_t base = 0) {
    if (threads <= 1 || bytes < (4u << 20)) {
      copy_bytes(dst, src, 0, bytes, width, pitch, base);
      return;
    }
    // (a forked child has the parent's pool object but none of its threads)
    if (!workers || workers->owner != getpid() || (int)workers->threads.size() + 1 < threads) {
      Workers *w = new (std::nothrow) Workers();
      if (!w) {
        copy_bytes(dst, src, 0, bytes, width, pitch, base);
        return;
      }
      w->owner = getpid();
      try {
        for (int t = 1; t < threads; t++) w->threads.emplace_back(worker_main, w, t);
      } catch (...) {  // fewer workers than asked for: the parts below adapt
      }
      for (auto &th : w->threads) th.detach();
      workers = w;  // an earlier, smaller pool keeps sleeping
    }
    Workers *w = workers;
    const int nworkers = (int)w->threads.size();
    const int parts = std::min(threads, nworkers + 1);
    {
      std::lock_guard<std::mutex> lock(w->m);
      w->dst = dst;
      w->src = src;
      w->bytes = bytes;
      w->width = width;
      w->pitch = pitch;
      w->base = base;
      w->per = ((bytes + parts - 1) / parts + 4095) & ~(size_t)4095;
      w->parts = parts;
      w->pending = nworkers;
      w->generation++;
    }
    w->wake.notify_all();
    copy_part(w, 0);
    std::unique_lock<std::mutex> lock(w->m);
    w->done.wait(lock, [&] { return w->pending == 0; });
  }

  // Transfers below MIN_STAGED go the plain way. Above it the pieces are a quarter of the
  // transfer, at least 4 MB (what the copy threads need to be worth waking) and at most CHUNK.
  static constexpr size_t MIN_STAGED = 24u << 20;
  static size_t piece_size(size_t bytes) {
    size_t p = (bytes / 4 + ((1u << 20) - 1)) & ~(size_t)((1u << 20) - 1);
    if (p < (4u << 20)) p = 4u << 20;
    return p > CHUNK ? CHUNK : p;
  }

  // Pinned buffers and events of a device, created on first use (caller holds mu).
  bool ensure(int dev) {
    if (broken[dev]) return false;
    if (buf[dev][1] && done[dev][1] && xfer[dev]) return true;
    if (!xfer[dev] && hipStreamCreateWithFlags(&xfer[dev], hipStreamNonBlocking) != hipSuccess) {
      (void)hipGetLastError();
      xfer[dev] = nullptr;
      broken[dev] = true;
      return false;
    }
    for (int i = 0; i < 2; i++) {
      if (hipHostMalloc(&buf[dev][i], CHUNK, hipHostMallocDefault) != hipSuccess ||
          hipEventCreateWithFlags(&done[dev][i], hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        broken[dev] = true;
        return false;
      }
    }
    return true;
  }

  // Returns 0 on success; a positive value means "staging unavailable, use a plain copy".
  // wait_for_stream false: dst is memory that nothing queued on the caller's stream touches
  // (the next piece of a transfer whose earlier pieces are already being worked on)
  int upload(int dev, hipStream_t stream, void *dst, const void *src, size_t bytes, bool wait_for_stream = true) {
    if (dev < 0 || dev >= MAX_DEV || bytes < MIN_STAGED) return 1;
    std::lock_guard<std::mutex> lock(mu);
    if (!ensure(dev)) return 1;
    unsigned hw = std::thread::hardware_concurrency();
    const char *env = getenv("H2O4GPU_KMEANS_UPLOAD_THREADS");
    int threads = env ? atoi(env) : (int)std::min(8u, hw ? hw : 1u);
    if (threads < 1) threads = 1;
    const size_t piece = piece_size(bytes);
    size_t off = 0;
    if (wait_for_stream) KM_HIP_TRY(hipStreamSynchronize(stream));  // whatever the caller's stream still does with dst
    for (int i = 0; off < bytes; i ^= 1) {
      const size_t len = std::min(piece, bytes - off);
      KM_HIP_TRY(hipEventSynchronize(done[dev][i]));  // the DMA that last read this buffer
      parallel_copy(static_cast<char *>(buf[dev][i]), static_cast<const char *>(src) + off, len,
                    threads);
      KM_HIP_TRY(hipMemcpyAsync(static_cast<char *>(dst) + off, buf[dev][i], len,
                                hipMemcpyHostToDevice, xfer[dev]));
      KM_HIP_TRY(hipEventRecord(done[dev][i], xfer[dev]));
      off += len;
    }
    // both buffers must be drained before the next caller (or this one) refills them
    KM_HIP_TRY(hipEventSynchronize(done[dev][0]));
    KM_HIP_TRY(hipEventSynchronize(done[dev][1]));
    return 0;
  }

  // The way back: the DMA engine fills one buffer while host threads copy the other out.
  // width != 0: the device bytes are a dense [bytes / width][width] matrix whose rows go to
  // dst `pitch` bytes apart (a batch of columns of a wider host matrix). ready: the event
  // after the kernels that produce src, when the stream has later work queued that the
  // download need not wait for.
  int download(int dev, hipStream_t stream, void *dst, const void *src, size_t bytes, size_t width = 0,
               size_t pitch = 0, hipEvent_t ready = nullptr) {
    if (dev < 0 || dev >= MAX_DEV || bytes < MIN_STAGED) return 1;
    std::lock_guard<std::mutex> lock(mu);
    if (!ensure(dev)) return 1;
    unsigned hw = std::thread::hardware_concurrency();
    const char *env = getenv("H2O4GPU_KMEANS_UPLOAD_THREADS");
    int threads = env ? atoi(env) : (int)std::min(8u, hw ? hw : 1u);
    if (threads < 1) threads = 1;
    const size_t piece = piece_size(bytes);
    const size_t chunks = (bytes + piece - 1) / piece;
    if (ready) KM_HIP_TRY(hipEventSynchronize(ready));
    else KM_HIP_TRY(hipStreamSynchronize(stream));  // the kernels that produce src
    for (size_t c = 0; c <= chunks; c++) {
      const int b = (int)(c & 1);
      if (c < chunks) {
        const size_t off = c * piece, len = std::min(piece, bytes - off);
        KM_HIP_TRY(hipMemcpyAsync(buf[dev][b], static_cast<const char *>(src) + off, len,
                                  hipMemcpyDeviceToHost, xfer[dev]));
        KM_HIP_TRY(hipEventRecord(done[dev][b], xfer[dev]));
      }
      if (c >= 1) {  // chunk c-1 sits in the other buffer
        const size_t off = (c - 1) * piece, len = std::min(piece, bytes - off);
        KM_HIP_TRY(hipEventSynchronize(done[dev][b ^ 1]));
        if (width == 0)
          parallel_copy(static_cast<char *>(dst) + off, static_cast<const char *>(buf[dev][b ^ 1]), len,
                        threads);
        else
          parallel_copy(static_cast<char *>(dst), static_cast<const char *>(buf[dev][b ^ 1]), len, threads,
                        width, pitch, off);
      }
    }
    return 0;
  }

  // Gives a device's buffers back (before the device is reset: the reset frees them
  // behind the pool's back). The next transfer allocates new ones.
  void forget(int dev) {
    if (dev < 0 || dev >= MAX_DEV) return;
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < 2; i++) {
      if (done[dev][i]) (void)hipEventDestroy(done[dev][i]);
      if (buf[dev][i]) (void)hipHostFree(buf[dev][i]);
      done[dev][i] = nullptr;
      buf[dev][i] = nullptr;
    }
    if (xfer[dev]) (void)hipStreamDestroy(xfer[dev]);
    xfer[dev] = nullptr;
    broken[dev] = false;
  }
};
static StagingPool g_staging;

static int download_rows(int dev, hipStream_t stream, void *dst, const void *src, size_t bytes) {
  const int rc = g_staging.download(dev, stream, dst, src, bytes);
  if (rc <= 0) return rc;
  KM_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream));
  return 0;
}

// A dense device matrix of `height` rows of `width` bytes into host rows `pitch` bytes apart;
// `ready` as in StagingPool::download. Returns after the bytes have arrived.
static int download_matrix(int dev, hipStream_t stream, void *dst, size_t pitch, const void *src, size_t width,
                           size_t height, hipEvent_t ready) {
  const int rc = g_staging.download(dev, stream, dst, src, width * height, width, pitch, ready);
  if (rc <= 0) return rc;
  if (ready) KM_HIP_TRY(hipEventSynchronize(ready));
  else KM_HIP_TRY(hipStreamSynchronize(stream));
  KM_HIP_TRY(hipMemcpy2D(dst, pitch, src, width, width, height, hipMemcpyDeviceToHost));
  return 0;
}

static int upload_rows(int dev, hipStream_t stream, void *dst, const void *src, size_t bytes,
                       bool wait_for_stream = true) {
  const int rc = g_staging.upload(dev, stream, dst, src, bytes, wait_for_stream);
  if (rc <= 0) return rc;
  KM_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream));
  return 0;
}

#define PROFILED(name, call)   \
  do {                         \
    prof_begin(name);          \
    int _prc = (call);         \
    prof_end();                \
    if (_prc != 0) return _prc; \
  } while (0)

template <typename T>
struct Engine : h2o4gpu_kmeans_handle {
  T *X = nullptr;
  bool own_X = false;
  T *xnorm = nullptr;
  T *C[2] = {nullptr, nullptr};
  int cur = 0;
  T *cnorm = nullptr;
  int *labels = nullptr;
  T *mindist = nullptr;
  int *counts = nullptr;
  UpdatePlan plan;
  double *psums = nullptr;
  int *pcounts = nullptr;
  T *shift_partials = nullptr;
  T *shift2 = nullptr;
  int *order = nullptr, *order_label = nullptr, *bucket_offsets = nullptr, *bucket_hist = nullptr;
  int *bucket_seg = nullptr, *bucket_total = nullptr;
  double *bucket_partials = nullptr;
  bool use_buckets = false;
  double *sum_partials = nullptr;  // [sum_partials_needed() + 1]
  double *kpp_bsums = nullptr;
  int *kpp_rows = nullptr;  // [k] rows chosen so far by k-means++
  T *kpp_dcc = nullptr;     // [k] distances newest centre -> earlier centres
  bool have_data = false, have_centroids = false, have_mindist = false;
  int *d_frozen = nullptr;  // [sets] flags of a stacked handle's sets that have converged
  // (option fp32_split, tiled kernel) the centroids' bfloat16 parts, rewritten by every launch
  unsigned char *d_split = nullptr;
  size_t split_bytes = 0;
  // The scratch a launch with the option needs, allocated on first use (an in-flight launch
  // may still read the old one: the stream is drained before it is replaced); null when the
  // option is off or does not apply, and when the allocation fails (the launch then runs the
  // float32 instructions).
  SplitScratch split_scratch() { return split_scratch(k); }
  SplitScratch split_scratch(int model_rows) {  // (the seeding runs models of other sizes)
    SplitScratch sc;
    sc.through_registers = opt_tiled_direct == 0;
    const size_t need = opt_split ? tiled_split_scratch_bytes<T>(opt_split, d, model_rows) : 0;
    if (need == 0) return sc;
    if (need > split_bytes) {
      (void)hipStreamSynchronize(stream);
      if (d_split) (void)hipFree(d_split);
      d_split = nullptr;
      split_bytes = 0;
      if (dalloc(&d_split, need) != 0) return sc;
      split_bytes = need;
    }
    sc.ptr = d_split;
    sc.bytes = split_bytes;
    return sc;
  }
  StackShape shape() const {
    StackShape st;
    st.sets = sets;
    st.kps = kps;
    st.kset = kset;
    return st;
  }
  size_t set_off() const { return sets > 1 ? (size_t)cur_set * kps : 0; }  // first model row of the set
  size_t row_off() const { return sets > 1 ? (size_t)cur_set * (size_t)n : 0; }  // its block of labels

  template <typename U>
  int dalloc(U **p, size_t count) {
    *p = nullptr;
    if (count == 0) count = 1;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(p), count * sizeof(U));
    if (e != hipSuccess) {
      (void)hipGetLastError();
      // the reference's message and level (log_error(verbose, ...), kmeans_impl.h:81-94):
      // printed when verbose >= 200, and the call returns -1
      log_msg(verbose, LOG_ERROR,
              "Unable to allocate memory for gpu: %d | n: %lld | k: %d | d: %d | error: %s "
              "(%zu bytes)",
              dev, (long long)n, k, d, hipGetErrorString(e), count * sizeof(U));
      return H2O4GPU_KMEANS_EALLOC;
    }
    return 0;
  }

  int create() {
    KM_HIP_TRY(hipSetDevice(dev));
    hipDeviceProp_t prop;
    KM_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    num_cu = prop.multiProcessorCount;
    KM_HIP_TRY(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    plan = plan_update<T>(n, d, k, num_cu);
    const size_t kd = (size_t)k * d;
    // Centroid buffers are padded to a multiple of CENTROID_PAD rows (zeros) and the
    // norms to as many entries (+inf): the tiled MFMA kernels read whole centroid
    // blocks without bounds tests and the padding can never win an argmin.
    const size_t kpad = ((size_t)k + CENTROID_PAD - 1) / CENTROID_PAD * CENTROID_PAD;
    KM_TRY(dalloc(&C[0], kpad * d));
    KM_TRY(dalloc(&C[1], kpad * d));
    KM_TRY(dalloc(&cnorm, kpad));
    KM_HIP_TRY(hipMemsetAsync(C[0], 0, kpad * d * sizeof(T), stream));
    KM_HIP_TRY(hipMemsetAsync(C[1], 0, kpad * d * sizeof(T), stream));
    {
      std::vector<T> inf(kpad, std::numeric_limits<T>::infinity());
      KM_HIP_TRY(hipMemcpyAsync(cnorm, inf.data(), kpad * sizeof(T), hipMemcpyHostToDevice, stream));
      KM_HIP_TRY(hipStreamSynchronize(stream));
    }
    if (sets > 1) {
      // every step of a stacked handle is the fused row-stationary kernel over the whole model
      if (pick_assign_variant<T>(ASSIGN_AUTO, n, d, k) != ASSIGN_ROWSTAT ||
          fused_slots<T>(ASSIGN_AUTO, n, d, k, num_cu) <= 0)
        return H2O4GPU_KMEANS_EARG;
      KM_TRY(dalloc(&d_frozen, sets));
      KM_HIP_TRY(hipMemsetAsync(d_frozen, 0, (size_t)sets * sizeof(int), stream));
    }
    KM_TRY(dalloc(&counts, k));
    KM_TRY(dalloc(&labels, (size_t)n * sets));
    KM_TRY(dalloc(&xnorm, n));
    KM_TRY(dalloc(&mindist, (size_t)n * sets));
    int slots = plan.row_blocks;
    const int fs = fused_slots<T>(ASSIGN_AUTO, n, d, k, num_cu);
    if (fs > slots) slots = fs;
    // (a shape the long-row kernel takes only when asked to writes more slots than the default kernel's)
    if (sets == 1 && longrow_applies<T>(d, k)) slots = std::max(slots, longrow_max_slots<T>(d, k, num_cu));
    KM_TRY(dalloc(&psums, (size_t)slots * kd));
    KM_TRY(dalloc(&pcounts, (size_t)slots * k));
    use_buckets = bucketed_update_applies(plan.k_chunks, k, d);
    if (use_buckets) {
      KM_TRY(dalloc(&order, n));
      KM_TRY(dalloc(&order_label, n));
      KM_TRY(dalloc(&bucket_offsets, k));
      KM_TRY(dalloc(&bucket_hist, (size_t)bucket_blocks(n) * k));
      KM_TRY(dalloc(&bucket_seg, (size_t)32 * k));
      KM_TRY(dalloc(&bucket_total, 1));
      KM_TRY(dalloc(&bucket_partials, bucket_partial_slots(n, k) * d));
    }
    KM_TRY(dalloc(&shift_partials, (size_t)max_shift_partials(d, k) + 1));
    KM_TRY(dalloc(&shift2, (size_t)sets));
    KM_TRY(dalloc(&sum_partials, sum_partials_needed() + 1));
    KM_TRY(dalloc(&kpp_bsums, (n + KPP_BLOCK - 1) / KPP_BLOCK + 1));
    KM_TRY(dalloc(&kpp_rows, (size_t)k + 1));
    KM_TRY(dalloc(&kpp_dcc, (size_t)k + 1));
    // the reference's label vector starts zeroed (thrust::device_vector<int>)
    KM_HIP_TRY(hipMemsetAsync(labels, 0, (size_t)n * sets * sizeof(int), stream));
    KM_HIP_TRY(hipMemsetAsync(counts, 0, (size_t)k * sizeof(int), stream));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    log_msg(verbose, LOG_DEBUG,
            "handle: rows=%lld cols=%d k=%d elem=%d device=%d CUs=%d update plan: "
            "row_blocks=%d kc=%d k_chunks=%d vec=%d",
            (long long)n, d, k, (int)sizeof(T), dev, num_cu, plan.row_blocks, plan.kc,
            plan.k_chunks, plan.vec);
    return 0;
  }

  int release() override {
    (void)hipSetDevice(dev);
    if (stream) (void)hipStreamSynchronize(stream);
    prof_free();
    if (host_shift) (void)hipHostFree(host_shift);
    host_shift = nullptr;
    for (auto &e : shift_ready) {
      if (e) (void)hipEventDestroy(e);
      e = nullptr;
    }
    if (own_X && X) (void)hipFree(X);
    void *ptrs[] = {xnorm,  C[0],    C[1],           cnorm,  labels,       mindist,
                    counts, psums,   pcounts,        shift_partials, shift2,
                    sum_partials, kpp_bsums, kpp_rows, kpp_dcc, order, order_label, bucket_offsets,
                    bucket_hist, bucket_seg, bucket_total, bucket_partials, d_frozen, d_split};
    for (void *p : ptrs)
      if (p) (void)hipFree(p);
    if (stream) (void)hipStreamDestroy(stream);
    stream = nullptr;
    return 0;
  }

  int set_data_host(const void *hX) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!hX) return H2O4GPU_KMEANS_EARG;
    if (!own_X || !X) {
      X = nullptr;
      KM_TRY(dalloc(&X, (size_t)n * d));
      own_X = true;
    }
    KM_TRY(upload_rows(dev, stream, X, hX, (size_t)n * d * sizeof(T)));
    PROFILED("row_norms", launch_row_norms<T>(stream, X, xnorm, n, d));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    have_data = true;
    return 0;
  }

  int set_data_device(const void *dX) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!dX) return H2O4GPU_KMEANS_EARG;
    if (own_X && X) (void)hipFree(X);
    X = const_cast<T *>(static_cast<const T *>(dX));
    own_X = false;
    PROFILED("row_norms", launch_row_norms<T>(stream, X, xnorm, n, d));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    have_data = true;
    return 0;
  }

  int centroids_changed() {
    PROFILED("row_norms", launch_row_norms<T>(stream, C[cur], cnorm, k, d));
    cnorm_stale = false;
    have_centroids = true;
    return 0;
  }

  int set_centroids_host(const void *hC) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!hC) return H2O4GPU_KMEANS_EARG;
    KM_HIP_TRY(hipMemcpyAsync(C[cur] + set_off() * d, hC, (size_t)kk() * d * sizeof(T),
                              hipMemcpyHostToDevice, stream));
    KM_TRY(centroids_changed());
    KM_HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }

  // Seeded random distinct rows: the same two standard-library calls as
  // kmeans_h2o4gpu.cu:662-669; centroids are rows v[0..k-1] (:79-84, :692-693).
  int init_random_rows(int seed) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data) return H2O4GPU_KMEANS_ESTATE;
    const int k = kk();
    if ((int64_t)k > n) return H2O4GPU_KMEANS_EARG;
    unsigned useed = (unsigned)seed;
    if (seed < 0) {
      std::random_device rd;
      useed = rd();
    }
    std::vector<int> v((size_t)k);
    first_rows_of_shuffle(n, k, useed, v.data());
    last_seed_rows = v;
    return init_from_rows(v.data());
  }

  int start_from_rows(const int *rows) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data || !rows) return H2O4GPU_KMEANS_ESTATE;
    last_seed_rows.assign(rows, rows + kk());
    return init_from_rows(rows);
  }

  int init_from_rows(const int *idx_host) {
    const int k = kk();
    int *didx = nullptr;
    KM_TRY(dalloc(&didx, k));
    hipError_t e = hipMemcpyAsync(didx, idx_host, (size_t)k * sizeof(int), hipMemcpyHostToDevice, stream);
    int rc = e == hipSuccess ? launch_gather_rows<T>(stream, X, didx, C[cur] + set_off() * d, k, d)
                             : H2O4GPU_KMEANS_EDEVICE;
    if (rc == 0) rc = centroids_changed();
    (void)hipStreamSynchronize(stream);
    (void)hipFree(didx);
    return rc;
  }

  // k-means++ (D^2 sampling). First centre: mt19937(seed) uniform over rows,
  // as the reference draws its first k-means|| centre
  // (kmeans_h2o4gpu.cu:343-347). Every further centre: u ~ U[0,1) from the same
  // generator, target = u * total where total is the ordered double sum of the
  // block sums; the block is found by an ordered scan of the block sums, the
  // row by an ordered scan (in double) of that block's minima.
  int init_plusplus(int seed) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data) return H2O4GPU_KMEANS_ESTATE;
    const int k = kk();
    if ((int64_t)k > n) return H2O4GPU_KMEANS_EARG;
    std::mt19937 gen(seed >= 0 ? (unsigned)seed : std::random_device{}());
    std::uniform_int_distribution<> first(0, (int)(n - 1));
    std::uniform_real_distribution<double> uni(0.0, 1.0);
    const int64_t nb = (n + KPP_BLOCK - 1) / KPP_BLOCK;
    std::vector<int> idx(k);
    std::vector<double> bs((size_t)nb);
    std::vector<T> blk(KPP_BLOCK);
    idx[0] = first(gen);
    // per-row scratch of the seeding: the selected set's own block of a stacked handle
    T *const md = mindist + row_off();
    int *const lb = labels + row_off();
    for (int c = 1; c <= k; c++) {
      PROFILED("min_dist_update",
               launch_min_dist_update<T>(stream, X, xnorm, idx[c - 1], md, lb,
                                         kpp_rows, kpp_dcc, c - 1, kpp_bsums, n, d));
      if (c == k) break;
      KM_HIP_TRY(hipMemcpyAsync(bs.data(), kpp_bsums, (size_t)nb * sizeof(double),
                                hipMemcpyDeviceToHost, stream));
      KM_HIP_TRY(hipStreamSynchronize(stream));
      double total = 0;
      for (int64_t b = 0; b < nb; b++) total += bs[b];
      const double u = uni(gen);
      int64_t pick;
      if (!(total > 0)) {
        pick = (int64_t)(u * (double)n);
        if (pick >= n) pick = n - 1;
      } else {
        const double target = u * total;
        double run = 0;
        int64_t b = 0;
        for (; b < nb - 1; b++) {
          if (run + bs[b] > target) break;
          run += bs[b];
        }
        const int64_t lo = b * KPP_BLOCK;
        const int cntb = (int)std::min<int64_t>(KPP_BLOCK, n - lo);
        KM_HIP_TRY(hipMemcpyAsync(blk.data(), md + lo, (size_t)cntb * sizeof(T),
                                  hipMemcpyDeviceToHost, stream));
        KM_HIP_TRY(hipStreamSynchronize(stream));
        int i = 0, last_pos = 0;
        for (; i < cntb; i++) {
          if ((double)blk[i] > 0) last_pos = i;
          if (run + (double)blk[i] > target) break;
          run += (double)blk[i];
        }
        if (i >= cntb) i = last_pos;  // rounding left the target past the end
        pick = lo + i;
      }
      idx[c] = (int)pick;
    }
    have_mindist = sets == 1;  // minimum distance of every row to the k chosen centres
    last_seed_rows = idx;
    return init_from_rows(idx.data());
  }

  // k-means|| followed by the reference's host k-means++ over the weighted candidates
  // (kmeans_parallel, kmeans_h2o4gpu.cu:331-563, one device; kmeans_plus_plus :201-279;
  // pick_point_idx_weighted :154-199). Kept as the reference has them: the first centre
  // from mt19937(seed); min(8, (int)(2 + log(k))) rounds; a round measures the rows against
  // the candidates of the previous round only and keeps a running minimum; a row becomes
  // a candidate when T(2.0 * k * cost / total) exceeds its threshold, which depends on
  // (seed, row) alone; a potential of 0 skips the selection; more than k candidates are
  // weighted by the rows nearest to each and reduced on the host with the re-seeded
  // sampler; at most k candidates become the first centres followed by zero rows. The
  // seed is used as given, negative or not (:339-342 re-declares the variable it means to
  // replace). Not the reference's: the order of the sums (distances come from these
  // kernels instead of cuBLAS, the sum of the costs is a fixed tree in double, rounded to T).
  int init_parallel(int seed) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data) return H2O4GPU_KMEANS_ESTATE;
    if ((int64_t)kk() > n) return H2O4GPU_KMEANS_EARG;
    seed_info = ParallelSeedInfo();
    std::mt19937 gen(seed);
    std::uniform_int_distribution<> dis(0, (int)(n - 1));
    std::vector<int> all(1, dis(gen));
    std::vector<int> recent = all;
    T *cost = nullptr, *Cc = nullptr, *ccn = nullptr, *best = nullptr;
    int *list = nullptr, *didx = nullptr, *dcount = nullptr, *near = nullptr;
    int rc = parallel_rounds(seed, all, recent, &cost, &Cc, &ccn, &best, &list, &didx, &dcount, &near);
    (void)hipStreamSynchronize(stream);
    void *ptrs[] = {cost, Cc, ccn, best, list, didx, dcount, near};
    for (void *p : ptrs)
      if (p) (void)hipFree(p);
    have_mindist = false;  // mindist served as scratch
    // and so did this set's labels (they number the candidates, not the centroids)
    if (hipMemsetAsync(labels + row_off(), 0, (size_t)n * sizeof(int), stream) != hipSuccess && rc == 0)
      rc = H2O4GPU_KMEANS_EDEVICE;
    return rc;
  }
  // (re)allocates a device buffer of at least `count` elements
  template <typename U>
  int regrow(U **p, size_t *have, size_t count) {
    if (*p && *have >= count) return 0;
    if (*p) (void)hipFree(*p);
    *p = nullptr;
    *have = 0;
    KM_TRY(dalloc(p, count));
    *have = count;
    return 0;
  }
  int parallel_rounds(int seed, std::vector<int> &all, std::vector<int> &recent, T **cost, T **Cc,
                      T **ccn, T **best, int **list, int **didx, int **dcount, int **near) {
    const int k = kk();
    const int64_t nb = (n + KPP_BLOCK - 1) / KPP_BLOCK;
    size_t cap_model = 0, cap_norm = 0, cap_idx = 0, cap_best = 0;
    const int list_cap = (int)n;
    // per-row scratch of the rounds: the selected set's own block of a stacked handle (the
    // block that init_parallel clears afterwards)
    T *const md = mindist + row_off();
    int *const lb = labels + row_off();
    KM_TRY(dalloc(cost, n));
    KM_TRY(dalloc(near, n));
    KM_TRY(dalloc(list, list_cap));
    KM_TRY(dalloc(dcount, 1));
    std::vector<double> bs((size_t)nb);
    // stage m candidate rows as a padded model
    auto stage = [&](const std::vector<int> &rows) -> int {
      const size_t m = rows.size();
      const size_t mpad = (m + CENTROID_PAD - 1) / CENTROID_PAD * CENTROID_PAD;
      KM_TRY(regrow(Cc, &cap_model, mpad * d));
      KM_TRY(regrow(ccn, &cap_norm, mpad));
      KM_TRY(regrow(didx, &cap_idx, m));
      KM_HIP_TRY(hipMemcpyAsync(*didx, rows.data(), m * sizeof(int), hipMemcpyHostToDevice, stream));
      return launch_gather_model<T>(stream, X, xnorm, *didx, (int)m, (int)mpad, *Cc, *ccn, d);
    };
    uint32_t state0 = (uint32_t)seed % 2147483647u;  // thrust seeds minstd_rand like this
    if (state0 == 0) state0 = 1;
    const int rounds = std::min(8, (int)(2 + std::log((double)k)));
    // Every round also notes which candidate each row's running minimum belongs to (numbered
    // as in `all`), so the rows per nearest candidate that the weights need are there when
    // the rounds end, without another pass over all candidates (500k x 784, 8304 candidates:
    // 53 ms of 0.28 s). recent_off: where this round's candidates start in `all`; measured:
    // whether `recent` has been through a pass yet.
    int recent_off = 0;
    bool measured = false;
    // A round that adds no candidate leaves `recent` as it was: the next round would measure
    // the same candidates again, find the same costs, the same potential and, the thresholds
    // depending on (seed, row) alone, the same empty selection. Such rounds are not run; their
    // potential and count are the previous round's.
    bool settled = false;
    for (int counter = 0; counter < rounds; counter++) {
      log_msg(verbose, LOG_VERBOSE, "KMeans|| - Iteration %d.", counter);
      if (settled) {
        seed_info.phi[counter] = seed_info.phi[counter - 1];
        seed_info.round_count[counter] = 0;
        log_msg(verbose, LOG_VERBOSE, "KMeans|| - Total min cost from centers %g.", seed_info.phi[counter]);
        if (seed_info.phi[counter] != 0) log_msg(verbose, LOG_VERBOSE, "KMeans|| - New potential centroids %d.", 0);
        continue;
      }
      KM_TRY(stage(recent));
      // minimum distance to this round's candidates, compared as floats (no integer keys)
      PROFILED("seed_assign", launch_assign<T>(stream, opt_assign, X, xnorm, *Cc, *ccn, lb, md,
                                               n, d, (int)recent.size(), num_cu, nullptr, true, StackShape(),
                                               opt_split, split_scratch((int)recent.size())));
      PROFILED("seed_fold", launch_fold_min<T>(stream, md, *cost, kpp_bsums, n, counter == 0, lb, *near,
                                               recent_off));
      measured = true;
      KM_HIP_TRY(hipMemcpyAsync(bs.data(), kpp_bsums, (size_t)nb * sizeof(double), hipMemcpyDeviceToHost,
                                stream));
      KM_HIP_TRY(hipStreamSynchronize(stream));
      double sum = 0;
      for (int64_t b = 0; b < nb; b++) sum += bs[(size_t)b];
      const T total = (T)sum;
      seed_info.phi[counter] = (double)total;
      log_msg(verbose, LOG_VERBOSE, "KMeans|| - Total min cost from centers %g.", (double)total);
      if (total == (T)0) {
        settled = true;
        continue;
      }
      KM_HIP_TRY(hipMemsetAsync(*dcount, 0, sizeof(int), stream));
      PROFILED("seed_select", launch_select_rows<T>(stream, *cost, total, state0, k, *list, *dcount,
                                                    list_cap, n));
      int count = 0;
      KM_HIP_TRY(hipMemcpyAsync(&count, *dcount, sizeof(int), hipMemcpyDeviceToHost, stream));
      KM_HIP_TRY(hipStreamSynchronize(stream));
      if (count > list_cap) count = list_cap;  // (cannot happen: one entry per row at most)
      seed_info.round_count[counter] = count;
      log_msg(verbose, LOG_VERBOSE, "KMeans|| - New potential centroids %d.", count);
      if (count == 0) settled = true;
      if (count > 0) {
        recent.resize((size_t)count);
        KM_HIP_TRY(hipMemcpyAsync(recent.data(), *list, (size_t)count * sizeof(int), hipMemcpyDeviceToHost,
                                  stream));
        KM_HIP_TRY(hipStreamSynchronize(stream));
        std::sort(recent.begin(), recent.end());  // the reference's copy_if keeps row order
        recent_off = (int)all.size();
        measured = false;
        all.insert(all.end(), recent.begin(), recent.end());
      }
    }
    seed_info.cand_rows = all;
    const int M = (int)all.size();
    seed_info.chosen.assign((size_t)k, -1);
    if (M <= k) {  // kmeans_h2o4gpu.cu:536-540: the candidates, then zero rows
      for (int c = 0; c < M; c++) seed_info.chosen[(size_t)c] = c;
      KM_HIP_TRY(hipMemsetAsync(C[cur] + set_off() * d, 0, (size_t)k * d * sizeof(T), stream));
      KM_TRY(regrow(didx, &cap_idx, (size_t)M));
      KM_HIP_TRY(hipMemcpyAsync(*didx, all.data(), (size_t)M * sizeof(int), hipMemcpyHostToDevice, stream));
      KM_TRY(launch_gather_rows<T>(stream, X, *didx, C[cur] + set_off() * d, M, d));
      last_seed_rows.assign((size_t)k, -1);
      std::copy(all.begin(), all.end(), last_seed_rows.begin());
      KM_TRY(centroids_changed());
      KM_HIP_TRY(hipStreamSynchronize(stream));
      return 0;
    }
    // weights: rows per nearest candidate (count_pts_per_centroid, kmeans_h2o4gpu.h:90-126). The
    // rounds have kept the nearest candidate of every row so far; what the last round added has
    // not been through a pass yet.
    if (!measured) {
      KM_TRY(stage(recent));
      PROFILED("seed_weights", launch_assign<T>(stream, opt_assign, X, xnorm, *Cc, *ccn, lb, md, n, d,
                                                (int)recent.size(), num_cu, nullptr, true, StackShape(),
                                                opt_split, split_scratch((int)recent.size())));
      PROFILED("seed_fold", launch_fold_min<T>(stream, md, *cost, kpp_bsums, n, 0, lb, *near, recent_off));
    }
    KM_TRY(stage(all));  // the picks below read all candidates
    int *dhist = nullptr;
    size_t cap_hist = 0;
    KM_TRY(regrow(&dhist, &cap_hist, (size_t)M));
    std::vector<int> hist((size_t)M);
    int rc = hipMemsetAsync(dhist, 0, (size_t)M * sizeof(int), stream) == hipSuccess ? 0 : H2O4GPU_KMEANS_EDEVICE;
    if (rc == 0) rc = launch_label_histogram(stream, *near, dhist, n);
    if (rc == 0 && hipMemcpyAsync(hist.data(), dhist, (size_t)M * sizeof(int), hipMemcpyDeviceToHost, stream) != hipSuccess)
      rc = H2O4GPU_KMEANS_EDEVICE;
    if (rc == 0 && hipStreamSynchronize(stream) != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
    (void)hipFree(dhist);
    KM_TRY(rc);
    std::vector<T> w((size_t)M);
    seed_info.weights.resize((size_t)M);
    for (int c = 0; c < M; c++) {
      w[(size_t)c] = (T)hist[(size_t)c];
      seed_info.weights[(size_t)c] = (double)hist[(size_t)c];
    }
    // the host k-means++ (kmeans_h2o4gpu.cu:201-279); its distances run on the device
    KM_TRY(regrow(best, &cap_best, (size_t)M));
    std::vector<T> thr((size_t)M), share((size_t)M);
    {
      std::mt19937 mt(seed);  // the sampler makes a fresh one on every call: same draws
      std::uniform_real_distribution<> dist(0.0, 1.0);
      for (int i = 0; i < M; i++) thr[(size_t)i] = (T)dist(mt);
    }
    auto pick = [&](const T *data) -> int {  // pick_point_idx_weighted
      T weighted_sum = 0;
      for (int i = 0; i < M; i++) weighted_sum += data ? data[i] * w[(size_t)i] : w[(size_t)i];
      // the shares first, in a loop without an exit (it vectorises; the divisions are the same
      // IEEE divisions), then the reference's walk over them
      for (int i = 0; i < M; i++) share[(size_t)i] = (data ? data[i] * w[(size_t)i] : w[(size_t)i]) / weighted_sum;
      // The walk, `if (share > threshold) return i; if (share >= best) { best = share; idx = i; }`
      // from a best of 0, in loops without an exit where it matters: whether any entry passes
      // its threshold at all (rarely: a share is about 1/M), then the largest share that is not
      // below 0 and the last entry that has it (a NaN share is neither passed nor kept, as in
      // the walk; -0 equals 0 in both).
      int passes = 0;
      for (int i = 0; i < M; i++) passes += share[(size_t)i] > thr[(size_t)i] ? 1 : 0;
      if (passes)
        for (int i = 0; i < M; i++)
          if (share[(size_t)i] > thr[(size_t)i]) return i;
      T lane_best[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // (eight running maxima: no chain of dependent compares)
      int i8 = 0;
      for (; i8 + 8 <= M; i8 += 8)
        for (int u = 0; u < 8; u++)
          lane_best[u] = share[(size_t)(i8 + u)] > lane_best[u] ? share[(size_t)(i8 + u)] : lane_best[u];
      T best_prob = 0;
      for (; i8 < M; i8++) best_prob = share[(size_t)i8] > best_prob ? share[(size_t)i8] : best_prob;
      for (int u = 0; u < 8; u++) best_prob = lane_best[u] > best_prob ? lane_best[u] : best_prob;
      for (int i = M - 1; i > 0; i--)
        if (share[(size_t)i] == best_prob) return i;
      return 0;
    };
    // With the scalar-order kernels asked for ("assign" = valu: every distance of the seeding
    // is then what a scalar loop gives, bit for bit) the distances between candidates are
    // summed in feature order too, one thread per candidate on a column-major copy; otherwise
    // by several lanes per candidate.
    // Otherwise, while M x M distances fit 1 GiB, all of them are computed at once by the
    // transform kernels (the candidates against themselves, |v| where the reference has v: the
    // two differ for v < 0 only, i.e. within rounding of a candidate's distance to a copy of
    // itself) and brought to the host, where a pick is then a minimum over one row of that
    // matrix and the sampler's two loops, with no launch and no wait: 8304 candidates of 784
    // features, 4095 picks: 57 ms of kernels and as many waits become 1 ms + a 276 MB download.
    if (opt_seed_matrix && opt_assign != ASSIGN_VALU && (size_t)M * (size_t)M * sizeof(T) <= ((size_t)1 << 30)) {
      std::vector<T> hb((size_t)M);
      // (left uninitialised: the download fills it, and zeroing up to 1 GiB first costs as
      // much as the download)
      std::unique_ptr<T[]> hG(new (std::nothrow) T[(size_t)M * M]);
      T *G = nullptr;
      if (hG && dalloc(&G, (size_t)M * M) == 0) {
        int grc = 0;
        prof_begin("seed_gram");
        grc = launch_transform<T>(stream, *Cc, *ccn, *Cc, *ccn, G, (int64_t)M, (int64_t)M, d, M, num_cu,
                                  opt_split, split_scratch(M));
        prof_end();
        if (grc == 0) grc = download_rows(dev, stream, hG.get(), G, (size_t)M * M * sizeof(T));
        if (grc == 0 && hipStreamSynchronize(stream) != hipSuccess) grc = H2O4GPU_KMEANS_EDEVICE;
        (void)hipFree(G);
        KM_TRY(grc);
        int idx = pick(nullptr);
        for (int c = 0; c < k; c++) {
          seed_info.chosen[(size_t)c] = idx;
          w[(size_t)idx] = 0;
          if (c == k - 1) break;
          const T *g = hG.get() + (size_t)idx * M;
          if (c == 0) {
            std::copy(g, g + M, hb.begin());
          } else {
            hb[(size_t)idx] = 0;  // (the reference takes the centre's own running value as 0)
            for (int i = 0; i < M; i++) hb[(size_t)i] = g[i] < hb[(size_t)i] ? g[i] : hb[(size_t)i];
          }
          idx = pick(hb.data());
        }
        std::vector<int> rows((size_t)k);
        for (int c = 0; c < k; c++) rows[(size_t)c] = all[(size_t)seed_info.chosen[(size_t)c]];
        last_seed_rows = rows;
        return init_from_rows(rows.data());
      }
      (void)hipGetLastError();  // no room for the matrix: one kernel per pick, below
    }
    T *CcT = nullptr;
    int prc = 0;
    if (opt_assign == ASSIGN_VALU) {
      KM_TRY(dalloc(&CcT, (size_t)M * d));
      prc = launch_transpose_candidates<T>(stream, *Cc, CcT, M, d);
    }
    // every pick ends with the M distances on the host: the kernel writes them into pinned host
    // memory itself, beside its device copy, so a pick costs one launch and one wait and no
    // copy command (8304 candidates, 4096 picks: 0.317 -> 0.29 s for the whole seeding)
    T *hbest = nullptr;
    if (prc == 0 && hipHostMalloc(reinterpret_cast<void **>(&hbest), (size_t)M * sizeof(T), hipHostMallocDefault) != hipSuccess) {
      (void)hipGetLastError();
      prc = H2O4GPU_KMEANS_EALLOC;
    }
    int idx = pick(nullptr);
    for (int c = 0; c < k && prc == 0; c++) {
      seed_info.chosen[(size_t)c] = idx;
      w[(size_t)idx] = 0;
      if (c == k - 1) break;
      prof_begin("seed_pick");
      prc = launch_candidate_dists<T>(stream, *Cc, CcT, *ccn, idx, *best, hbest, M, d, c == 0);
      prof_end();
      if (prc == 0 && hipStreamSynchronize(stream) != hipSuccess) prc = H2O4GPU_KMEANS_EDEVICE;
      if (prc == 0) idx = pick(hbest);
    }
    (void)hipStreamSynchronize(stream);
    if (hbest) (void)hipHostFree(hbest);
    if (CcT) (void)hipFree(CcT);
    KM_TRY(prc);
    std::vector<int> rows((size_t)k);
    for (int c = 0; c < k; c++) rows[(size_t)c] = all[(size_t)seed_info.chosen[(size_t)c]];
    last_seed_rows = rows;
    return init_from_rows(rows.data());
  }

  // The fused kernels compute the centroid norms themselves, so a Lloyd loop that needs no
  // convergence scalar skips the post-update launch and leaves cnorm behind the current
  // centroids; every other consumer of cnorm refreshes it first.
  bool cnorm_stale = false;
  int ensure_cnorm() {
    if (!cnorm_stale) return 0;
    PROFILED("row_norms", launch_row_norms<T>(stream, C[cur], cnorm, k, d));
    cnorm_stale = false;
    return 0;
  }

  int assign() override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data || !have_centroids) return H2O4GPU_KMEANS_ESTATE;
    KM_TRY(ensure_cnorm());
    PROFILED("assign", launch_assign<T>(stream, opt_assign, X, xnorm, C[cur], cnorm,
                                        labels, mindist, n, d, k, num_cu, &last_variant,
                                        opt_exact != 0, shape(), opt_split, split_scratch()));
    have_mindist = true;
    return 0;
  }

  int update_async() {
    if (use_buckets && opt_buckets) {
      PROFILED("accumulate", launch_bucketed_accumulate<T>(stream, X, labels, order, order_label,
                                                           bucket_offsets, bucket_hist, bucket_seg,
                                                           bucket_total, bucket_partials, psums,
                                                           pcounts, n, d, k));
      return finish_update(1, true);
    }
    PROFILED("accumulate", launch_accumulate<T>(stream, plan, X, labels, psums, pcounts, n, d, k));
    return finish_update(plan.row_blocks, true);
  }

  // one Lloyd step: labels against the current centroids, then the update.
  // want_shift: the caller will read the convergence scalar of this step.
  // want_mindist false: the step need not leave the rows' minimum distances behind (a later
  // assignment pass will, before anyone reads them): one store per row less in the fused step.
  int step_async(bool want_shift, bool want_mindist = true) {
    // (the exact-compare argmin exists in the assignment-only kernels)
    const int fam = pick_assign_variant<T>(opt_assign, n, d, k);
    const bool exact_mfma = opt_exact && sizeof(T) == 4 && fam != ASSIGN_VALU && fam != ASSIGN_LONGROW;
    if ((opt_fuse || sets > 1) && !exact_mfma && fused_slots<T>(opt_assign, n, d, k, num_cu) > 0) {
      int slots = 0;
      PROFILED("assign_accumulate",
               launch_assign_accumulate<T>(stream, opt_assign, X, xnorm, C[cur], (const T *)nullptr,
                                           labels, (want_mindist || sets > 1) ? mindist : (T *)nullptr, n, d,
                                           k, num_cu, psums, pcounts, &slots, &last_variant, shape(),
                                           opt_split));
      have_mindist = want_mindist || sets > 1;
      return finish_update(slots, want_shift);
    }
    if (sets > 1) return H2O4GPU_KMEANS_ESTATE;  // a stacked handle has no other step
    KM_TRY(assign());
    return update_async();
  }

  // post: also run pass 3 (norms of the new centroids + the shift scalar). Without it the
  // norms are marked stale and the scalar of this step does not exist.
  int finish_update(int slots, bool post) {
    int nsp = 0;
    if (sets > 1 && post) {
      // per-set convergence: frozen sets keep their centroids; every set's squared shift is
      // the ordered sum of its own partials
      PROFILED("finalize", launch_finalize<T>(stream, slots, psums, pcounts, C[cur], C[cur ^ 1],
                                              counts, shift_partials, &nsp, d, k, d_frozen, kps));
      const int per = nsp / sets;
      for (int s = 0; s < sets; s++)
        PROFILED("post_update",
                 launch_post_update<T>(stream, C[cur ^ 1] + (size_t)s * kps * d, cnorm + (size_t)s * kps,
                                       shift_partials + (size_t)s * per, per, shift2 + s, d, kps));
      cnorm_stale = false;
      cur ^= 1;
      return 0;
    }
    PROFILED("finalize", launch_finalize<T>(stream, slots, psums, pcounts, C[cur], C[cur ^ 1],
                                            counts, shift_partials, &nsp, d, k));
    if (post)
      PROFILED("post_update", launch_post_update<T>(stream, C[cur ^ 1], cnorm, shift_partials,
                                                    nsp, shift2, d, k));
    cnorm_stale = !post;
    cur ^= 1;
    return 0;
  }

  int read_shift2(double *out) {
    T v;
    KM_HIP_TRY(hipMemcpyAsync(&v, shift2, sizeof(T), hipMemcpyDeviceToHost, stream));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    *out = (double)v;
    return 0;
  }

  int update(double *s2) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data || !have_centroids || sets > 1) return H2O4GPU_KMEANS_ESTATE;
    KM_TRY(update_async());
    if (s2) KM_TRY(read_shift2(s2));
    return 0;
  }

  // kmeans_impl.h:109-232. The convergence scalar is only fetched when it can
  // matter (threshold > 0): shift^2 >= 0 can never be below a threshold <= 0,
  // so a fixed-iteration run has no host synchronisation inside the loop.
  int fit(int max_iterations, double threshold, int *iters) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data || !have_centroids) return H2O4GPU_KMEANS_ESTATE;
    maybe_install_signal_handlers();
    int updates = 0;
    if (max_iterations <= 0) {
      // The reference's loop then never runs, its final relabel included, and the labels it
      // returns are the zeros its vector was created with (kmeans_impl.h:109-232,
      // kmeans_h2o4gpu.cu:747); the centroids stay the starting ones. No minimum distances,
      // hence no inertia, exist for such a fit.
      KM_HIP_TRY(hipMemsetAsync(labels, 0, (size_t)n * sets * sizeof(int), stream));
      have_mindist = false;
    } else if (sets > 1) {
      KM_TRY(fit_stacked(max_iterations, threshold, &updates));
    } else if (threshold > 0 && max_iterations > 0) {
      KM_TRY(fit_with_threshold(max_iterations, threshold, &updates));
    } else {
      for (int i = 0; i < max_iterations; i++) {
        log_msg(verbose, LOG_VERBOSE, "KMeans - Iteration %d/%d", i, max_iterations);
        KM_TRY(step_async(false, false));  // (the final relabel below leaves the minimum distances)
        updates++;
        bool done = false;
        if (g_stop_flag) {
          fprintf(stderr, "Signal caught. Terminated early.\n");
          g_stop_flag = 0;
          done = true;
        }
        if (done || i == max_iterations - 1) {
          KM_TRY(assign());  // final relabel with the final centroids
          break;
        }
      }
    }
    KM_HIP_TRY(hipStreamSynchronize(stream));
    if (iters) *iters = updates;
    return 0;
  }

  // Every set of a stacked handle runs the loop of kmeans_impl.h:109-232 on its own: the
  // same kernel labels the rows against all sets and sums them per set; with a threshold,
  // a set whose squared shift falls below it keeps its centroids from then on (its labels
  // are still refreshed, and stay what its final relabel would give) while the others go
  // on. The scalars of an iteration are read before the next one is queued: unlike the
  // single-set loop this one waits for the host once per iteration.
  int fit_stacked(int max_iterations, double threshold, int *updates_out) {
    const bool test = threshold > 0;
    std::vector<int> frozen((size_t)sets, 0);
    std::vector<T> sh((size_t)sets);
    set_iterations.assign((size_t)sets, 0);
    KM_HIP_TRY(hipMemsetAsync(d_frozen, 0, (size_t)sets * sizeof(int), stream));
    int updates = 0, live = sets;
    for (int i = 0; i < max_iterations && live > 0; i++) {
      KM_TRY(step_async(test));
      updates = i + 1;
      for (int s = 0; s < sets; s++)
        if (!frozen[(size_t)s]) set_iterations[(size_t)s] = i + 1;
      if (test) {
        KM_HIP_TRY(hipMemcpyAsync(sh.data(), shift2, (size_t)sets * sizeof(T), hipMemcpyDeviceToHost, stream));
        KM_HIP_TRY(hipStreamSynchronize(stream));
        bool changed = false;
        for (int s = 0; s < sets; s++) {
          if (!frozen[(size_t)s] && (double)sh[(size_t)s] < threshold) {
            frozen[(size_t)s] = 1;
            changed = true;
            live--;
          }
        }
        if (changed)
          KM_HIP_TRY(hipMemcpyAsync(d_frozen, frozen.data(), (size_t)sets * sizeof(int), hipMemcpyHostToDevice,
                                    stream));
      }
      if (g_stop_flag) {
        fprintf(stderr, "Signal caught. Terminated early.\n");
        g_stop_flag = 0;
        break;
      }
    }
    if (max_iterations > 0) KM_TRY(relabel_sets());  // final relabel of every set with its final centroids
    *updates_out = updates;
    return 0;
  }

  // The final relabel of a stacked fit, one set at a time as an ordinary model of kset
  // centroids: the kernels (and hence the labels and minimum distances, near-ties included)
  // are those a handle of one set runs on these centroids, so predicting the training rows
  // with the winning centroids gives back its labels whichever way the restarts ran.
  int relabel_sets() {
    const size_t kpad = ((size_t)kset + CENTROID_PAD - 1) / CENTROID_PAD * CENTROID_PAD;
    T *Cp = nullptr, *cn = nullptr;
    KM_TRY(dalloc(&Cp, kpad * d));
    int rc = dalloc(&cn, kpad);
    const std::vector<T> inf(kpad, std::numeric_limits<T>::infinity());
    for (int s = 0; s < sets && rc == 0; s++) {
      // padded like an ordinary model: zero rows with +inf norms past the last centroid
      if (hipMemsetAsync(Cp, 0, kpad * d * sizeof(T), stream) != hipSuccess ||
          hipMemcpyAsync(Cp, C[cur] + (size_t)s * kps * d, (size_t)kset * d * sizeof(T),
                         hipMemcpyDeviceToDevice, stream) != hipSuccess ||
          hipMemcpyAsync(cn, inf.data(), kpad * sizeof(T), hipMemcpyHostToDevice, stream) != hipSuccess ||
          hipStreamSynchronize(stream) != hipSuccess) {
        rc = H2O4GPU_KMEANS_EDEVICE;
        break;
      }
      prof_begin("row_norms");
      rc = launch_row_norms<T>(stream, Cp, cn, kset, d);
      prof_end();
      if (rc != 0) break;
      prof_begin("assign");
      rc = launch_assign<T>(stream, opt_assign, X, xnorm, Cp, cn, labels + (size_t)s * n,
                            mindist + (size_t)s * n, n, d, kset, num_cu, &last_variant, opt_exact != 0,
                            StackShape(), opt_split, split_scratch(kset));
      prof_end();
    }
    (void)hipStreamSynchronize(stream);
    if (Cp) (void)hipFree(Cp);
    if (cn) (void)hipFree(cn);
    KM_TRY(rc);
    have_mindist = true;
    return 0;
  }

  // The loop with a convergence test (kmeans_impl.h:189-232: stop after the update whose
  // squared shift is below the threshold, then relabel with the final centroids). The
  // scalar of iteration i travels to pinned host memory while iteration i+1 is already
  // queued, so the device never waits for the host. When iteration i turns out to be the
  // last one, the queued iteration's assignment pass IS the final relabel (it ran with the
  // centroids of update i); only its centroid update is dropped: the buffers are flipped
  // back and the centroid norms recomputed.
  T *host_shift = nullptr;            // [2] pinned
  hipEvent_t shift_ready[2] = {nullptr, nullptr};
  int fit_with_threshold(int max_iterations, double threshold, int *updates_out) {
    if (!host_shift) {
      KM_HIP_TRY(hipHostMalloc(reinterpret_cast<void **>(&host_shift), 2 * sizeof(T), hipHostMallocDefault));
      for (int i = 0; i < 2; i++)
        KM_HIP_TRY(hipEventCreateWithFlags(&shift_ready[i], hipEventDisableTiming));
    }
    auto queue_iteration = [&](int i) -> int {
      log_msg(verbose, LOG_VERBOSE, "KMeans - Iteration %d/%d", i, max_iterations);
      KM_TRY(step_async(true));
      KM_HIP_TRY(hipMemcpyAsync(host_shift + (i & 1), shift2, sizeof(T), hipMemcpyDeviceToHost, stream));
      KM_HIP_TRY(hipEventRecord(shift_ready[i & 1], stream));
      return 0;
    };
    KM_TRY(queue_iteration(0));
    int updates = 0;
    for (int i = 0; i < max_iterations; i++) {
      const bool queued_next = i + 1 < max_iterations;
      if (queued_next) KM_TRY(queue_iteration(i + 1));
      KM_HIP_TRY(hipEventSynchronize(shift_ready[i & 1]));
      updates = i + 1;
      bool done = (double)host_shift[i & 1] < threshold;
      if (done) log_msg(verbose, LOG_INFO, "Threshold triggered. Terminating early.");
      if (g_stop_flag) {
        fprintf(stderr, "Signal caught. Terminated early.\n");
        g_stop_flag = 0;
        done = true;
      }
      if (!done && queued_next) continue;
      if (queued_next) {
        // labels and minimum distances of the queued iteration are the final relabel
        cur ^= 1;
        PROFILED("row_norms", launch_row_norms<T>(stream, C[cur], cnorm, k, d));
        cnorm_stale = false;
      } else {
        KM_TRY(assign());
      }
      break;
    }
    *updates_out = updates;
    return 0;
  }

  int iterate(int steps) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data || !have_centroids) return H2O4GPU_KMEANS_ESTATE;
    // only the last step's minimum distances can be read afterwards
    for (int i = 0; i < steps; i++) KM_TRY(step_async(false, i == steps - 1));
    return 0;
  }

  int set_labels_host(const int *h) override {
    if (sets > 1) return H2O4GPU_KMEANS_ESTATE;
    KM_HIP_TRY(hipSetDevice(dev));
    KM_HIP_TRY(hipMemcpyAsync(labels, h, (size_t)n * sizeof(int), hipMemcpyHostToDevice, stream));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }
  int d2h(void *dst, const void *src, size_t bytes) {
    KM_HIP_TRY(hipSetDevice(dev));
    KM_TRY(download_rows(dev, stream, dst, src, bytes));  // staged when large (labels of 10M rows)
    KM_HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }
  int get_centroids(void *out) override {
    return d2h(out, C[cur] + set_off() * d, (size_t)kk() * d * sizeof(T));
  }
  int get_labels(int *out) override { return d2h(out, labels + row_off(), (size_t)n * sizeof(int)); }
  int get_counts(int *out) override { return d2h(out, counts + set_off(), (size_t)kk() * sizeof(int)); }
  int get_min_distances(void *out) override {
    if (!have_mindist) return H2O4GPU_KMEANS_ESTATE;
    return d2h(out, mindist + row_off(), (size_t)n * sizeof(T));
  }
  int inertia(double *out) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_mindist) return H2O4GPU_KMEANS_ESTATE;
    const int np = sum_partials_needed();
    PROFILED("inertia_sum", launch_sum<T>(stream, mindist + row_off(), n, sum_partials, np, sum_partials + np));
    return d2h(out, sum_partials + np, sizeof(double));
  }

  int predict_host(size_t rows, const void *hX, int *out) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_centroids || sets > 1) return H2O4GPU_KMEANS_ESTATE;
    if (rows == 0) return 0;
    T *dX = nullptr, *dxn = nullptr, *dmin = nullptr;
    int *dl = nullptr;
    int rc = dalloc(&dX, rows * d);
    if (rc == 0) rc = dalloc(&dxn, rows);
    if (rc == 0) rc = dalloc(&dl, rows);
    // running minimum per row: a model swept in chunks of centroids merges through it
    if (rc == 0) rc = dalloc(&dmin, rows);
    if (rc == 0) rc = run_predict(rows, hX, out, dX, dxn, dl, dmin);
    (void)hipStreamSynchronize(stream);
    if (dX) (void)hipFree(dX);
    if (dxn) (void)hipFree(dxn);
    if (dl) (void)hipFree(dl);
    if (dmin) (void)hipFree(dmin);
    return rc;
  }
  int run_predict(size_t rows, const void *hX, int *out, T *dX, T *dxn, int *dl, T *dmin) {
    KM_TRY(ensure_cnorm());
    // Large inputs go up in pieces, and the kernels of a piece are queued as soon as it has
    // arrived: they run while the host threads and the copy engine move the next piece, so
    // the call takes the transfer plus the last piece's kernels instead of the sum of both
    // (2M x 256, k = 1024: 51.5 -> 42.7 ms; 500k x 784, k = 4096: 34.9 ms for a transfer of
    // 30 ms and a kernel of 26 ms). The staged transfer returns when its bytes are on the device.
    const size_t row_bytes = (size_t)d * sizeof(T);
    size_t piece = rows;
    if (rows * row_bytes >= ((size_t)128 << 20)) {
      piece = std::max<size_t>((rows + 7) / 8, ((size_t)32 << 20) / row_bytes);
      piece = (piece + 1023) / 1024 * 1024;
    }
    const SplitScratch scratch = split_scratch();  // (before the first launch: it may drain the stream)
    for (size_t lo = 0; lo < rows; lo += piece) {
      const size_t cnt = std::min(piece, rows - lo);
      KM_TRY(upload_rows(dev, stream, dX + lo * d, static_cast<const T *>(hX) + lo * d, cnt * row_bytes, lo == 0));
      PROFILED("row_norms", launch_row_norms<T>(stream, dX + lo * d, dxn + lo, (int64_t)cnt, d));
      PROFILED("assign", launch_assign<T>(stream, opt_assign, dX + lo * d, dxn + lo, C[cur], cnorm, dl + lo,
                                          dmin + lo, (int64_t)cnt, d, k, num_cu, &last_variant,
                                          opt_exact != 0, StackShape(), opt_split, scratch));
    }
    KM_TRY(download_rows(dev, stream, out, dl, rows * sizeof(int)));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }

  // The n x k result is produced in row batches of at most ~4 GB so the device
  // buffer stays bounded; the reference materialises it whole ("TODO batch
  // this", kmeans_h2o4gpu.cu:936). With more than one batch there are two sets of device
  // buffers: the kernels of batch i + 1 are queued before the host starts to bring batch i
  // back, so they run under that download, and a batch's [k][its rows] block goes through
  // the pinned staging buffers into its columns of the caller's [k][rows] matrix (a strided
  // copy straight into pageable memory moved a quarter of the bytes per second).
  int transform_host(size_t rows, const void *hX, void *hD) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_centroids || sets > 1) return H2O4GPU_KMEANS_ESTATE;
    if (rows == 0) return 0;
    size_t batch = ((size_t)opt_transform_batch_mb << 20) / ((size_t)k * sizeof(T));
    batch = batch / 128 * 128;
    if (batch < 128) batch = 128;
    if (batch > rows) batch = rows;
    const size_t nbatch = (rows + batch - 1) / batch;
    int nbuf = nbatch > 1 && opt_transform_buffers == 2 ? 2 : 1;
    T *dX[2] = {nullptr, nullptr}, *dxn[2] = {nullptr, nullptr}, *dD[2] = {nullptr, nullptr};
    hipEvent_t ready[2] = {nullptr, nullptr};
    int rc = ensure_cnorm();
    for (int b = 0; b < nbuf && rc == 0; b++) {
      int arc = dalloc(&dX[b], batch * d);
      if (arc == 0) arc = dalloc(&dxn[b], batch);
      if (arc == 0) arc = dalloc(&dD[b], batch * k);
      if (arc == 0 && hipEventCreateWithFlags(&ready[b], hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        arc = H2O4GPU_KMEANS_EDEVICE;
      }
      if (arc != 0 && b == 1) {
        // no room for the second set: one batch at a time, each downloaded before the next is computed
        if (dX[1]) (void)hipFree(dX[1]);
        if (dxn[1]) (void)hipFree(dxn[1]);
        if (dD[1]) (void)hipFree(dD[1]);
        if (ready[1]) (void)hipEventDestroy(ready[1]);
        dX[1] = dxn[1] = dD[1] = nullptr;
        ready[1] = nullptr;
        nbuf = 1;
        break;
      }
      rc = arc;
    }
    const SplitScratch scratch = rc == 0 ? split_scratch() : SplitScratch();
    // upload + kernels of batch i, left running
    auto queue_batch = [&](size_t i) -> int {
      const size_t lo = i * batch, cur_rows = std::min(batch, rows - lo);
      const int b = (int)(i % (size_t)nbuf);
      // (nothing on the stream touches this buffer: its last kernels ended before the
      // download of batch i - 2 returned)
      KM_TRY(upload_rows(dev, stream, dX[b], static_cast<const T *>(hX) + lo * d, cur_rows * d * sizeof(T),
                         false));
      PROFILED("row_norms", launch_row_norms<T>(stream, dX[b], dxn[b], (int64_t)cur_rows, d));
      PROFILED("transform", launch_transform<T>(stream, dX[b], dxn[b], C[cur], cnorm, dD[b],
                                                (int64_t)cur_rows, (int64_t)cur_rows, d, k, num_cu,
                                                opt_split, scratch));
      KM_HIP_TRY(hipEventRecord(ready[b], stream));
      return 0;
    };
    if (rc == 0) rc = queue_batch(0);
    for (size_t i = 0; rc == 0 && i < nbatch; i++) {
      if (i > 0 && nbuf == 1) rc = queue_batch(i);  // (the only buffers are free again)
      if (nbuf == 2 && i + 1 < nbatch && rc == 0) rc = queue_batch(i + 1);
      if (rc != 0) break;
      const size_t lo = i * batch, cur_rows = std::min(batch, rows - lo);
      const int b = (int)(i % (size_t)nbuf);
      T *dst = static_cast<T *>(hD) + lo;
      if (nbatch == 1) {  // one contiguous [k][rows] block
        rc = download_rows(dev, stream, dst, dD[b], (size_t)k * rows * sizeof(T));
        if (rc == 0 && hipStreamSynchronize(stream) != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
      } else {
        rc = download_matrix(dev, stream, dst, rows * sizeof(T), dD[b], cur_rows * sizeof(T), (size_t)k,
                             ready[b]);
      }
    }
    (void)hipStreamSynchronize(stream);
    for (int b = 0; b < 2; b++) {
      if (dX[b]) (void)hipFree(dX[b]);
      if (dxn[b]) (void)hipFree(dxn[b]);
      if (dD[b]) (void)hipFree(dD[b]);
      if (ready[b]) (void)hipEventDestroy(ready[b]);
    }
    return rc;
  }
  int transform_resident(void *d_dist) override {
    KM_HIP_TRY(hipSetDevice(dev));
    if (!have_data || !have_centroids || !d_dist || sets > 1) return H2O4GPU_KMEANS_ESTATE;
    KM_TRY(ensure_cnorm());
    PROFILED("transform", launch_transform<T>(stream, X, xnorm, C[cur], cnorm,
                                              static_cast<T *>(d_dist), n, n, d, k, num_cu, opt_split,
                                              split_scratch()));
    KM_HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }
};

template <typename T>
static int create_engine(h2o4gpu_kmeans_handle **out, size_t rows, size_t cols, int k,
                         int gpu_id, int verbose, int sets = 1) {
  const int nvis = visible_devices();
  if (nvis < 1) {
    log_msg(verbose ? verbose : LOG_ERROR, LOG_ERROR, "no HIP device visible");
    return H2O4GPU_KMEANS_EDEVICE;
  }
  Engine<T> *e = new (std::nothrow) Engine<T>();
  if (!e) return H2O4GPU_KMEANS_EALLOC;
  e->elem_size = sizeof(T);
  e->n = (int64_t)rows;
  e->d = (int)cols;
  e->k = k;
  if (sets > 1) {
    e->sets = sets;
    e->kset = k;
    e->kps = (k + 31) / 32 * 32;
    e->k = sets * e->kps;
  }
  e->verbose = verbose;
  // The reference's entry points have no argument for it: H2O4GPU_KMEANS_FP32_SPLIT=6 (or 9)
  // in the environment turns the "fp32_split" option on for every handle created afterwards.
  if (const char *env = getenv("H2O4GPU_KMEANS_FP32_SPLIT")) {
    const int v = atoi(env);
    if (v == 6 || v == 9) e->opt_split = v;
  }
  if (gpu_id < 0) gpu_id = 0;
  e->dev = gpu_id % nvis;  // kmeans_init: gpu_id = gpu_idtry % n_gpuvis
  int rc = e->create();
  if (rc != 0) {
    e->release();
    delete e;
    return rc;
  }
  *out = e;
  return 0;
}

}  // namespace kmhip

#define KM_API __attribute__((visibility("default")))
extern "C" KM_API int h2o4gpu_kmeans_create(h2o4gpu_kmeans_handle **out, int elem_size, size_t rows,
                                            size_t cols, int k, int gpu_id, int verbose);
extern "C" KM_API int h2o4gpu_kmeans_destroy(h2o4gpu_kmeans_handle *h);

__global__ void copy_probe_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst,
                                  size_t nvec) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride)
    dst[i] = src[i];
}

// Read-only stream: every thread keeps four 16-byte loads in flight and adds what arrives;
// one value per thread leaves at the end (so the loads cannot be dropped).
typedef float floatx4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void read_probe_kernel(const floatx4 *__restrict__ src,
                                                         float *__restrict__ out, size_t nvec) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  floatx4 a0 = {0, 0, 0, 0}, a1 = a0, a2 = a0, a3 = a0;
  for (; i + 3 * stride < nvec; i += 4 * stride) {
    // (loads that do not displace cached lines: 6.0 against 5.5 TB/s with plain ones)
    const floatx4 v0 = __builtin_nontemporal_load(&src[i]), v1 = __builtin_nontemporal_load(&src[i + stride]),
                  v2 = __builtin_nontemporal_load(&src[i + 2 * stride]),
                  v3 = __builtin_nontemporal_load(&src[i + 3 * stride]);
    a0.x += v0.x; a0.y += v0.y; a0.z += v0.z; a0.w += v0.w;
    a1.x += v1.x; a1.y += v1.y; a1.z += v1.z; a1.w += v1.w;
    a2.x += v2.x; a2.y += v2.y; a2.z += v2.z; a2.w += v2.w;
    a3.x += v3.x; a3.y += v3.y; a3.z += v3.z; a3.w += v3.w;
  }
  for (; i < nvec; i += stride) {
    const floatx4 v0 = src[i];
    a0.x += v0.x; a0.y += v0.y; a0.z += v0.z; a0.w += v0.w;
  }
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] =
      (a0.x + a0.y + a0.z + a0.w) + (a1.x + a1.y + a1.z + a1.w) + (a2.x + a2.y + a2.z + a2.w) +
      (a3.x + a3.y + a3.z + a3.w);
}
// Write-only stream.
__global__ __launch_bounds__(256) void fill_probe_kernel(float4 *__restrict__ dst, size_t nvec, float v) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const float4 val = {v, v, v, v};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) dst[i] = val;
}

// ---------------------------------------------------------------------------
// C ABI, part 1: the reference's entry points
// ---------------------------------------------------------------------------
// Inertia and iteration count of the calling thread's most recent successful fit
// through make_ptr_*_kmeans: the reference's signature has no slot for either.
struct LastFitInfo {
  bool valid = false;
  double inertia = 0.0;
  int iterations = 0;
};
static thread_local LastFitInfo g_last_fit;

template <typename T>
static int fit_entry(int verbose, int seed, int gpu_id, size_t rows, size_t cols, int k,
                     int max_iterations, int init_from_data, double threshold,
                     const T *srcdata, const T *centroids, T **pred_centroids,
                     int **pred_labels) {
  if (!srcdata || !pred_centroids || !pred_labels || rows < 1 || cols < 1 || k < 1)
    return H2O4GPU_KMEANS_EARG;
  if ((size_t)k > rows) {  // kmeans_h2o4gpu.cu:630-635
    k = (int)rows;
    fprintf(stderr, "Number of clusters adjusted to be equal to number of rows.\n");
    fflush(stderr);
  }
  h2o4gpu_kmeans_handle *h = nullptr;
  KM_TRY(h2o4gpu_kmeans_create(&h, sizeof(T), rows, cols, k, gpu_id, verbose));
  // the seeded permutation behind the random-row start is host work that needs only the
  // row count: it runs beside the upload
  std::vector<int> start_rows;
  std::thread row_picker;
  if (init_from_data == 0 && seed >= 0) {
    start_rows.resize((size_t)k);
    row_picker = std::thread(first_rows_of_shuffle, (int64_t)rows, k, (unsigned)seed,
                             start_rows.data());
  }
  int rc = h->set_data_host(srcdata);
  if (row_picker.joinable()) row_picker.join();
  if (rc == 0) {
    if (init_from_data == 0) {
      rc = start_rows.empty() ? h->init_random_rows(seed) : h->start_from_rows(start_rows.data());
    } else if (init_from_data == 1) {
      rc = h->init_parallel(seed);  // k-means||, as the reference (kmeans_h2o4gpu.cu:733-737)
    } else if (init_from_data == 2) {
      rc = centroids ? h->set_centroids_host(centroids) : H2O4GPU_KMEANS_EARG;
    } else if (init_from_data == 3) {
      rc = h->init_plusplus(seed);  // extension: k-means++ (D^2 sampling)
    } else {
      // the reference has no branch for other values and runs from all-zero
      // centroids (kmeans_h2o4gpu.cu:684-740); same here
      std::vector<T> zeros((size_t)k * cols, (T)0);
      rc = h->set_centroids_host(zeros.data());
    }
  }
  int iters = 0;
  double inertia = 0.0;
  g_last_fit.valid = false;
  if (rc == 0) rc = h->fit(max_iterations, threshold, &iters);
  // minimum distances of the final relabel; a run of zero iterations has none
  bool have_inertia = false;
  if (rc == 0) have_inertia = h->inertia(&inertia) == 0;
  T *oc = nullptr;
  int *ol = nullptr;
  if (rc == 0) {
    oc = static_cast<T *>(malloc((size_t)k * cols * sizeof(T)));
    ol = static_cast<int *>(malloc(rows * sizeof(int)));
    if (!oc || !ol) rc = H2O4GPU_KMEANS_EALLOC;
  }
  if (rc == 0) rc = h->get_centroids(oc);
  if (rc == 0) rc = h->get_labels(ol);
  h2o4gpu_kmeans_destroy(h);
  if (rc != 0) {
    free(oc);
    free(ol);
    // kmeans_h2o4gpu.cu:758-761
    log_msg(verbose, LOG_ERROR, "KMeans algorithm failed (%d).", rc);
    return rc;
  }
  *pred_centroids = oc;
  *pred_labels = ol;
  g_last_fit.valid = have_inertia;
  g_last_fit.inertia = inertia;
  g_last_fit.iterations = iters;
  log_msg(verbose, LOG_INFO, "fit: %d iterations, inertia %.9g", iters, inertia);
  return 0;
}

template <typename T>
static int predict_entry(int verbose, int gpu_id, size_t rows, size_t cols, int k,
                         const T *srcdata, const T *centroids, int **pred_labels) {
  if (!srcdata || !centroids || !pred_labels || rows < 1 || cols < 1 || k < 1)
    return H2O4GPU_KMEANS_EARG;
  h2o4gpu_kmeans_handle *h = nullptr;
  // a predict handle needs no resident rows: size its working set for one row
  KM_TRY(h2o4gpu_kmeans_create(&h, sizeof(T), (size_t)std::max(k, 1), cols, k, gpu_id, verbose));
  int rc = h->set_centroids_host(centroids);
  int *ol = nullptr;
  if (rc == 0) {
    ol = static_cast<int *>(malloc(rows * sizeof(int)));
    if (!ol) rc = H2O4GPU_KMEANS_EALLOC;
  }
  if (rc == 0) rc = h->predict_host(rows, srcdata, ol);
  h2o4gpu_kmeans_destroy(h);
  if (rc != 0) {
    free(ol);
    return rc;
  }
  *pred_labels = ol;
  return 0;
}

template <typename T>
static int transform_entry(int verbose, int gpu_id, size_t rows, size_t cols, int k,
                           const T *srcdata, const T *centroids, T **preds) {
  if (!srcdata || !centroids || !preds || rows < 1 || cols < 1 || k < 1)
    return H2O4GPU_KMEANS_EARG;
  h2o4gpu_kmeans_handle *h = nullptr;
  KM_TRY(h2o4gpu_kmeans_create(&h, sizeof(T), (size_t)std::max(k, 1), cols, k, gpu_id, verbose));
  int rc = h->set_centroids_host(centroids);
  T *out = nullptr;
  if (rc == 0) {
    out = static_cast<T *>(malloc(rows * (size_t)k * sizeof(T)));
    if (!out) rc = H2O4GPU_KMEANS_EALLOC;
  }
  if (rc == 0) rc = h->transform_host(rows, srcdata, out);
  h2o4gpu_kmeans_destroy(h);
  if (rc != 0) {
    free(out);
    return rc;
  }
  *preds = out;
  return 0;
}


// ---------------------------------------------------------------------------
// C ABI, part 4: assignment of device-resident rows without any allocation
// ---------------------------------------------------------------------------
// Everything predict_host obtains from hipMalloc beyond the caller's inputs and outputs
// (row norms, running minimum distances, the zero-padded copy of the centroids and their
// norms) lives in this fixed array instead. Every device the library runs on holds its
// own copy for the life of the process. In host code the name `scratch` is only a
// stand-in for the symbol: the device address is asked for once per device and it is
// that address, never the name, that kernels receive.
static __device__ __align__(256) unsigned char scratch[H2O4GPU_KMEANS_NOALLOC_SCRATCH_BYTES];

struct NoAllocDevice {
  unsigned char *ptr = nullptr;  // device address of `scratch` on this device
  int num_cu = 0;
};
static std::mutex g_noalloc_mu;
static NoAllocDevice g_noalloc[StagingPool::MAX_DEV];
static void forget_noalloc(int dev) {
  std::lock_guard<std::mutex> lock(g_noalloc_mu);
  if (dev >= 0 && dev < StagingPool::MAX_DEV) g_noalloc[dev] = NoAllocDevice();
}

// Cpad [kpad][d] = C [k][d] followed by zero rows; cnorm [k, kpad) = +inf.
template <typename T>
__global__ __launch_bounds__(256) void stage_model_kernel(const T *__restrict__ C, T *__restrict__ Cpad,
                                                          T *__restrict__ cnorm, int k, int kpad, int d) {
  const size_t kd = (size_t)k * d, total = (size_t)kpad * d;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t t0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (size_t e = t0; e < total; e += stride) Cpad[e] = e < kd ? C[e] : (T)0;
  for (size_t c = (size_t)k + t0; c < (size_t)kpad; c += stride)
    cnorm[c] = std::numeric_limits<T>::infinity();
}

// Address of this device's copy of `scratch` and the device's CU count, looked up on the
// first call on a device (which must be current). A plain function, not a template: the
// device compilation only gives a file-scope static variable a symbol the runtime can find
// when it sees ordinary host code name it.
static int noalloc_device(NoAllocDevice *out) {
  int dev = 0;
  KM_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= StagingPool::MAX_DEV) return H2O4GPU_KMEANS_EDEVICE;
  std::lock_guard<std::mutex> lock(g_noalloc_mu);
  if (!g_noalloc[dev].ptr) {
    void *p = nullptr;
    KM_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    hipDeviceProp_t prop;
    KM_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    g_noalloc[dev].num_cu = prop.multiProcessorCount;
    g_noalloc[dev].ptr = static_cast<unsigned char *>(p);
  }
  *out = g_noalloc[dev];
  return 0;
}

template <typename T>
static int predict_device_noalloc(size_t rows, size_t cols, int k, const T *dX, const T *dC,
                                  int *d_labels, hipStream_t stream) {
  NoAllocDevice nd;
  KM_TRY(noalloc_device(&nd));
  const int d = (int)cols;
  const size_t kpad = ((size_t)k + CENTROID_PAD - 1) / CENTROID_PAD * CENTROID_PAD;
  auto up = [](size_t b) { return (b + 255) / 256 * 256; };
  const size_t b_model = up(kpad * cols * sizeof(T)), b_cnorm = up(kpad * sizeof(T));
  const size_t b_rows = up(rows * sizeof(T));
  const size_t need = b_model + b_cnorm + 2 * b_rows;
  if (need > (size_t)H2O4GPU_KMEANS_NOALLOC_SCRATCH_BYTES) {
    log_msg(LOG_ERROR, LOG_ERROR,
            "predict_device_noalloc: rows=%zu cols=%zu k=%d need %zu bytes of scratch, the "
            "library's fixed buffer holds %zu; split the rows or use a handle",
            rows, cols, k, need, (size_t)H2O4GPU_KMEANS_NOALLOC_SCRATCH_BYTES);
    return H2O4GPU_KMEANS_ESCRATCH;
  }
  T *Cpad = reinterpret_cast<T *>(nd.ptr);
  T *cnorm = reinterpret_cast<T *>(nd.ptr + b_model);
  T *xnorm = reinterpret_cast<T *>(nd.ptr + b_model + b_cnorm);
  T *mind = reinterpret_cast<T *>(nd.ptr + b_model + b_cnorm + b_rows);
  // the array keeps the previous call's contents: everything read below is written first
  // (model rows and padding, all kpad norms, one norm per row; the running minimum is
  // written before it is read by every kernel that uses it)
  const size_t total = kpad * cols;
  const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 2048);
  hipLaunchKernelGGL((stage_model_kernel<T>), dim3(blocks), dim3(256), 0, stream, dC, Cpad, cnorm, k,
                     (int)kpad, d);
  KM_HIP_TRY(hipGetLastError());
  KM_TRY(launch_row_norms<T>(stream, Cpad, cnorm, k, d));
  KM_TRY(launch_row_norms<T>(stream, dX, xnorm, (int64_t)rows, d));
  return launch_assign<T>(stream, ASSIGN_AUTO, dX, xnorm, Cpad, cnorm, d_labels, mind, (int64_t)rows, d,
                          k, nd.num_cu, nullptr);
}

// Largest number of centroid sets (at most max_sets) of k centroids each that one stacked
// handle can hold for rows of `cols` values: the stacked model and its per-centroid sums
// must fit one CU's LDS beside each other. 1: no stacking for this shape.
template <typename T>
static int stack_width(size_t rows, size_t cols, int k, int max_sets) {
  const int kps = (k + 31) / 32 * 32;
  int best = 1;
  for (int s = 2; s <= max_sets; s++) {
    const int64_t K = (int64_t)s * kps;
    if (K > 65536) break;
    if (pick_assign_variant<T>(ASSIGN_AUTO, (int64_t)rows, (int)cols, (int)K) != ASSIGN_ROWSTAT) break;
    if (fused_slots<T>(ASSIGN_AUTO, (int64_t)rows, (int)cols, (int)K, 1) <= 0) break;
    best = s;
  }
  return best;
}

// ---------------------------------------------------------------------------
// C ABI, part 3
// ---------------------------------------------------------------------------
extern "C" {

#define KM_CHECK_HANDLE(h) \
  if (!(h)) return H2O4GPU_KMEANS_EARG

KM_API int h2o4gpu_kmeans_create(h2o4gpu_kmeans_handle **out, int elem_size, size_t rows,
                                 size_t cols, int k, int gpu_id, int verbose) {
  if (!out) return H2O4GPU_KMEANS_EARG;
  *out = nullptr;
  // rows must fit int32 (labels and row indices are int32, as in kmeans_init
  // kmeans_h2o4gpu.cu:574-579, which exits instead)
  // k may exceed rows (a shard can hold fewer rows than the model has centroids); only
  // the row-based starts need k <= rows
  if (rows < 1 || cols < 1 || k < 1 || rows > 2147483647ull || cols > 1000000ull)
    return H2O4GPU_KMEANS_EARG;
  if (elem_size == 4) return create_engine<float>(out, rows, cols, k, gpu_id, verbose);
  if (elem_size == 8) return create_engine<double>(out, rows, cols, k, gpu_id, verbose);
  return H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_stack_width(int elem_size, size_t rows, size_t cols, int k, int max_sets) {
  if (rows < 1 || cols < 1 || k < 1 || cols > 1000000ull || rows > 2147483647ull) return 1;
  if (elem_size == 4) return stack_width<float>(rows, cols, k, max_sets);
  if (elem_size == 8) return stack_width<double>(rows, cols, k, max_sets);
  return 1;
}
KM_API int h2o4gpu_kmeans_create_stacked(h2o4gpu_kmeans_handle **out, int elem_size, size_t rows,
                                         size_t cols, int k, int sets, int gpu_id, int verbose) {
  if (!out) return H2O4GPU_KMEANS_EARG;
  *out = nullptr;
  if (sets < 2) return h2o4gpu_kmeans_create(out, elem_size, rows, cols, k, gpu_id, verbose);
  if (rows < 1 || cols < 1 || k < 1 || rows > 2147483647ull || cols > 1000000ull ||
      sets > h2o4gpu_kmeans_stack_width(elem_size, rows, cols, k, sets))
    return H2O4GPU_KMEANS_EARG;
  if (elem_size == 4) return create_engine<float>(out, rows, cols, k, gpu_id, verbose, sets);
  if (elem_size == 8) return create_engine<double>(out, rows, cols, k, gpu_id, verbose, sets);
  return H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_select_set(h2o4gpu_kmeans_handle *h, int set) {
  KM_CHECK_HANDLE(h);
  if (set < 0 || set >= h->sets) return H2O4GPU_KMEANS_EARG;
  h->cur_set = set;
  return 0;
}
KM_API int h2o4gpu_kmeans_set_iterations(h2o4gpu_kmeans_handle *h, int *iterations) {
  KM_CHECK_HANDLE(h);
  if (!iterations || (int)h->set_iterations.size() != h->sets) return H2O4GPU_KMEANS_ESTATE;
  memcpy(iterations, h->set_iterations.data(), (size_t)h->sets * sizeof(int));
  return 0;
}
KM_API int h2o4gpu_kmeans_destroy(h2o4gpu_kmeans_handle *h) {
  KM_CHECK_HANDLE(h);
  h->release();
  delete h;
  return 0;
}
KM_API int h2o4gpu_kmeans_set_data_host(h2o4gpu_kmeans_handle *h, const void *X) {
  KM_CHECK_HANDLE(h);
  return h->set_data_host(X);
}
KM_API int h2o4gpu_kmeans_set_data_device(h2o4gpu_kmeans_handle *h, const void *dX) {
  KM_CHECK_HANDLE(h);
  return h->set_data_device(dX);
}
KM_API int h2o4gpu_kmeans_set_centroids_host(h2o4gpu_kmeans_handle *h, const void *C) {
  KM_CHECK_HANDLE(h);
  return h->set_centroids_host(C);
}
KM_API int h2o4gpu_kmeans_init_random_rows(h2o4gpu_kmeans_handle *h, int seed) {
  KM_CHECK_HANDLE(h);
  return h->init_random_rows(seed);
}
KM_API int h2o4gpu_kmeans_init_plusplus(h2o4gpu_kmeans_handle *h, int seed) {
  KM_CHECK_HANDLE(h);
  return h->init_plusplus(seed);
}
KM_API int h2o4gpu_kmeans_init_parallel(h2o4gpu_kmeans_handle *h, int seed) {
  KM_CHECK_HANDLE(h);
  return h->init_parallel(seed);
}
KM_API int h2o4gpu_kmeans_parallel_seed_info(h2o4gpu_kmeans_handle *h, int cap, int *cand_rows,
                                             int *n_candidates, int *round_count, double *phi,
                                             double *weights, int *chosen) {
  KM_CHECK_HANDLE(h);
  const auto &si = h->seed_info;
  if (si.cand_rows.empty()) return H2O4GPU_KMEANS_ESTATE;
  const int m = (int)si.cand_rows.size();
  if (n_candidates) *n_candidates = m;
  if (round_count) memcpy(round_count, si.round_count, sizeof(si.round_count));
  if (phi) memcpy(phi, si.phi, sizeof(si.phi));
  if (chosen) memcpy(chosen, si.chosen.data(), si.chosen.size() * sizeof(int));
  if (cand_rows || weights) {
    if (cap < m) return H2O4GPU_KMEANS_EARG;
    if (cand_rows) memcpy(cand_rows, si.cand_rows.data(), (size_t)m * sizeof(int));
    if (weights) {
      for (int c = 0; c < m; c++) weights[c] = si.weights.empty() ? 0.0 : si.weights[(size_t)c];
    }
  }
  return 0;
}
KM_API int h2o4gpu_kmeans_get_seed_rows(h2o4gpu_kmeans_handle *h, int *rows) {
  KM_CHECK_HANDLE(h);
  if (!rows || (int)h->last_seed_rows.size() != h->kk()) return H2O4GPU_KMEANS_ESTATE;
  memcpy(rows, h->last_seed_rows.data(), (size_t)h->kk() * sizeof(int));
  return 0;
}
KM_API int h2o4gpu_kmeans_fit(h2o4gpu_kmeans_handle *h, int max_iterations, double threshold,
                              int *iterations_run) {
  KM_CHECK_HANDLE(h);
  return h->fit(max_iterations, threshold, iterations_run);
}
KM_API int h2o4gpu_kmeans_assign(h2o4gpu_kmeans_handle *h) {
  KM_CHECK_HANDLE(h);
  int rc = h->assign();
  if (rc == 0 && hipStreamSynchronize(h->stream) != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
  return rc;
}
KM_API int h2o4gpu_kmeans_update(h2o4gpu_kmeans_handle *h, double *shift2) {
  KM_CHECK_HANDLE(h);
  int rc = h->update(shift2);
  if (rc == 0 && hipStreamSynchronize(h->stream) != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
  return rc;
}
KM_API int h2o4gpu_kmeans_set_labels_host(h2o4gpu_kmeans_handle *h, const int *labels) {
  KM_CHECK_HANDLE(h);
  if (!labels) return H2O4GPU_KMEANS_EARG;
  return h->set_labels_host(labels);
}
KM_API int h2o4gpu_kmeans_iterate(h2o4gpu_kmeans_handle *h, int steps) {
  KM_CHECK_HANDLE(h);
  return h->iterate(steps);
}
KM_API int h2o4gpu_kmeans_get_centroids(h2o4gpu_kmeans_handle *h, void *C) {
  KM_CHECK_HANDLE(h);
  return C ? h->get_centroids(C) : H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_get_labels(h2o4gpu_kmeans_handle *h, int *labels) {
  KM_CHECK_HANDLE(h);
  return labels ? h->get_labels(labels) : H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_get_counts(h2o4gpu_kmeans_handle *h, int *counts) {
  KM_CHECK_HANDLE(h);
  return counts ? h->get_counts(counts) : H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_get_min_distances(h2o4gpu_kmeans_handle *h, void *m) {
  KM_CHECK_HANDLE(h);
  return m ? h->get_min_distances(m) : H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_random_start_rows(int seed, size_t rows, int k, int *out) {
  if (!out || k < 1 || rows < (size_t)k || rows > 2147483647ull || seed < 0)
    return H2O4GPU_KMEANS_EARG;
  first_rows_of_shuffle((int64_t)rows, k, (unsigned)seed, out);
  return 0;
}

// 1 if every value is finite, 0 if one is an infinity or a NaN, negative on bad arguments.
// Host memory, host threads: the estimator's input check (solvers/utils.py:144-158 in the
// reference, two numpy passes with a temporary the size of the data) as one parallel pass.
KM_API int h2o4gpu_kmeans_host_all_finite(const void *data, size_t count, int elem_size) {
  if ((!data && count) || (elem_size != 4 && elem_size != 8)) return H2O4GPU_KMEANS_EARG;
  unsigned hw = std::thread::hardware_concurrency();
  int threads = (int)std::min(8u, hw ? hw : 1u);
  if (count < (1u << 20)) threads = 1;
  std::atomic<int> bad(0);
  auto scan = [&](size_t lo, size_t hi) {
    // a value is non-finite exactly when its exponent bits are all ones
    constexpr size_t BLOCK = 1 << 16;
    for (size_t b = lo; b < hi && !bad.load(std::memory_order_relaxed); b += BLOCK) {
      const size_t e = std::min(hi, b + BLOCK);
      unsigned long long any = 0;
      if (elem_size == 4) {
        const uint32_t *p = static_cast<const uint32_t *>(data);
        for (size_t i = b; i < e; i++) any |= (p[i] & 0x7F800000u) == 0x7F800000u;
      } else {
        const uint64_t *p = static_cast<const uint64_t *>(data);
        for (size_t i = b; i < e; i++) any |= (p[i] & 0x7FF0000000000000ull) == 0x7FF0000000000000ull;
      }
      if (any) bad.store(1, std::memory_order_relaxed);
    }
  };
  std::vector<std::thread> pool;
  const size_t per = (count + threads - 1) / threads;
  try {
    for (int t = 1; t < threads; t++)
      if (per * t < count) pool.emplace_back(scan, per * t, std::min(count, per * (t + 1)));
  } catch (...) {
    for (auto &th : pool) th.join();
    pool.clear();
    scan(per, count);  // whatever the threads would have covered
  }
  scan(0, std::min(per, count));
  for (auto &th : pool) th.join();
  return bad.load() ? 0 : 1;
}

KM_API int h2o4gpu_kmeans_last_fit_info(double *inertia, int *iterations) {
  if (!g_last_fit.valid) return H2O4GPU_KMEANS_ESTATE;
  if (inertia) *inertia = g_last_fit.inertia;
  if (iterations) *iterations = g_last_fit.iterations;
  return 0;
}

KM_API int h2o4gpu_kmeans_inertia(h2o4gpu_kmeans_handle *h, double *inertia) {
  KM_CHECK_HANDLE(h);
  return inertia ? h->inertia(inertia) : H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_predict_host(h2o4gpu_kmeans_handle *h, size_t rows, const void *X,
                                       int *labels) {
  KM_CHECK_HANDLE(h);
  if (rows > 0 && (!X || !labels)) return H2O4GPU_KMEANS_EARG;
  if (rows > 2147483647ull) return H2O4GPU_KMEANS_EARG;
  return h->predict_host(rows, X, labels);
}
KM_API int h2o4gpu_kmeans_transform_host(h2o4gpu_kmeans_handle *h, size_t rows, const void *X,
                                         void *dist) {
  KM_CHECK_HANDLE(h);
  if (rows > 0 && (!X || !dist)) return H2O4GPU_KMEANS_EARG;
  if (rows > 2147483647ull) return H2O4GPU_KMEANS_EARG;
  return h->transform_host(rows, X, dist);
}
KM_API int h2o4gpu_kmeans_transform_resident(h2o4gpu_kmeans_handle *h, void *d_dist) {
  KM_CHECK_HANDLE(h);
  return h->transform_resident(d_dist);
}
KM_API int h2o4gpu_kmeans_set_option(h2o4gpu_kmeans_handle *h, const char *name, int value) {
  KM_CHECK_HANDLE(h);
  if (!name) return H2O4GPU_KMEANS_EARG;
  if (strcmp(name, "assign") == 0) {
    if (value < ASSIGN_AUTO || value > ASSIGN_LONGROW) return H2O4GPU_KMEANS_EARG;
    h->opt_assign = value;
    return 0;
  }
  if (strcmp(name, "buckets") == 0) {
    if (value != 0 && value != 1) return H2O4GPU_KMEANS_EARG;
    h->opt_buckets = value;
    return 0;
  }
  if (strcmp(name, "exact_argmin") == 0) {
    if (value != 0 && value != 1) return H2O4GPU_KMEANS_EARG;
    h->opt_exact = value;
    return 0;
  }
  if (strcmp(name, "transform_batch_mb") == 0) {
    if (value < 1 || value > 65536) return H2O4GPU_KMEANS_EARG;
    h->opt_transform_batch_mb = value;
    return 0;
  }
  if (strcmp(name, "fp32_split") == 0) {
    if (value != 0 && value != 6 && value != 9) return H2O4GPU_KMEANS_EARG;
    h->opt_split = value;
    return 0;
  }
  if (strcmp(name, "fuse") == 0) {
    if (value != 0 && value != 1) return H2O4GPU_KMEANS_EARG;
    h->opt_fuse = value;
    return 0;
  }
  if (strcmp(name, "transform_buffers") == 0) {
    if (value != 1 && value != 2) return H2O4GPU_KMEANS_EARG;
    h->opt_transform_buffers = value;
    return 0;
  }
  if (strcmp(name, "tiled_direct") == 0) {
    if (value != 0 && value != 1) return H2O4GPU_KMEANS_EARG;
    h->opt_tiled_direct = value;
    return 0;
  }
  if (strcmp(name, "seed_matrix") == 0) {
    if (value != 0 && value != 1) return H2O4GPU_KMEANS_EARG;
    h->opt_seed_matrix = value;
    return 0;
  }
  return H2O4GPU_KMEANS_EARG;
}
KM_API int h2o4gpu_kmeans_timer_start(h2o4gpu_kmeans_handle *h) {
  KM_CHECK_HANDLE(h);
  KM_HIP_TRY(hipSetDevice(h->dev));
  if (!h->t0) KM_HIP_TRY(hipEventCreate(&h->t0));
  if (!h->t1) KM_HIP_TRY(hipEventCreate(&h->t1));
  KM_HIP_TRY(hipEventRecord(h->t0, h->stream));
  return 0;
}
KM_API int h2o4gpu_kmeans_timer_stop(h2o4gpu_kmeans_handle *h, float *ms) {
  KM_CHECK_HANDLE(h);
  if (!h->t0 || !h->t1 || !ms) return H2O4GPU_KMEANS_ESTATE;
  KM_HIP_TRY(hipSetDevice(h->dev));
  KM_HIP_TRY(hipEventRecord(h->t1, h->stream));
  KM_HIP_TRY(hipEventSynchronize(h->t1));
  KM_HIP_TRY(hipEventElapsedTime(ms, h->t0, h->t1));
  return 0;
}
KM_API int h2o4gpu_kmeans_profile(h2o4gpu_kmeans_handle *h, int on) {
  KM_CHECK_HANDLE(h);
  KM_HIP_TRY(hipSetDevice(h->dev));
  KM_TRY(h->prof_resolve());
  h->prof_on = on != 0;
  if (on) h->prof.clear();
  return 0;
}
KM_API int h2o4gpu_kmeans_kernel_time(h2o4gpu_kmeans_handle *h, const char *kernel,
                                      int *launches, double *ms) {
  KM_CHECK_HANDLE(h);
  if (!kernel) return H2O4GPU_KMEANS_EARG;
  KM_HIP_TRY(hipSetDevice(h->dev));
  KM_TRY(h->prof_resolve());
  auto it = h->prof.find(kernel);
  if (launches) *launches = it == h->prof.end() ? 0 : it->second.first;
  if (ms) *ms = it == h->prof.end() ? 0.0 : it->second.second;
  return 0;
}
KM_API const char *h2o4gpu_kmeans_assign_variant(h2o4gpu_kmeans_handle *h) {
  if (!h) return "";
  int v = h->elem_size == 4 ? pick_assign_variant<float>(h->opt_assign, h->n, h->d, h->k)
                            : pick_assign_variant<double>(h->opt_assign, h->n, h->d, h->k);
  if (v < 0) return "unsupported";
  if (h->elem_size == 4) {
    const int sp = assign_split_products<float>(h->opt_assign, h->opt_split, h->n, h->d, h->k, false);
    if (v == ASSIGN_ROWSTAT && sp == 9) return "mfma_rowstat_bf16x9";
    if (v == ASSIGN_ROWSTAT && sp == 6) return "mfma_rowstat_bf16x6";
    if (v == ASSIGN_TILED && sp == 9) return "mfma_tiled_bf16x9";
    if (v == ASSIGN_TILED && sp == 6) return "mfma_tiled_bf16x6";
  }
  return assign_variant_name(v);
}

KM_API int h2o4gpu_kmeans_bandwidth_probe(int gpu_id, int kind, size_t bytes, int reps, float *ms) {
  if (!ms || reps < 1 || bytes < 16 || kind < 0 || kind > 3) return H2O4GPU_KMEANS_EARG;
  const int nvis = visible_devices();
  if (nvis < 1) return H2O4GPU_KMEANS_EDEVICE;
  KM_HIP_TRY(hipSetDevice((gpu_id < 0 ? 0 : gpu_id) % nvis));
  const unsigned grid = 256 * 8, block = 256;
  void *a = nullptr, *b = nullptr;
  float *sink = nullptr;
  if (hipMalloc(&a, bytes) != hipSuccess || hipMalloc(&b, bytes) != hipSuccess ||
      hipMalloc(reinterpret_cast<void **>(&sink), (size_t)2 * grid * block * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    return H2O4GPU_KMEANS_EALLOC;
  }
  hipEvent_t e0, e1;
  int rc = 0;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
  if (rc == 0) {
    (void)hipMemset(a, 1, bytes);
    (void)hipMemset(b, 0, bytes);
    const size_t nvec = bytes / 16;
    auto once = [&]() {
      if (kind == H2O4GPU_KMEANS_PROBE_COPY)
        hipLaunchKernelGGL(copy_probe_kernel, dim3(grid), dim3(block), 0, 0, (const float4 *)a, (float4 *)b, nvec);
      else if (kind == H2O4GPU_KMEANS_PROBE_READ)
        hipLaunchKernelGGL(read_probe_kernel, dim3(grid * 2), dim3(block), 0, 0, (const floatx4 *)a, sink, nvec);
      else if (kind == H2O4GPU_KMEANS_PROBE_WRITE)
        hipLaunchKernelGGL(fill_probe_kernel, dim3(grid), dim3(block), 0, 0, (float4 *)b, nvec, 1.0f);
      else
        (void)hipMemcpyAsync(b, a, bytes, hipMemcpyDeviceToDevice, 0);
    };
    once();
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0, 0);
    for (int r = 0; r < reps; r++) once();
    (void)hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
    if (rc == 0 && hipGetLastError() != hipSuccess) rc = H2O4GPU_KMEANS_EDEVICE;
    float t = 0;
    if (rc == 0 && hipEventElapsedTime(&t, e0, e1) == hipSuccess) *ms = t / reps;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
  }
  (void)hipFree(a);
  (void)hipFree(b);
  (void)hipFree(sink);
  return rc;
}
KM_API int h2o4gpu_kmeans_copy_probe(int gpu_id, size_t bytes, int reps, float *ms) {
  return h2o4gpu_kmeans_bandwidth_probe(gpu_id, H2O4GPU_KMEANS_PROBE_COPY, bytes, reps, ms);
}

KM_API int h2o4gpu_kmeans_predict_device_noalloc(int elem_size, size_t rows, size_t cols, int k,
                                                 const void *d_X, const void *d_centroids,
                                                 int *d_labels, void *stream) {
  if (!d_X || !d_centroids || !d_labels || rows < 1 || cols < 1 || k < 1 ||
      rows > 2147483647ull || cols > 1000000ull)
    return H2O4GPU_KMEANS_EARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (elem_size == 4)
    return predict_device_noalloc<float>(rows, cols, k, static_cast<const float *>(d_X),
                                         static_cast<const float *>(d_centroids), d_labels, s);
  if (elem_size == 8)
    return predict_device_noalloc<double>(rows, cols, k, static_cast<const double *>(d_X),
                                          static_cast<const double *>(d_centroids), d_labels, s);
  return H2O4GPU_KMEANS_EARG;
}

KM_API int make_ptr_float_kmeans(int dopredict, int verbose, int seed, int gpu_id, int n_gpu,
                                 size_t mTrain, size_t n, int k, int max_iterations,
                                 int init_from_data, float threshold, const float *srcdata,
                                 const float *centroids, float **pred_centroids,
                                 int **pred_labels) {
  (void)n_gpu;
  if (dopredict == 0)
    return fit_entry<float>(verbose, seed, gpu_id, mTrain, n, k, max_iterations, init_from_data,
                            (double)threshold, srcdata, centroids, pred_centroids, pred_labels);
  return predict_entry<float>(verbose, gpu_id, mTrain, n, k, srcdata, centroids, pred_labels);
}
KM_API int make_ptr_double_kmeans(int dopredict, int verbose, int seed, int gpu_id, int n_gpu,
                                  size_t mTrain, size_t n, int k, int max_iterations,
                                  int init_from_data, double threshold, const double *srcdata,
                                  const double *centroids, double **pred_centroids,
                                  int **pred_labels) {
  (void)n_gpu;
  if (dopredict == 0)
    return fit_entry<double>(verbose, seed, gpu_id, mTrain, n, k, max_iterations, init_from_data,
                             threshold, srcdata, centroids, pred_centroids, pred_labels);
  return predict_entry<double>(verbose, gpu_id, mTrain, n, k, srcdata, centroids, pred_labels);
}
KM_API int kmeans_transform_float(int verbose, int gpu_id, int n_gpu, size_t m, size_t n, int k,
                                  const float *srcdata, const float *centroids, float **preds) {
  (void)n_gpu;
  return transform_entry<float>(verbose, gpu_id, m, n, k, srcdata, centroids, preds);
}
KM_API int kmeans_transform_double(int verbose, int gpu_id, int n_gpu, size_t m, size_t n, int k,
                                   const double *srcdata, const double *centroids,
                                   double **preds) {
  (void)n_gpu;
  return transform_entry<double>(verbose, gpu_id, m, n, k, srcdata, centroids, preds);
}

// ---------------------------------------------------------------------------
// C ABI, part 2: device information
// ---------------------------------------------------------------------------
KM_API int h2o4gpu_kmeans_device_count(void) { return visible_devices(); }

KM_API int get_gpu_info_c(int verbose, int return_memory, int return_name, int return_usage,
                          int return_free_memory, int return_capability,
                          int return_memory_by_pid, int return_usage_by_pid, int return_all,
                          unsigned int *n_gpus, int *gpu_percent_usage,
                          unsigned long long *gpu_total_memory,
                          unsigned long long *gpu_free_memory, char **gpu_name, int *majors,
                          int *minors, unsigned int *num_pids, unsigned int *pids,
                          unsigned long long *usedGpuMemorys, unsigned int *num_pids_usage,
                          unsigned int *pids_usage, unsigned long long *usedGpuUsage) {
  (void)pids;
  (void)usedGpuMemorys;
  (void)pids_usage;
  (void)usedGpuUsage;
  const int nvis = visible_devices();
  if (n_gpus) *n_gpus = (unsigned)nvis;
  if (nvis < 1) {
    log_msg(verbose, LOG_FATAL, "no HIP device visible");
    return 1;
  }
  for (int i = 0; i < nvis; i++) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, i) != hipSuccess) continue;
    if ((return_memory || return_all) && gpu_total_memory) gpu_total_memory[i] = prop.totalGlobalMem;
    if ((return_free_memory || return_all) && gpu_free_memory) {
      size_t fr = 0, tot = 0;
      if (hipSetDevice(i) == hipSuccess && hipMemGetInfo(&fr, &tot) == hipSuccess) gpu_free_memory[i] = fr;
    }
    if ((return_name || return_all) && gpu_name && gpu_name[i]) {
      strncpy(gpu_name[i], prop.name, 29);
      gpu_name[i][29] = '\0';
    }
    if ((return_capability || return_all) && majors && minors) {
      majors[i] = prop.major;
      minors[i] = prop.minor;
    }
    if ((return_usage || return_all) && gpu_percent_usage) gpu_percent_usage[i] = 0;
    if ((return_memory_by_pid || return_all) && num_pids) num_pids[i] = 0;
    if ((return_usage_by_pid || return_all) && num_pids_usage) num_pids_usage[i] = 0;
  }
  return 0;
}
KM_API int get_compute_capability(int d_idx, int *major, int *minor, int *ratioperf) {
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, d_idx);
  if (e != hipSuccess) return (int)e;
  if (major) *major = prop.major;
  if (minor) *minor = prop.minor;
  if (ratioperf) *ratioperf = 2;  // fp32 : fp64 matrix rate on MI355X
  return 0;
}
// Handles that still exist on the device do not survive a reset; the staging buffers of
// the upload path are released first and come back with the next transfer.
KM_API int cudaresetdevice(int wDev, int nDev) {
  (void)nDev;
  if (hipSetDevice(wDev) != hipSuccess) return 1;
  g_staging.forget(wDev);
  forget_dynamic_lds(wDev);
  forget_noalloc(wDev);
  return hipDeviceReset() == hipSuccess ? 0 : 1;
}
KM_API int cudaresetdevice_bare(void) {
  int dev = 0;
  if (hipGetDevice(&dev) == hipSuccess) {
    g_staging.forget(dev);
    forget_dynamic_lds(dev);
    forget_noalloc(dev);
  }
  return hipDeviceReset() == hipSuccess ? 0 : 1;
}

}  // extern "C"
