// TEST INFRASTRUCTURE ONLY -- CPU restatement of the k-means (Lloyd) path of
// h2oai/h2o4gpu, used as the parity checker and as the CPU baseline in the
// benchmark. Nothing in the shipped engine (h2o4gpu_amd/) links, loads or
// calls this file.
//
// Every function cites the reference text it restates (paths relative to the
// reference checkout). Arithmetic is done in T (float or double) with
// floating-point contraction switched off at build time, so a sum written
// "a*b + c" is a rounded multiply followed by a rounded add.
//
// Pinning status (what independent evidence fixes each function):
//   row_norms, distances, assign  : brute-force float64 closed form on tiny
//       inputs, D(x,x)=0 after fabs, tie rule, the reference's gtest
//       known-answer cases CountsPerCentroids / CentroidPerDataPoint.
//   update                        : the reference's gtest cases
//       CalculateCentroids, CalculateCentroids2GPU (shard additivity),
//       RevertCentroidZeroing, CentroidsScaling; mass invariants.
//   lloyd                         : k=1 closed form, k=n fixed point, an
//       independent Lloyd implementation (scikit-learn, explicit init) on
//       data without empty clusters, labels == argmin against final centroids.
//   random_rows                   : the two standard-library calls the
//       reference makes, compiled as written; distinctness, determinism.
//   transform                     : scipy cdist(sqeuclidean), transposed.
//   top2_exact, pair_dist_exact   : numpy float64 on the direct form with per-row
//       centroid pairs chosen asymmetrically (an a/b swap fails).
//   descending dot order          : bit-equal to a numpy evaluation that adds the
//       products of the column-reversed arrays in ascending order, norms untouched.
//   kmeanspp_*                    : not part of the reference (which seeds with
//       k-means||); pinned against the textbook D^2-sampling definition.
//   kmeans_parallel, weighted_kmeanspp, pick_point_idx_weighted, row thresholds:
//       the two generators by their published 10000th values, the row thresholds
//       bit for bit by rocThrust's host code, the host sampler's draws by numpy's
//       MT19937, the sampler on cases worked from the draws alone, every round's
//       candidates by float64 brute force over the thresholds, the weights by
//       brute-force nearest-candidate cells. Parity unpinned against a run of the
//       reference itself: its distances come out of cuBLAS / cblas and its sum of
//       costs out of thrust::reduce, both in an unspecified order (j ascending
//       and a fixed tree in double here).
//
// Build: make -C oracle   (g++ -O3 -fopenmp -ffp-contract=off)

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <numeric>
#include <random>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---------------------------------------------------------------------------
// self_dots: dots[i] = sum_j data[i,j]^2, accumulated in T, j ascending.
// Reference: src/gpu/kmeans/kmeans_labels.h:187-199.
// ---------------------------------------------------------------------------
template <typename T>
void row_norms(int64_t n, int d, const T *X, T *out, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < n; i++) {
    T acc = 0;
    const T *x = X + i * (int64_t)d;
    for (int j = 0; j < d; j++) {
      T v = x[j];
      acc += v * v;
    }
    out[i] = acc;
  }
}

// Centroids transposed to [d][kp] so the inner loop runs over centroids while
// each (row, centroid) dot product is still summed over j in ascending order.
template <typename T>
std::vector<T> transpose_centroids(int d, int k, const T *C) {
  std::vector<T> Ct((size_t)d * k);
  for (int c = 0; c < k; c++)
    for (int j = 0; j < d; j++) Ct[(size_t)j * k + c] = C[(size_t)c * d + j];
  return Ct;
}

// Summation order of the dot product: 0 = features ascending (default), 1 =
// descending. The reference leaves this order to cuBLAS; the switch exists so a
// test can measure how much a fixed-iteration trajectory depends on it.
static int g_dot_order = 0;

// dist(row, c) = | (xx + cc[c]) - 2 * dot(x, C[c]) |
// Reference: all_dots writes xx + cc (kmeans_labels.h:216-244); the GEMM then
// forms alpha*dot + beta*D with alpha=-2, beta=1 (kmeans_labels.cu:183-228);
// absolute_value is applied in place (kmeans_labels.cu:236-239).
// The summation order inside the reference's GEMM is a cuBLAS internal; this
// restatement uses j ascending.
template <typename T>
__attribute__((target_clones("avx2", "default"))) void
dist_row(int d, int k, const T *x, T xx, const T *Ct, const T *cc, T *acc) {
  for (int c = 0; c < k; c++) acc[c] = 0;
  const int order = g_dot_order;
  for (int jj = 0; jj < d; jj++) {
    const int j = order ? d - 1 - jj : jj;
    const T xj = x[j];
    const T *ct = Ct + (size_t)j * k;
    for (int c = 0; c < k; c++) acc[c] += xj * ct[c];
  }
  for (int c = 0; c < k; c++) {
    T t = xx + cc[c];
    T v = t - (T)2 * acc[c];
    acc[c] = std::fabs(v);
  }
}

// argmin with the reference's rule: running minimum starts at FLT_MAX (also for
// double), strict '<', first (lowest) index wins, index -1 if nothing is below
// the start value. Reference: kmeans_labels.h:360-377.
template <typename T>
inline int argmin_row(int k, const T *dist, T *best_out) {
  T best = (T)FLT_MAX;
  int idx = -1;
  for (int c = 0; c < k; c++) {
    if (dist[c] < best) {
      best = dist[c];
      idx = c;
    }
  }
  if (best_out) *best_out = best;
  return idx;
}

template <typename T>
void assign(int64_t n, int d, int k, const T *X, const T *C, int *labels,
            T *mindist, int threads) {
  std::vector<T> Ct = transpose_centroids(d, k, C);
  std::vector<T> cc(k);
  row_norms<T>(k, d, C, cc.data(), 1);
#pragma omp parallel num_threads(threads)
  {
    std::vector<T> acc(k);
#pragma omp for schedule(static)
    for (int64_t i = 0; i < n; i++) {
      const T *x = X + i * (int64_t)d;
      T xx = 0;
      for (int j = 0; j < d; j++) xx += x[j] * x[j];
      dist_row<T>(d, k, x, xx, Ct.data(), cc.data(), acc.data());
      T best;
      labels[i] = argmin_row<T>(k, acc.data(), &best);
      if (mindist) mindist[i] = best;
    }
  }
}

// Full distance matrix, centroid-major [k][n] (index c*n + i), squared
// distances, no sqrt. Reference: kmeans_transform, kmeans_h2o4gpu.cu:891-975;
// layout kmeans_labels.h:241.
template <typename T>
void distances(int64_t n, int d, int k, const T *X, const T *C, T *D,
               int threads) {
  std::vector<T> Ct = transpose_centroids(d, k, C);
  std::vector<T> cc(k);
  row_norms<T>(k, d, C, cc.data(), 1);
#pragma omp parallel num_threads(threads)
  {
    std::vector<T> acc(k);
#pragma omp for schedule(static)
    for (int64_t i = 0; i < n; i++) {
      const T *x = X + i * (int64_t)d;
      T xx = 0;
      for (int j = 0; j < d; j++) xx += x[j] * x[j];
      dist_row<T>(d, k, x, xx, Ct.data(), cc.data(), acc.data());
      for (int c = 0; c < k; c++) D[(size_t)c * n + i] = acc[c];
    }
  }
}

// Centroid update. Reference: find_centroids, kmeans_centroids.h:108-189:
//   keep a copy of the old centroids, zero sums and counts, add every row to
//   the sum of its label (calculate_centroids :40-75), restore the old
//   centroid where count < 1 (revert_zeroed_centroids :77-88), multiply by
//   1/T(max(count,1)) (scale_centroids :90-105; reciprocal then multiply).
// The reference adds with floating-point atomics in no fixed order, so the
// order of the additions is not part of its semantics. This restatement adds
// in double and rounds the total to T once: for float data whose column values
// span fewer than ~20 binades every partial sum is exact, so the result is the
// correctly rounded sum whatever the order or the number of threads. Rows with
// a label outside [0, k) are skipped.
template <typename T>
void update_sums(int64_t n, int d, int k, const T *X, const int *labels,
                 T *sums, int *counts, int threads) {
  if (threads < 1) threads = 1;
  std::vector<std::vector<double>> psum(threads);
  std::vector<std::vector<int>> pcnt(threads);
#pragma omp parallel num_threads(threads)
  {
    int t = 0, nt = 1;
#ifdef _OPENMP
    t = omp_get_thread_num();
    nt = omp_get_num_threads();
#endif
    psum[t].assign((size_t)k * d, 0.0);
    pcnt[t].assign(k, 0);
    int64_t lo = n * t / nt, hi = n * (t + 1) / nt;
    for (int64_t i = lo; i < hi; i++) {
      int l = labels[i];
      if (l < 0 || l >= k) continue;
      pcnt[t][l]++;
      double *s = psum[t].data() + (size_t)l * d;
      const T *x = X + i * (int64_t)d;
      for (int j = 0; j < d; j++) s[j] += (double)x[j];
    }
  }
  std::vector<double> tot((size_t)k * d, 0.0);
  std::fill(counts, counts + k, 0);
  for (int t = 0; t < threads; t++) {
    if (psum[t].empty()) continue;
    for (size_t e = 0; e < (size_t)k * d; e++) tot[e] += psum[t][e];
    for (int c = 0; c < k; c++) counts[c] += pcnt[t][c];
  }
  for (size_t e = 0; e < (size_t)k * d; e++) sums[e] = (T)tot[e];
}

template <typename T>
void finalize_centroids(int d, int k, const T *sums, const int *counts,
                        const T *old_c, T *new_c) {
  for (int c = 0; c < k; c++) {
    int count = counts[c];
    if (count < 1) {
      for (int j = 0; j < d; j++) new_c[(size_t)c * d + j] = old_c[(size_t)c * d + j];
      // scale_centroids multiplies by 1/T(1) == 1 here: value unchanged.
    } else {
      T scale = (T)1.0 / (T)count;
      for (int j = 0; j < d; j++) new_c[(size_t)c * d + j] = sums[(size_t)c * d + j] * scale;
    }
  }
}

template <typename T>
void update(int64_t n, int d, int k, const T *X, const int *labels, T *C,
            int *counts, int threads) {
  std::vector<T> old_c(C, C + (size_t)k * d);
  std::vector<T> sums((size_t)k * d);
  update_sums<T>(n, d, k, X, labels, sums.data(), counts, threads);
  finalize_centroids<T>(d, k, sums.data(), counts, old_c.data(), C);
}

// The Lloyd loop. Reference: kmeans::kmeans, kmeans_impl.h:109-232.
//   for i in [0, max_iterations): old = C; relabel; update; shift2 = sum
//   (old-new)^2 accumulated in T; done = shift2 < threshold (threshold is held
//   as double there); if done or last iteration: relabel once more with the
//   final centroids and stop. Returns i as the reference does (the index of
//   the iteration at which the loop was left; max_iterations-1 when it ran
//   to the end, max_iterations if max_iterations <= 0).
template <typename T>
int lloyd(int64_t n, int d, int k, const T *X, T *C, int *labels,
          int max_iterations, double threshold, int threads, double *shift_hist) {
  std::vector<T> old_c((size_t)k * d);
  std::vector<int> counts(k);
  int i = 0;
  for (; i < max_iterations; i++) {
    std::copy(C, C + (size_t)k * d, old_c.begin());
    assign<T>(n, d, k, X, C, labels, nullptr, threads);
    update<T>(n, d, k, X, labels, C, counts.data(), threads);
    T shift2 = 0;
    for (size_t e = 0; e < (size_t)k * d; e++) {
      T diff = old_c[e] - C[e];
      shift2 += diff * diff;
    }
    if (shift_hist) shift_hist[i] = (double)shift2;
    bool done = (double)shift2 < threshold;
    if (done || i == max_iterations - 1) {
      assign<T>(n, d, k, X, C, labels, nullptr, threads);
      break;
    }
  }
  return i;
}

// Exact squared distances ||x - c||^2 in double, direct form (no expansion),
// returning best index, best and second-best value per row: used by the tests
// to decide whether a label mismatch sits on a near-tie. Not part of the
// reference; mathematics only.
template <typename T>
void top2_exact(int64_t n, int d, int k, const T *X, const T *C, int *best_idx,
                double *d1, double *d2, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < n; i++) {
    const T *x = X + i * (int64_t)d;
    double b1 = std::numeric_limits<double>::infinity(), b2 = b1;
    int bi = -1;
    for (int c = 0; c < k; c++) {
      const T *cp = C + (size_t)c * d;
      double s = 0;
      for (int j = 0; j < d; j++) {
        double df = (double)x[j] - (double)cp[j];
        s += df * df;
      }
      if (s < b1) {
        b2 = b1;
        b1 = s;
        bi = c;
      } else if (s < b2) {
        b2 = s;
      }
    }
    best_idx[i] = bi;
    d1[i] = b1;
    d2[i] = b2;
  }
}

// Exact squared distance of every row to two given centroids per row
// (labels a[i], b[i]) in double: lets a test price a mismatch without a full
// n*k pass.
template <typename T>
void pair_dist_exact(int64_t n, int d, const T *X, const T *C, const int *a,
                     const int *b, double *da, double *db, int threads) {
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int64_t i = 0; i < n; i++) {
    const T *x = X + i * (int64_t)d;
    const T *ca = C + (size_t)a[i] * d;
    const T *cb = C + (size_t)b[i] * d;
    double sa = 0, sb = 0;
    for (int j = 0; j < d; j++) {
      double u = (double)x[j] - (double)ca[j];
      double v = (double)x[j] - (double)cb[j];
      sa += u * u;
      sb += v * v;
    }
    da[i] = sa;
    db[i] = sb;
  }
}

// k-means++ (D^2 sampling), the textbook algorithm with the draw rule spelled out so
// that a GPU implementation can follow it to the bit:
//   first centre: std::mt19937 gen(seed); uniform_int_distribution<>(0, n-1)(gen)
//     (how the reference draws the first centre of its k-means||,
//      kmeans_h2o4gpu.cu:343-347);
//   mind[i] = min over chosen centres of |(xx_i + cc) - 2 x_i.c|  (the distance
//     form of kmeans_labels.cu:183-244; running minimum as min_calc_functor,
//     kmeans_h2o4gpu.cu:281-304);
//   next centre: u = uniform_real_distribution<double>(0,1)(gen); target = u*total,
//     total = ordered sum of block sums; block sums cover 1024 rows each and are
//     formed in double by 256 partial sums (rows t, t+256, t+512, t+768) combined by
//     a halving tree; the block is the first whose running total exceeds the target,
//     the row the first inside it whose running total exceeds the target (last
//     positive row if rounding runs past the end).
// Not part of the reference (it seeds with k-means||); parity unpinned against it.
template <typename T>
void kmeanspp(int64_t n, int d, int k, const T *X, int seed, int *rows_out, T *mind_out) {
  const int BLOCK = 1024, W = 256;
  std::vector<T> xx((size_t)n), mind((size_t)n);
  row_norms<T>(n, d, X, xx.data(), 1);
  std::mt19937 gen((unsigned)seed);
  std::uniform_int_distribution<> first(0, (int)(n - 1));
  std::uniform_real_distribution<double> uni(0.0, 1.0);
  const int64_t nb = (n + BLOCK - 1) / BLOCK;
  std::vector<double> bs((size_t)nb);
  rows_out[0] = first(gen);
  for (int c = 1; c <= k; c++) {
    const T *cp = X + (int64_t)rows_out[c - 1] * d;
    const T cc = xx[rows_out[c - 1]];
    for (int64_t i = 0; i < n; i++) {
      const T *x = X + i * (int64_t)d;
      T dot = 0;
      for (int j = 0; j < d; j++) dot += x[j] * cp[j];
      T t = xx[i] + cc;
      T dist = std::fabs(t - (T)2 * dot);
      mind[i] = (c == 1) ? dist : std::min(dist, mind[i]);
    }
    if (c == k) break;
    for (int64_t b = 0; b < nb; b++) {
      double part[W];
      for (int t = 0; t < W; t++) {
        double acc = 0;
        for (int q = 0; q < BLOCK / W; q++) {
          int64_t row = b * BLOCK + t + q * W;
          if (row < n) acc += (double)mind[row];
        }
        part[t] = acc;
      }
      for (int off = W / 2; off > 0; off >>= 1)
        for (int t = 0; t < off; t++) part[t] += part[t + off];
      bs[b] = part[0];
    }
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
      const int64_t lo = b * BLOCK;
      const int cnt = (int)std::min<int64_t>(BLOCK, n - lo);
      int i = 0, last_pos = 0;
      for (; i < cnt; i++) {
        if ((double)mind[lo + i] > 0) last_pos = i;
        if (run + (double)mind[lo + i] > target) break;
        run += (double)mind[lo + i];
      }
      if (i >= cnt) i = last_pos;
      pick = lo + i;
    }
    rows_out[c] = (int)pick;
  }
  if (mind_out) std::copy(mind.begin(), mind.end(), mind_out);
}


// ---------------------------------------------------------------------------
// k-means|| seeding, the reference's init_from_data == 1
// (kmeans_parallel, kmeans_h2o4gpu.cu:331-563) followed by its host-side weighted
// k-means++ over the candidates (:154-279).
// ---------------------------------------------------------------------------

// thrust::default_random_engine is minstd_rand: x <- 48271 x mod (2^31 - 1), state seeded
// with seed mod m, or 1 when that is 0. The value the engine returns is the new state.
static const uint32_t MINSTD_M = 2147483647u;
static inline uint32_t minstd_seed(int seed) {
  const uint32_t s = (uint32_t)seed % MINSTD_M;  // int -> result_type (uint32) first
  return s == 0 ? 1u : s;
}
static inline uint32_t minstd_next(uint32_t x) {
  return (uint32_t)(((uint64_t)x * 48271u) % MINSTD_M);
}
// thrust::uniform_real_distribution<> has RealType float and maps one engine value x to
//   float(x - min) / (1.0f + float(max - min)) * (b - a) + a,   min = 1, max = m - 1,
// all in float (thrust/random/detail/uniform_real_distribution.inl). With a = 0, b = 1.
static inline float thrust_uniform01(uint32_t x) {
  float result = static_cast<float>(x - 1u);
  result /= (1.0f + static_cast<float>((MINSTD_M - 1u) - 1u));
  return (result * (1.0f - 0.0f)) + 0.0f;
}
// The threshold of a row: rng(seed); rng.discard(row); dist(rng)  (:444-449). It does not
// depend on the round.
static float row_threshold(int seed, int64_t row) {
  uint32_t x = minstd_seed(seed);
  for (int64_t i = 0; i <= row; i++) x = minstd_next(x);
  return thrust_uniform01(x);
}

// Sum of n values in double: blocks of 1024 rows, each formed from 256 partial sums (rows
// t, t+256, t+512, t+768) combined by a halving tree, the block sums then added in block
// order. The reference calls thrust::reduce in T, whose order is unspecified; this is the
// order the GPU engine uses, so that both sides agree to the bit.
template <typename T>
double blocked_sum(int64_t n, const T *v) {
  const int BLOCK = 1024, W = 256;
  double total = 0;
  for (int64_t b0 = 0; b0 < n; b0 += BLOCK) {
    double part[W];
    for (int t = 0; t < W; t++) {
      double acc = 0;
      for (int q = 0; q < BLOCK / W; q++) {
        const int64_t row = b0 + t + q * W;
        if (row < n) acc += (double)v[row];
      }
      part[t] = acc;
    }
    for (int off = W / 2; off > 0; off >>= 1)
      for (int t = 0; t < off; t++) part[t] += part[t + off];
    total += part[0];
  }
  return total;
}

// pick_point_idx_weighted (:154-199). weighted_sum is a sequential sum in T of weights[i]
// (data == null) or data[i]*weights[i]. A fresh mt19937(seed) is made on every call; entry
// i is taken as soon as its share of the sum exceeds the i-th draw of
// std::uniform_real_distribution<double>(0,1) cast to T. When no entry is taken the result
// is the last entry whose share reached the running maximum (start 0, updated on >=).
template <typename T>
int pick_point_idx_weighted(int seed, const T *data, const T *weights, int m) {
  T weighted_sum = 0;
  for (int i = 0; i < m; i++) weighted_sum += data ? data[i] * weights[i] : weights[i];
  T best_prob = 0;
  int best_idx = 0;
  std::mt19937 mt(seed);
  std::uniform_real_distribution<> dist(0.0, 1.0);
  for (int i = 0; i < m; i++) {
    const T threshold = (T)dist(mt);
    T val = weights[i];
    if (data) val *= data[i];
    const T share = val / weighted_sum;
    if (share > threshold) return i;
    if (share >= best_prob) {
      best_prob = share;
      best_idx = i;
    }
  }
  return best_idx;
}

// compute_distances for one centroid (src/common/utils.cpp:7-57): xx + cc formed first,
// then the GEMM adds -2 * dot to it; no absolute value. The order inside the reference's
// cblas GEMM is not specified; j ascending here.
template <typename T>
void host_dists_to_one(int m, int d, const T *data, const T *centre, T *out) {
  T cc = 0;
  for (int j = 0; j < d; j++) cc += centre[j] * centre[j];
  for (int i = 0; i < m; i++) {
    const T *x = data + (size_t)i * d;
    T xx = 0, dot = 0;
    for (int j = 0; j < d; j++) xx += x[j] * x[j];
    for (int j = 0; j < d; j++) dot += x[j] * centre[j];
    const T t = xx + cc;
    out[i] = (T)-2 * dot + t;
  }
}

// kmeans_plus_plus over the candidates (:201-279): first entry drawn from the weights
// alone; every chosen entry gets weight 0; the running minimum of a chosen entry is set
// to 0 before the distances to it are folded in. chosen receives k candidate indices.
template <typename T>
void weighted_kmeanspp(int seed, int m, int d, int k, const T *data, T *weights, int *chosen) {
  std::vector<T> best((size_t)m), curr((size_t)m);
  int idx = pick_point_idx_weighted<T>(seed, nullptr, weights, m);
  chosen[0] = idx;
  weights[idx] = 0;
  host_dists_to_one<T>(m, d, data, data + (size_t)idx * d, best.data());
  for (int it = 0; it < k - 1; it++) {
    idx = pick_point_idx_weighted<T>(seed, best.data(), weights, m);
    chosen[it + 1] = idx;
    weights[idx] = 0;
    best[idx] = 0;
    host_dists_to_one<T>(m, d, data, data + (size_t)idx * d, curr.data());
    for (int i = 0; i < m; i++) best[i] = std::min(curr[i], best[i]);
  }
}

// kmeans_parallel (:331-563), one device.
//   first centre: mt19937(seed), uniform_int_distribution<>(0, rows-1)   (:343-347)
//   min_costs start at numeric_limits<T>::max()                          (:372-377)
//   rounds: min(8, (int)(2 + log(k)))                                    (:382)
//   a round measures every row against the candidates the PREVIOUS round added
//     (|xx + cc - 2 x.c|, running minimum: min_calc_functor :281-304), sums the minima,
//     and, unless the sum is 0, takes every row with
//     T(2.0 * k * min_cost / total) > T(threshold(row)) as a new candidate, in row order
//     (:436-476). A round that adds nothing leaves the previous candidate list in place.
//   more than k candidates: weights = rows per nearest candidate (count_functor,
//     kmeans_h2o4gpu.h:44-72: first index wins, start value the distance to candidate 0),
//     then weighted_kmeanspp; otherwise the candidates followed by zero rows (:536-540).
// cand_rows receives the data row of every candidate in the order found (capacity cap),
// round_count[r] the number added by round r (r < 8; the first centre is not counted),
// phi[r] the sum of minima of round r, weights the per-candidate counts (when computed),
// chosen the k candidate indices of the final centres (-1: zero row). Returns the number
// of candidates, or -1 when cap is too small.
template <typename T>
int kmeans_parallel(int64_t n, int d, int k, const T *X, int seed, int cap, int *cand_rows,
                    int *round_count, double *phi, T *weights, int *chosen, T *C_out,
                    int threads) {
  std::mt19937 gen(seed);
  std::uniform_int_distribution<> dis(0, (int)(n - 1));
  std::vector<int> all;
  all.push_back(dis(gen));
  std::vector<int> recent = all;
  std::vector<T> min_costs((size_t)n, std::numeric_limits<T>::max());
  std::vector<T> xx((size_t)n);
  row_norms<T>(n, d, X, xx.data(), threads);
  std::vector<float> thr((size_t)n);
  {
    uint32_t x = minstd_seed(seed);
    for (int64_t i = 0; i < n; i++) {
      x = minstd_next(x);
      thr[(size_t)i] = thrust_uniform01(x);
    }
  }
  auto gather = [&](const std::vector<int> &rows) {
    std::vector<T> c(rows.size() * (size_t)d);
    for (size_t r = 0; r < rows.size(); r++)
      std::copy(X + (int64_t)rows[r] * d, X + ((int64_t)rows[r] + 1) * d, c.begin() + r * d);
    return c;
  };
  const int max_iter = std::min(8, (int)(2 + std::log((double)k)));
  for (int r = 0; r < 8; r++) {
    round_count[r] = 0;
    phi[r] = 0;
  }
  for (int counter = 0; counter < max_iter; counter++) {
    const int m = (int)recent.size();
    std::vector<T> Cc = gather(recent);
    std::vector<T> Ct = transpose_centroids(d, m, Cc.data());
    std::vector<T> cc(m);
    row_norms<T>(m, d, Cc.data(), cc.data(), 1);
#pragma omp parallel num_threads(threads)
    {
      std::vector<T> acc(m);
#pragma omp for schedule(static)
      for (int64_t i = 0; i < n; i++) {
        dist_row<T>(d, m, X + i * (int64_t)d, xx[(size_t)i], Ct.data(), cc.data(), acc.data());
        T best = std::numeric_limits<T>::max();
        for (int c = 0; c < m; c++) best = std::min(best, acc[c]);
        min_costs[(size_t)i] = std::min(min_costs[(size_t)i], best);
      }
    }
    const T total = (T)blocked_sum<T>(n, min_costs.data());
    phi[counter] = (double)total;
    if (total == (T)0) continue;
    std::vector<int> fresh;
    for (int64_t i = 0; i < n; i++) {
      const T threshold = (T)thr[(size_t)i];
      const T prob = (T)((2.0 * k * min_costs[(size_t)i]) / total);
      if (prob > threshold) fresh.push_back((int)i);
    }
    round_count[counter] = (int)fresh.size();
    if (!fresh.empty()) {
      recent = fresh;
      all.insert(all.end(), fresh.begin(), fresh.end());
    }
  }
  const int M = (int)all.size();
  if (M > cap) return -1;
  std::copy(all.begin(), all.end(), cand_rows);
  std::fill(C_out, C_out + (size_t)k * d, (T)0);
  if (M <= k) {
    for (int c = 0; c < k; c++) chosen[c] = c < M ? c : -1;
    for (int c = 0; c < M; c++)
      std::copy(X + (int64_t)all[c] * d, X + ((int64_t)all[c] + 1) * d, C_out + (size_t)c * d);
    return M;
  }
  std::vector<T> Call = gather(all);
  {
    std::vector<T> Ct = transpose_centroids(d, M, Call.data());
    std::vector<T> cc(M);
    row_norms<T>(M, d, Call.data(), cc.data(), 1);
    std::vector<int64_t> counts((size_t)M, 0);
#pragma omp parallel num_threads(threads)
    {
      std::vector<T> acc(M);
      std::vector<int64_t> local((size_t)M, 0);
#pragma omp for schedule(static)
      for (int64_t i = 0; i < n; i++) {
        dist_row<T>(d, M, X + i * (int64_t)d, xx[(size_t)i], Ct.data(), cc.data(), acc.data());
        int closest = 0;
        T best = acc[0];
        for (int c = 1; c < M; c++) {
          if (acc[c] < best) {
            best = acc[c];
            closest = c;
          }
        }
        local[(size_t)closest]++;
      }
#pragma omp critical
      for (int c = 0; c < M; c++) counts[(size_t)c] += local[(size_t)c];
    }
    for (int c = 0; c < M; c++) weights[c] = (T)counts[(size_t)c];
  }
  std::vector<T> w(weights, weights + M);
  weighted_kmeanspp<T>(seed, M, d, k, Call.data(), w.data(), chosen);
  for (int c = 0; c < k; c++)
    std::copy(Call.begin() + (size_t)chosen[c] * d, Call.begin() + ((size_t)chosen[c] + 1) * d,
              C_out + (size_t)c * d);
  return M;
}

}  // namespace

extern "C" {

#define ORACLE_EXPORT __attribute__((visibility("default")))

ORACLE_EXPORT void oracle_set_dot_order(int order) { g_dot_order = order ? 1 : 0; }

ORACLE_EXPORT int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

#define DEFINE_FOR(T, SUF)                                                        \
  ORACLE_EXPORT void oracle_row_norms_##SUF(int64_t n, int d, const T *X, T *out, \
                                            int threads) {                        \
    row_norms<T>(n, d, X, out, threads);                                          \
  }                                                                               \
  ORACLE_EXPORT void oracle_assign_##SUF(int64_t n, int d, int k, const T *X,     \
                                         const T *C, int *labels, T *mindist,     \
                                         int threads) {                           \
    assign<T>(n, d, k, X, C, labels, mindist, threads);                           \
  }                                                                               \
  ORACLE_EXPORT void oracle_distances_##SUF(int64_t n, int d, int k, const T *X,  \
                                            const T *C, T *D, int threads) {      \
    distances<T>(n, d, k, X, C, D, threads);                                      \
  }                                                                               \
  ORACLE_EXPORT void oracle_update_sums_##SUF(int64_t n, int d, int k,            \
                                              const T *X, const int *labels,      \
                                              T *sums, int *counts,               \
                                              int threads) {                      \
    update_sums<T>(n, d, k, X, labels, sums, counts, threads);                    \
  }                                                                               \
  ORACLE_EXPORT void oracle_finalize_##SUF(int d, int k, const T *sums,           \
                                           const int *counts, const T *old_c,     \
                                           T *new_c) {                            \
    finalize_centroids<T>(d, k, sums, counts, old_c, new_c);                      \
  }                                                                               \
  ORACLE_EXPORT void oracle_update_##SUF(int64_t n, int d, int k, const T *X,     \
                                         const int *labels, T *C, int *counts,    \
                                         int threads) {                           \
    update<T>(n, d, k, X, labels, C, counts, threads);                            \
  }                                                                               \
  ORACLE_EXPORT int oracle_lloyd_##SUF(int64_t n, int d, int k, const T *X, T *C, \
                                       int *labels, int max_iterations,           \
                                       double threshold, int threads,             \
                                       double *shift_hist) {                      \
    return lloyd<T>(n, d, k, X, C, labels, max_iterations, threshold, threads,    \
                    shift_hist);                                                  \
  }                                                                               \
  ORACLE_EXPORT void oracle_top2_exact_##SUF(int64_t n, int d, int k, const T *X, \
                                             const T *C, int *best, double *d1,   \
                                             double *d2, int threads) {           \
    top2_exact<T>(n, d, k, X, C, best, d1, d2, threads);                          \
  }                                                                               \
  ORACLE_EXPORT void oracle_pair_dist_exact_##SUF(                                \
      int64_t n, int d, const T *X, const T *C, const int *a, const int *b,       \
      double *da, double *db, int threads) {                                      \
    pair_dist_exact<T>(n, d, X, C, a, b, da, db, threads);                        \
  }

DEFINE_FOR(float, f32)
DEFINE_FOR(double, f64)

ORACLE_EXPORT void oracle_kmeanspp_f32(int64_t n, int d, int k, const float *X, int seed,
                                       int *rows_out, float *mind_out) {
  kmeanspp<float>(n, d, k, X, seed, rows_out, mind_out);
}
ORACLE_EXPORT void oracle_kmeanspp_f64(int64_t n, int d, int k, const double *X, int seed,
                                       int *rows_out, double *mind_out) {
  kmeanspp<double>(n, d, k, X, seed, rows_out, mind_out);
}

ORACLE_EXPORT float oracle_kmeans_parallel_row_threshold(int seed, int64_t row) {
  return row_threshold(seed, row);
}
ORACLE_EXPORT unsigned oracle_minstd_nth(int seed, int64_t nth) {  // value of the nth call, nth >= 1
  uint32_t x = minstd_seed(seed);
  for (int64_t i = 0; i < nth; i++) x = minstd_next(x);
  return x;
}
#define DEFINE_SEED_FOR(T, SUF)                                                              \
  ORACLE_EXPORT int oracle_pick_point_idx_weighted_##SUF(int seed, int m, const T *data,    \
                                                         const T *weights) {                \
    return pick_point_idx_weighted<T>(seed, data, weights, m);                              \
  }                                                                                         \
  ORACLE_EXPORT void oracle_weighted_kmeanspp_##SUF(int seed, int m, int d, int k,           \
                                                    const T *data, const T *weights,        \
                                                    int *chosen) {                          \
    std::vector<T> w(weights, weights + m);                                                 \
    weighted_kmeanspp<T>(seed, m, d, k, data, w.data(), chosen);                            \
  }                                                                                         \
  ORACLE_EXPORT int oracle_kmeans_parallel_##SUF(int64_t n, int d, int k, const T *X,       \
                                                 int seed, int cap, int *cand_rows,         \
                                                 int *round_count, double *phi, T *weights, \
                                                 int *chosen, T *C_out, int threads) {      \
    return kmeans_parallel<T>(n, d, k, X, seed, cap, cand_rows, round_count, phi, weights,  \
                              chosen, C_out, threads);                                      \
  }
DEFINE_SEED_FOR(float, f32)
DEFINE_SEED_FOR(double, f64)

// Seeded random-row initialisation: a permutation of 0..n-1 by
// std::shuffle(v.begin(), v.end(), std::default_random_engine(seed)); the
// initial centroids are rows v[0..k-1]. These are the two standard-library
// calls the reference makes (kmeans_h2o4gpu.cu:662-669, rows taken at :79-84
// and :692-693); the permutation depends on the C++ standard library in use.
ORACLE_EXPORT void oracle_random_rows(int seed, int64_t n, int k, int *idx_out) {
  std::vector<int> v((size_t)n);
  std::iota(v.begin(), v.end(), 0);
  std::shuffle(v.begin(), v.end(), std::default_random_engine(seed));
  for (int c = 0; c < k; c++) idx_out[c] = v[c];
}

// First k-means++ centre: std::mt19937 gen(seed); uniform_int_distribution<>
// dis(0, rows-1); dis(gen). Reference: kmeans_parallel picks its first centre
// this way (kmeans_h2o4gpu.cu:343-347).
ORACLE_EXPORT int oracle_kmeanspp_first(int seed, int64_t n) {
  std::mt19937 gen(seed);
  std::uniform_int_distribution<> dis(0, (int)(n - 1));
  return dis(gen);
}

}  // extern "C"
