// k-means++ seeding kernels (D^2 sampling).
//
// The reference seeds init_from_data == 1 with k-means|| followed by a host
// k-means++ over the candidates (src/gpu/kmeans/kmeans_h2o4gpu.cu:231-563),
// whose building blocks are "distance of every row to the newest centres",
// "running minimum per row" (min_calc_functor, :281-304) and "sum of the
// minima" (thrust::reduce, :423-424). The same three blocks are provided here
// for plain k-means++: one kernel updates the running minimum against the
// newest centre and emits fixed-order block sums; the host draws the next
// centre from the block sums and one block of minima.
#include <algorithm>
#include <limits>

#include "kmeans_common.h"

namespace kmhip {

static constexpr int WG = 256;

template <typename T, int VEC>
struct SeedVec {  // 16 bytes of a row, aligned to the elements only
  typedef T type __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));
};
template <typename T>
struct SeedVec<T, 1> {
  typedef T type;
};

// Squared distances from the newest centre (row `new_row` of X) to the t centres chosen
// before it (rows[0..t-1]), direct form in double, one wavefront per earlier centre;
// also records rows[t] = new_row. The value is shaved by one part in 1e6 so that the
// pruning test below errs towards computing a distance.
template <typename T>
__global__ __launch_bounds__(WG) void centre_dists_kernel(const T *__restrict__ X,
                                                         int *__restrict__ rows, int t,
                                                         int new_row, T *__restrict__ dcc,
                                                         int d) {
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * (WG / 64) + (threadIdx.x >> 6);
  if (blockIdx.x == 0 && threadIdx.x == 0) rows[t] = new_row;
  if (j >= t) return;
  const T *a = X + (int64_t)rows[j] * d;
  const T *b = X + (int64_t)new_row * d;
  double acc = 0;
  for (int q = lane; q < d; q += 64) {
    const double diff = (double)a[q] - (double)b[q];
    acc += diff * diff;
  }
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) dcc[j] = (T)(acc * (1.0 - 1e-6));
}

// One k-means++ round against the centre c = row `centre_row` of X, the t-th chosen:
//   mind[i] = min(mind[i], |(xx_i + cc) - 2 x_i.c|),  nearest[i] = t where it improved
// (init != 0: overwrite), then bsums[block] = sum of the block's KPP_BLOCK minima in
// double with a fixed tree. One workgroup per KPP_BLOCK rows.
//
// Most rows cannot improve and are never loaded: with j = nearest[i], the triangle
// inequality gives |x - c| >= |c - c_j| - |x - c_j|, so dcc[j] >= 4 mind[i] implies
// |x - c|^2 >= mind[i]. Phase 1 reads 8 bytes per row and lists the rows that fail this
// test; phase 2 computes distances for the listed rows only, lpr lanes per row with
// coalesced (16-byte where possible) loads, U rows per lane group in flight. A row is
// skipped only when the bound holds with a 1e-4 margin; where the stored minimum is
// itself within rounding of zero the kept value can exceed what a recomputation would
// give by less than that rounding error.
// SUB: rows per workgroup. KPP_BLOCK: the workgroup also writes its block sum. Smaller
// (long rows, where 1024 of them per workgroup leave a 500,000-row data set with two
// workgroups per CU): the block sums come from block_sums_kernel afterwards.
template <typename T>
__device__ __forceinline__ void block_sum(const T *__restrict__ mind, double *__restrict__ bsums,
                                          int64_t block, int64_t n, double *red) {
  const int tid = threadIdx.x;
  const int64_t b0 = block * KPP_BLOCK;
  double acc = 0;
#pragma unroll
  for (int q = 0; q < KPP_BLOCK / WG; q++) {
    const int64_t row = b0 + tid + q * WG;
    if (row < n) acc += (double)mind[row];
  }
  red[tid] = acc;
  __syncthreads();
  for (int off = WG / 2; off > 0; off >>= 1) {
    if (tid < off) red[tid] += red[tid + off];
    __syncthreads();
  }
  if (tid == 0) bsums[block] = red[0];
}
template <typename T>
__global__ __launch_bounds__(WG) void block_sums_kernel(const T *__restrict__ mind,
                                                       double *__restrict__ bsums, int64_t n) {
  __shared__ double red[WG];
  block_sum<T>(mind, bsums, blockIdx.x, n, red);
}

template <typename T, int VEC, int SUB>
__global__ __launch_bounds__(WG) void min_dist_update_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm, int64_t centre_row,
    T *__restrict__ mind, int *__restrict__ nearest, const T *__restrict__ dcc, int t,
    double *__restrict__ bsums, int64_t n, int d, int init, int lpr) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *cs = reinterpret_cast<T *>(smem_raw);  // [d]
  __shared__ double red[WG];
  __shared__ int list[SUB];
  __shared__ int cnt;
  typedef typename SeedVec<T, VEC>::type vec_t;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  for (int j = tid; j < d; j += WG) cs[j] = X[centre_row * (int64_t)d + j];
  if (tid == 0) cnt = 0;
  const T cc = xnorm[centre_row];
  __syncthreads();
  const int64_t b0 = (int64_t)blockIdx.x * SUB;
#pragma unroll
  for (int q = 0; q < SUB / WG; q++) {
    const int r = tid + q * WG;
    const int64_t row = b0 + r;
    if (row < n) {
      bool pass = init != 0;
      if (!pass) pass = !(dcc[nearest[row]] >= (T)4.0004 * mind[row]);
      if (pass) list[atomicAdd(&cnt, 1)] = r;  // order is irrelevant: rows are independent
    }
  }
  __syncthreads();
  const int m = cnt;
  const int rps = 64 / lpr;           // rows per wavefront step
  const int groups = (WG / 64) * rps;  // lane groups in the workgroup
  const int gid = wave * rps + lane / lpr, col = lane % lpr;
  constexpr int U = 4;
  for (int base = 0; base < m; base += groups * U) {
    int r[U];
    const T *x[U];
    T dot[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int e = base + u * groups + gid;
      r[u] = e < m ? list[e] : -1;
      x[u] = X + (b0 + (r[u] < 0 ? list[0] : r[u])) * (int64_t)d;
      dot[u] = 0;
    }
    for (int j = col * VEC; j < d; j += lpr * VEC) {
      // a vector that would reach past the end of the row (d not a multiple of VEC) is
      // fetched from the row's last VEC values; its elements below `first` belong to
      // the neighbouring lane
      const int jc = min(j, d - VEC), first = j - jc;
      vec_t v[U];
#pragma unroll
      for (int u = 0; u < U; u++) v[u] = *reinterpret_cast<const vec_t *>(x[u] + jc);
#pragma unroll
      for (int u = 0; u < U; u++) {
        if constexpr (VEC == 1) {
          dot[u] += v[u] * cs[j];
        } else {
#pragma unroll
          for (int e = 0; e < VEC; e++) dot[u] += e >= first ? v[u][e] * cs[jc + e] : (T)0;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      for (int off = 1; off < lpr; off <<= 1) dot[u] += __shfl_xor(dot[u], off, 64);
      if (col == 0 && r[u] >= 0) {
        const int64_t row = b0 + r[u];
        const T s = xnorm[row] + cc;
        const T dist = fabs(s - (T)2 * dot[u]);
        if (init || dist < mind[row]) {
          mind[row] = dist;
          nearest[row] = t;
        }
      }
    }
  }
  if (SUB == KPP_BLOCK) {
    __syncthreads();
    block_sum<T>(mind, bsums, blockIdx.x, n, red);
  }
}

template <typename T>
int launch_min_dist_update(hipStream_t s, const T *X, const T *xnorm, int64_t centre_row,
                           T *mind, int *nearest, int *rows, T *dcc, int t, double *bsums,
                           int64_t n, int d) {
  if (n <= 0) return 0;
  const int init = t == 0;
  hipLaunchKernelGGL((centre_dists_kernel<T>), dim3((unsigned)(t / (WG / 64) + 1)), dim3(WG), 0, s,
                     X, rows, t, (int)centre_row, dcc, d);
  constexpr int VW = 16 / sizeof(T);
  const bool vec = d >= VW;  // 16-byte loads need element alignment only
  const int per_row = vec ? (d + VW - 1) / VW : d;  // loads that cover a row
  int lpr = 1;
  while (lpr < per_row && lpr < 64) lpr <<= 1;
  const unsigned blocks = (unsigned)((n + KPP_BLOCK - 1) / KPP_BLOCK);
  // long rows: 256 rows per workgroup, block sums afterwards (500k x 784: 489 workgroups
  // of 1024 rows are fewer than two per CU)
  const bool fine = (size_t)d * sizeof(T) >= 1024 && n >= 4 * KPP_BLOCK;
#define KM_MDU(VECW, SUB)                                                                      \
  hipLaunchKernelGGL((min_dist_update_kernel<T, VECW, SUB>),                                   \
                     dim3((unsigned)((n + SUB - 1) / SUB)), dim3(WG), (size_t)d * sizeof(T), s, \
                     X, xnorm, centre_row, mind, nearest, dcc, t, bsums, n, d, init, lpr)
  if (vec && fine) KM_MDU(VW, 256);
  else if (vec) KM_MDU(VW, KPP_BLOCK);
  else if (fine) KM_MDU(1, 256);
  else KM_MDU(1, KPP_BLOCK);
#undef KM_MDU
  if (fine)
    hipLaunchKernelGGL((block_sums_kernel<T>), dim3(blocks), dim3(WG), 0, s, mind, bsums, n);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// ---------------------------------------------------------------------------
// k-means|| (the reference's init_from_data == 1, kmeans_h2o4gpu.cu:331-563).
// A round measures every row against the candidates of the previous round with the
// assign kernels (their minimum distance is min_calc_functor's inner minimum, :281-304);
// the kernels below fold that into the running cost, sum it, and apply the reference's
// acceptance test to every row.
// ---------------------------------------------------------------------------

// Model of m candidate rows for the assign kernels: Cc [mpad][d] = rows idx[0..m-1] of X
// followed by zero rows, ccn [mpad] = their squared norms (taken from xnorm: the same
// value row_norms would compute) followed by +inf.
template <typename T>
__global__ __launch_bounds__(WG) void gather_model_kernel(const T *__restrict__ X,
                                                         const T *__restrict__ xnorm,
                                                         const int *__restrict__ idx, int m, int mpad,
                                                         T *__restrict__ Cc, T *__restrict__ ccn,
                                                         int d) {
  const int64_t total = (int64_t)mpad * d;
  const int64_t stride = (int64_t)gridDim.x * WG;
  const int64_t t0 = (int64_t)blockIdx.x * WG + threadIdx.x;
  for (int64_t e = t0; e < total; e += stride) {
    const int c = (int)(e / d), j = (int)(e - (int64_t)c * d);
    Cc[e] = c < m ? X[(int64_t)idx[c] * d + j] : (T)0;
  }
  for (int64_t c = t0; c < mpad; c += stride)
    ccn[c] = c < m ? xnorm[idx[c]] : (T)__builtin_huge_val();
}
template <typename T>
int launch_gather_model(hipStream_t s, const T *X, const T *xnorm, const int *idx, int m, int mpad,
                        T *Cc, T *ccn, int d) {
  const int64_t total = (int64_t)mpad * d;
  const unsigned blocks = (unsigned)std::min<int64_t>((total + WG - 1) / WG, 4096);
  hipLaunchKernelGGL((gather_model_kernel<T>), dim3(blocks), dim3(WG), 0, s, X, xnorm, idx, m, mpad,
                     Cc, ccn, d);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// cost[i] = min(cost[i], cur[i]) (init != 0: cost[i] = min(max(T), cur[i])), then the block
// sums of cost in double with the fixed tree of block_sum. One workgroup per KPP_BLOCK rows.
// With near != null the pass also keeps which candidate the running minimum belongs to:
// cur_label[i] numbers the candidates of this pass from 0, label_off is the place of the
// first of them in the list of all candidates, and a later pass replaces an earlier
// candidate only with a strictly smaller distance, so near[i] ends as the nearest of all
// candidates with the lowest index on ties, which is what one pass over all of them gives.
template <typename T>
__global__ __launch_bounds__(WG) void fold_min_kernel(const T *__restrict__ cur, T *__restrict__ cost,
                                                     double *__restrict__ bsums, int64_t n,
                                                     int init, const int *__restrict__ cur_label,
                                                     int *__restrict__ near, int label_off) {
  __shared__ double red[WG];
  const int64_t b0 = (int64_t)blockIdx.x * KPP_BLOCK;
#pragma unroll
  for (int q = 0; q < KPP_BLOCK / WG; q++) {
    const int64_t row = b0 + threadIdx.x + q * WG;
    if (row < n) {
      const T prev = init ? std::numeric_limits<T>::max() : cost[row];
      const T c = cur[row];
      cost[row] = c < prev ? c : prev;
      if (near && (init || c < prev)) {
        const int l = cur_label[row];
        near[row] = l < 0 ? -1 : label_off + l;  // (a row without a finite distance has no label)
      }
    }
  }
  __syncthreads();  // (each thread re-reads only what it wrote; the barrier orders the LDS use)
  block_sum<T>(cost, bsums, blockIdx.x, n, red);
}
template <typename T>
int launch_fold_min(hipStream_t s, const T *cur, T *cost, double *bsums, int64_t n, int init,
                    const int *cur_label, int *near, int label_off) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL((fold_min_kernel<T>), dim3((unsigned)((n + KPP_BLOCK - 1) / KPP_BLOCK)),
                     dim3(WG), 0, s, cur, cost, bsums, n, init, cur_label, near, label_off);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// a * b mod (2^31 - 1) for a, b below the modulus
__device__ __forceinline__ uint32_t mulmod_m31(uint32_t a, uint32_t b) {
  const uint64_t p = (uint64_t)a * b;
  uint64_t r = (p & 0x7FFFFFFFull) + (p >> 31);
  r = (r & 0x7FFFFFFFull) + (r >> 31);
  return (uint32_t)(r >= 0x7FFFFFFFull ? r - 0x7FFFFFFFull : r);
}

// The acceptance test of kmeans_h2o4gpu.cu:436-456 for every row:
//   thrust::default_random_engine rng(seed); rng.discard(row);
//   T threshold = (T)thrust::uniform_real_distribution<>(0, 1)(rng);     (a float)
//   T prob = (2.0 * k * cost[row]) / total;                               (formed in double)
//   take the row when prob > threshold.
// The engine is minstd_rand (x <- 48271 x mod 2^31 - 1), so the value row `row` draws is
// state0 * 48271^(row+1); the distribution maps x to float(x - 1) / (1.0f + float(m - 2)).
// Rows taken are appended to list in arrival order (the host sorts them); *count may
// exceed cap, in which case only cap entries were written.
template <typename T>
__global__ __launch_bounds__(WG) void select_rows_kernel(const T *__restrict__ cost, T total,
                                                        uint32_t state0, int k,
                                                        int *__restrict__ list,
                                                        int *__restrict__ count, int cap,
                                                        int64_t n) {
  const int64_t row = (int64_t)blockIdx.x * WG + threadIdx.x;
  if (row >= n) return;
  uint32_t acc = state0, base = 48271u;
  for (uint64_t e = (uint64_t)row + 1; e != 0; e >>= 1) {
    if (e & 1) acc = mulmod_m31(acc, base);
    base = mulmod_m31(base, base);
  }
  float u = static_cast<float>(acc - 1u);
  u /= (1.0f + static_cast<float>(2147483645u));
  const T threshold = (T)u;
  const T prob = (T)((2.0 * k * (double)cost[row]) / (double)total);
  if (prob > threshold) {
    const int pos = atomicAdd(count, 1);
    if (pos < cap) list[pos] = (int)row;
  }
}
template <typename T>
int launch_select_rows(hipStream_t s, const T *cost, T total, uint32_t state0, int k, int *list,
                       int *count, int cap, int64_t n) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL((select_rows_kernel<T>), dim3((unsigned)((n + WG - 1) / WG)), dim3(WG), 0, s,
                     cost, total, state0, k, list, count, cap, n);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// counts[label]++ over all rows (count_functor, kmeans_h2o4gpu.h:44-72, whose argmin starts
// at candidate 0: a row no distance could be compared for counts there). Integer atomics:
// the result does not depend on their order.
__global__ __launch_bounds__(WG) void label_histogram_kernel(const int *__restrict__ labels,
                                                            int *__restrict__ counts, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * WG;
  for (int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x; i < n; i += stride) {
    const int l = labels[i];
    atomicAdd(&counts[l < 0 ? 0 : l], 1);
  }
}
int launch_label_histogram(hipStream_t s, const int *labels, int *counts, int64_t n) {
  if (n <= 0) return 0;
  const unsigned blocks = (unsigned)std::min<int64_t>((n + WG - 1) / WG, 2048);
  hipLaunchKernelGGL(label_histogram_kernel, dim3(blocks), dim3(WG), 0, s, labels, counts, n);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// Column-major copy of the m candidate rows: out[j * m + i] = Cc[i * d + j], so that the
// kernel below reads a feature of consecutive candidates with consecutive lanes.
template <typename T>
__global__ __launch_bounds__(WG) void transpose_candidates_kernel(const T *__restrict__ Cc, T *__restrict__ out,
                                                                  int m, int d) {
  __shared__ T tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8 threads
  const int i0 = blockIdx.x * 32, j0 = blockIdx.y * 32;
  for (int r = ty; r < 32; r += WG / 32) {
    const int i = i0 + r, jj = j0 + tx;
    tile[r][tx] = (i < m && jj < d) ? Cc[(size_t)i * d + jj] : (T)0;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += WG / 32) {
    const int jj = j0 + r, i = i0 + tx;
    if (i < m && jj < d) out[(size_t)jj * m + i] = tile[tx][r];
  }
}
template <typename T>
int launch_transpose_candidates(hipStream_t s, const T *Cc, T *out, int m, int d) {
  if (m <= 0) return 0;
  hipLaunchKernelGGL((transpose_candidates_kernel<T>), dim3((unsigned)((m + 31) / 32), (unsigned)((d + 31) / 32)),
                     dim3(WG), 0, s, Cc, out, m, d);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// One step of the host k-means++ over the candidates (kmeans_h2o4gpu.cu:226-271), the part
// that touches every candidate: v = (xx + cc) - 2 x.c against candidate `centre` (the
// expanded form of src/common/utils.cpp:34-57, no absolute value), best = v at the first
// step, min(v, best) afterwards with best[centre] taken as 0. One thread per candidate sums
// its dot product over the features in ascending order, product and sum rounded separately,
// as a scalar loop does; CcT is the column-major copy of the candidates, so the loads of a
// wavefront are contiguous.
template <typename T>
__global__ __launch_bounds__(WG) void candidate_dists_kernel(const T *__restrict__ Cc, const T *__restrict__ CcT,
                                                            const T *__restrict__ ccn, int centre,
                                                            T *__restrict__ best, T *__restrict__ mirror, int m,
                                                            int d, int first) {
#pragma clang fp contract(off)
  const int i = blockIdx.x * WG + threadIdx.x;
  if (i >= m) return;
  const T *c = Cc + (size_t)centre * d;
  T dot = 0;
  for (int j = 0; j < d; j++) dot = dot + CcT[(size_t)j * m + i] * c[j];
  const T t = ccn[i] + ccn[centre];
  const T v = (T)-2 * dot + t;
  T nb = v;
  if (!first) {
    const T prev = i == centre ? (T)0 : best[i];
    nb = v < prev ? v : prev;
  }
  best[i] = nb;
  if (mirror) mirror[i] = nb;
}
// The same step with lpr lanes sharing a candidate (strided partial sums, then a tree over
// the lanes): another summation order, an order of magnitude faster when there are few
// thousand candidates of several hundred features (8304 x 784: 14 against 164 us per pick).
template <typename T>
__global__ __launch_bounds__(WG) void candidate_dists_tree_kernel(const T *__restrict__ Cc,
                                                                 const T *__restrict__ ccn, int centre,
                                                                 T *__restrict__ best, T *__restrict__ mirror,
                                                                 int m, int d, int first, int lpr) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rps = 64 / lpr;
  const int i = (blockIdx.x * (WG / 64) + wave) * rps + lane / lpr;
  const int col = lane % lpr;
  const T *x = Cc + (size_t)(i < m ? i : m - 1) * d;
  const T *c = Cc + (size_t)centre * d;
  T dot = 0;
  for (int j = col; j < d; j += lpr) dot += x[j] * c[j];
  for (int off = 1; off < lpr; off <<= 1) dot += __shfl_xor(dot, off, 64);
  if (col == 0 && i < m) {
    const T t = ccn[i] + ccn[centre];
    const T v = (T)-2 * dot + t;
    T nb = v;
    if (!first) {
      const T prev = i == centre ? (T)0 : best[i];
      nb = v < prev ? v : prev;
    }
    best[i] = nb;
    if (mirror) mirror[i] = nb;
  }
}
// CcT null: the lane-parallel form on the row-major candidates. mirror (may be null): a second
// copy of the result, meant for pinned host memory that the device writes directly, which
// spares the caller a copy command per step.
template <typename T>
int launch_candidate_dists(hipStream_t s, const T *Cc, const T *CcT, const T *ccn, int centre, T *best,
                           T *mirror, int m, int d, int first) {
  if (m <= 0) return 0;
  if (CcT) {
    hipLaunchKernelGGL((candidate_dists_kernel<T>), dim3((unsigned)((m + WG - 1) / WG)), dim3(WG), 0, s, Cc,
                       CcT, ccn, centre, best, mirror, m, d, first);
  } else {
    int lpr = 1;
    while (lpr < d && lpr < 64) lpr <<= 1;
    const int rows_per_block = (WG / 64) * (64 / lpr);
    hipLaunchKernelGGL((candidate_dists_tree_kernel<T>),
                       dim3((unsigned)((m + rows_per_block - 1) / rows_per_block)), dim3(WG), 0, s, Cc, ccn,
                       centre, best, mirror, m, d, first, lpr);
  }
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

#define KM_SEED_INSTANTIATE(T)                                                                  \
  template int launch_gather_model<T>(hipStream_t, const T *, const T *, const int *, int, int, \
                                      T *, T *, int);                                           \
  template int launch_fold_min<T>(hipStream_t, const T *, T *, double *, int64_t, int,          \
                                  const int *, int *, int);                                     \
  template int launch_select_rows<T>(hipStream_t, const T *, T, uint32_t, int, int *, int *,    \
                                     int, int64_t);                                             \
  template int launch_transpose_candidates<T>(hipStream_t, const T *, T *, int, int);           \
  template int launch_candidate_dists<T>(hipStream_t, const T *, const T *, const T *, int, T *, \
                                         T *, int, int, int);
KM_SEED_INSTANTIATE(float)
KM_SEED_INSTANTIATE(double)

template int launch_min_dist_update<float>(hipStream_t, const float *, const float *, int64_t,
                                           float *, int *, int *, float *, int, double *, int64_t,
                                           int);
template int launch_min_dist_update<double>(hipStream_t, const double *, const double *, int64_t,
                                            double *, int *, int *, double *, int, double *,
                                            int64_t, int);

}  // namespace kmhip
