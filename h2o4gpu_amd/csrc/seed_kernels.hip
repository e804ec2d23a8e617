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

template int launch_min_dist_update<float>(hipStream_t, const float *, const float *, int64_t,
                                           float *, int *, int *, float *, int, double *, int64_t,
                                           int);
template int launch_min_dist_update<double>(hipStream_t, const double *, const double *, int64_t,
                                            double *, int *, int *, double *, int, double *,
                                            int64_t, int);

}  // namespace kmhip
