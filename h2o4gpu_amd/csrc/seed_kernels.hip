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

// mind[i] = min(mind[i], |(xx_i + cc) - 2 x_i.c|) for the centre c = row
// `centre_row` of X (init != 0: overwrite). One workgroup per KPP_BLOCK rows;
// lpr lanes share a row so loads are coalesced. Afterwards the workgroup sums
// its KPP_BLOCK minima in double with a fixed tree into bsums[block].
template <typename T>
__global__ __launch_bounds__(WG) void min_dist_update_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm, int64_t centre_row,
    T *__restrict__ mind, double *__restrict__ bsums, int64_t n, int d, int init,
    int lpr) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *cs = reinterpret_cast<T *>(smem_raw);  // [d]
  __shared__ double red[WG];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  for (int j = tid; j < d; j += WG) cs[j] = X[centre_row * (int64_t)d + j];
  const T cc = xnorm[centre_row];
  __syncthreads();
  const int64_t b0 = (int64_t)blockIdx.x * KPP_BLOCK;
  const int rps = 64 / lpr;
  const int sub = lane / lpr, col = lane % lpr;
  for (int r = wave * rps + sub; r < KPP_BLOCK; r += (WG / 64) * rps) {
    const int64_t row = b0 + r;
    T dot = 0;
    if (row < n) {
      const T *x = X + row * (int64_t)d;
      for (int j = col; j < d; j += lpr) dot += x[j] * cs[j];
    }
    for (int off = 1; off < lpr; off <<= 1) dot += __shfl_xor(dot, off, 64);
    if (col == 0 && row < n) {
      const T t = xnorm[row] + cc;
      T dist = fabs(t - (T)2 * dot);
      if (!init) dist = fmin(dist, mind[row]);
      mind[row] = dist;
    }
  }
  __syncthreads();
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
  if (tid == 0) bsums[blockIdx.x] = red[0];
}

template <typename T>
int launch_min_dist_update(hipStream_t s, const T *X, const T *xnorm,
                           int64_t centre_row, T *mind, double *bsums, int64_t n,
                           int d, int init) {
  if (n <= 0) return 0;
  int lpr = 1;
  while (lpr < d && lpr < 64) lpr <<= 1;
  const unsigned blocks = (unsigned)((n + KPP_BLOCK - 1) / KPP_BLOCK);
  hipLaunchKernelGGL((min_dist_update_kernel<T>), dim3(blocks), dim3(WG),
                     (size_t)d * sizeof(T), s, X, xnorm, centre_row, mind, bsums, n, d,
                     init, lpr);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template int launch_min_dist_update<float>(hipStream_t, const float *, const float *,
                                           int64_t, float *, double *, int64_t, int, int);
template int launch_min_dist_update<double>(hipStream_t, const double *, const double *,
                                            int64_t, double *, double *, int64_t, int, int);

}  // namespace kmhip
