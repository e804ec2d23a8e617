// Long rows, a handful of centroids: one pass over X per Lloyd iteration.
//
// For k <= 16 and rows too long for the small-model kernels (more than 64 features) the
// matrix cores have nothing to offer (2 k d flop per 4 d bytes) and the reference's
// formulation, a GEMM for the distances (kmeans_labels.cu:158-165) and a second pass over the
// rows for the sums (kmeans_centroids.h:40-75), reads X twice. Here a wavefront takes four
// rows at a time with its 64 lanes side by side along the features (coalesced 16-byte
// loads, the rows stay in registers), forms the 4 x k partial dot products per lane against
// centroids staged once per workgroup in LDS, adds the partials of the 64 lanes with a
// transposing butterfly (63 exchanges for 64 sums instead of 6 each; fewer for 8 or 4
// centroids), closes the argmin among the lanes that end up with a row's distances, and adds
// the rows, still in their registers, into double-precision sums in LDS (component-major, so
// that the lanes of a wavefront add to consecutive doubles). Labels, minimum distances,
// per-workgroup partial sums and counts come out as from the other fused kernels.
//
// Semantics as everywhere (kmeans_labels.h:216-244, :360-377): dist = |(xx + cc) - 2 x.c|,
// strict '<' from FLT_MAX, lowest index on ties, label -1 when nothing is below the start
// value; the dot product is summed in another order than a scalar loop's, so parity with
// the CPU restatement is the matrix-core kernels' (near-tie rule), not bit for bit.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "kmeans_common.h"
#include "mfma_traits.h"

namespace kmhip {

namespace {

constexpr int LR_WG = 512;  // 8 wavefronts
constexpr int LR_NW = LR_WG / 64;
constexpr int LR_R = 4;    // rows per wavefront and step
constexpr int LR_KP = 16;  // centroids at most (a launch pads k to 4, 8 or 16)
constexpr int LR_MAX_NVL = 4;
constexpr size_t LR_LDS_MAX = 150 * 1024;

// lane -> the sum it holds after a butterfly over 2^NB values: bit s of the lane (s < NB) is
// bit NB - 1 - s of the index
template <int NB>
__device__ __forceinline__ int butterfly_index(int lane) {
  int i = 0;
#pragma unroll
  for (int s = 0; s < NB; s++) i |= ((lane >> s) & 1) << (NB - 1 - s);
  return i;
}

template <typename T>
size_t longrow_lds(int d, int k, bool sums) {
  return (size_t)k * d * sizeof(T) + LR_KP * sizeof(T) + LR_KP * sizeof(int) +
         (sums ? (size_t)k * d * sizeof(double) : 0);
}

template <typename T, int NVL, int KP, bool SUMS>
__global__ __launch_bounds__(LR_WG) void lloyd_longrow_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm, const T *__restrict__ C,
    const T *__restrict__ cnorm, int *__restrict__ labels, T *__restrict__ mindist,
    double *__restrict__ psums, int *__restrict__ pcounts, int64_t n, int d, int k) {
#pragma clang fp contract(off)
  typedef Mfma<T> M;
  constexpr int VW = M::VW;
  typedef typename M::vec_t vec_t;
  typedef typename M::uvec_t uvec_t;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int dq = d / VW;  // 16-byte vectors per row
  vec_t *cs = reinterpret_cast<vec_t *>(smem_raw);             // [k][dq]
  T *ccs = reinterpret_cast<T *>(cs + (size_t)k * dq);        // [LR_KP]
  int *cnt = reinterpret_cast<int *>(ccs + LR_KP);            // [LR_KP]
  double *sums = reinterpret_cast<double *>(cnt + LR_KP);     // [k][VW][dq]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  for (int e = tid; e < k * dq; e += LR_WG) {
    const uvec_t u = *reinterpret_cast<const uvec_t *>(C + (size_t)e * VW);
    vec_t v;
#pragma unroll
    for (int q = 0; q < VW; q++) v[q] = u[q];
    cs[e] = v;
  }
  if (SUMS) {
    for (int e = tid; e < k * d; e += LR_WG) sums[e] = 0.0;
    if (tid < LR_KP) cnt[tid] = 0;
  }
  __syncthreads();
  if (tid < LR_KP) {
    // squared norms: the stored ones, or (a loop that skips the post-update pass) the value
    // row_norms would store, summed in feature order with separate multiply and add
    T acc = pos_inf<T>();
    if (tid < k) {
      if (cnorm) {
        acc = cnorm[tid];
      } else {
        const T *crow = reinterpret_cast<const T *>(cs) + (size_t)tid * d;
        acc = 0;
        for (int j = 0; j < d; j++) {
          const T v = crow[j];
          acc = acc + v * v;
        }
      }
    }
    ccs[tid] = acc;
  }
  __syncthreads();

  const int64_t ngroups = (n + LR_R - 1) / LR_R;
  // which of the LR_R * KP sums this lane ends up with: row r of the step, centroid kk
  constexpr int NV = LR_R * KP;
  constexpr int NB = NV == 64 ? 6 : (NV == 32 ? 5 : 4);
  static_assert(NV == (1 << NB), "a power of two of sums, 64 at most");
  const int mine = butterfly_index<NB>(lane);
  const int my_r = mine / KP, my_k = mine % KP;
  const bool last_valid = lane + 64 * (NVL - 1) < dq;  // the last vector of this lane exists
  for (int64_t g = (int64_t)blockIdx.x * LR_NW + wave; g < ngroups; g += (int64_t)gridDim.x * LR_NW) {
    const int64_t row0 = g * LR_R;
    vec_t x[LR_R][NVL];
#pragma unroll
    for (int r = 0; r < LR_R; r++) {
      const T *xr = X + min(row0 + r, n - 1) * (int64_t)d;
#pragma unroll
      for (int j = 0; j < NVL; j++) {
        const int v = min(lane + 64 * j, dq - 1);  // clamped: stays inside the row
        const uvec_t u = *reinterpret_cast<const uvec_t *>(xr + (size_t)v * VW);
#pragma unroll
        for (int q = 0; q < VW; q++) x[r][j][q] = u[q];
      }
    }
    T val[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) val[i] = 0;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
      if (j + 1 < NVL || last_valid) {
        const vec_t *cp = cs + lane + 64 * j;
#pragma unroll
        for (int kk = 0; kk < KP; kk++) {
          if (kk < k) {  // (the same for the whole workgroup)
            const vec_t c = cp[(size_t)kk * dq];
#pragma unroll
            for (int r = 0; r < LR_R; r++) {
#pragma unroll
              for (int q = 0; q < VW; q++) val[r * KP + kk] = fma(x[r][j][q], c[q], val[r * KP + kk]);
            }
          }
        }
      }
    }
    // The sums over the 64 lanes: at step s a lane keeps the half of its values that its
    // bit s selects and receives its partner's partials of the same half; once a single value
    // is left (fewer than 64 sums) the remaining lane bits are plain exchanges.
#pragma unroll
    for (int s = 0; s < NB; s++) {
      const int half = (NV / 2) >> s;
      const bool up = (lane >> s) & 1;
#pragma unroll
      for (int i = 0; i < half; i++) {
        const T lo = val[i], hi = val[i + half];
        const T keep = up ? hi : lo;
        const T send = up ? lo : hi;
        val[i] = keep + __shfl_xor(send, 1 << s, 64);
      }
    }
#pragma unroll
    for (int s = NB; s < 6; s++) val[0] = val[0] + __shfl_xor(val[0], 1 << s, 64);
    const int64_t my_row = row0 + my_r;
    T best = argmin_start<T>();
    int bidx = -1;
    if (my_k < k) {
      const T t = xnorm[min(my_row, n - 1)] + ccs[my_k];
      const T dist = fabs(t - (T)2 * val[0]);
      if (dist < best) {
        best = dist;
        bidx = my_k;
      }
    }
    // the lanes of a row differ in lane bits 2..5
#pragma unroll
    for (int m = 4; m < 64; m <<= 1) {
      const T ob = __shfl_xor(best, m, 64);
      const int oi = __shfl_xor(bidx, m, 64);
      argmin_merge(best, bidx, ob, oi);
    }
    if (my_k == 0 && (lane >> NB) == 0 && my_row < n) {  // (one of the lanes that hold the row's result)
      labels[my_row] = bidx;
      if (mindist) mindist[my_row] = best;
    }
    if (SUMS) {
#pragma unroll
      for (int r = 0; r < LR_R; r++) {
        // row r's result sits in the lanes whose index has r in its two highest bits; the first
        // of them is lane (r >> 1) | ((r & 1) << 1)
        const int lab = __builtin_amdgcn_readlane(bidx, (r >> 1) | ((r & 1) << 1));
        if (row0 + r < n && lab >= 0) {
          double *srow = sums + (size_t)lab * d;
#pragma unroll
          for (int j = 0; j < NVL; j++) {
            if (j + 1 < NVL || last_valid) {
#pragma unroll
              for (int q = 0; q < VW; q++)
                unsafeAtomicAdd(srow + (size_t)q * dq + lane + 64 * j, (double)x[r][j][q]);
            }
          }
          if (lane == 0) atomicAdd(&cnt[lab], 1);
        }
      }
    }
  }
  if (!SUMS) return;
  __syncthreads();
  double *dst = psums + (size_t)blockIdx.x * k * d;
  for (int e = tid; e < k * d; e += LR_WG) {
    const int c = e / d, f = e - c * d;
    dst[e] = sums[(size_t)c * d + (size_t)(f % VW) * dq + f / VW];
  }
  int *cdst = pcounts + (size_t)blockIdx.x * k;
  for (int c = tid; c < k; c += LR_WG) cdst[c] = cnt[c];
}

}  // namespace

template <typename T>
bool longrow_applies(int d, int k) {
  const int vw = Mfma<T>::VW;
  if (k < 1 || k > LR_KP || d <= 64 || d % vw != 0) return false;
  if (d / vw > 64 * LR_MAX_NVL) return false;
  return longrow_lds<T>(d, k, true) <= LR_LDS_MAX;
}

template <typename T>
int longrow_max_slots(int d, int k, int num_cu) {
  const size_t lds = longrow_lds<T>(d, k, true);
  const int per_cu = (int)std::min<size_t>(4, std::max<size_t>(1, ((size_t)160 * 1024) / lds));
  return per_cu * num_cu;
}

template <typename T, bool SUMS>
int launch_longrow(hipStream_t s, const T *X, const T *xnorm, const T *C, const T *cnorm, int *labels,
                   T *mindist, int64_t n, int d, int k, int num_cu, double *psums, int *pcounts,
                   int *slots) {
  if (!longrow_applies<T>(d, k)) return H2O4GPU_KMEANS_EARG;
  const int dq = d / Mfma<T>::VW;
  const int nvl = (dq + 63) / 64;
  const size_t lds = longrow_lds<T>(d, k, SUMS);
  const int64_t groups = (n + LR_R - 1) / LR_R;
  int grid = 1;
#define KM_LR(NVL)                                                                                 \
  do {                                                                                             \
    if (k <= 4) KM_LR_K(NVL, 4);                                                                   \
    else if (k <= 8) KM_LR_K(NVL, 8);                                                              \
    else KM_LR_K(NVL, 16);                                                                         \
  } while (0)
#define KM_LR_K(NVL, KP)                                                                           \
  do {                                                                                             \
    auto kern = lloyd_longrow_kernel<T, NVL, KP, SUMS>;                                            \
    KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds));                         \
    int per_cu = resident_blocks_per_cu(reinterpret_cast<const void *>(kern), LR_WG, lds);         \
    if (per_cu < 1) per_cu = 1;                                                                    \
    if (SUMS) per_cu = std::min(per_cu, longrow_max_slots<T>(d, k, 1));                            \
    grid = (int)std::min<int64_t>((int64_t)per_cu * num_cu, (groups + LR_NW - 1) / LR_NW);         \
    if (grid < 1) grid = 1;                                                                        \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(LR_WG), lds, s, X, xnorm, C, cnorm, labels, mindist, \
                       psums, pcounts, n, d, k);                                                   \
  } while (0)
  switch (nvl) {
    case 1: KM_LR(1); break;
    case 2: KM_LR(2); break;
    case 3: KM_LR(3); break;
    case 4: KM_LR(4); break;
    default: return H2O4GPU_KMEANS_EARG;
  }
#undef KM_LR
#undef KM_LR_K
  KM_HIP_TRY(hipGetLastError());
  if (slots) *slots = grid;
  return 0;
}

template bool longrow_applies<float>(int, int);
template bool longrow_applies<double>(int, int);
template int longrow_max_slots<float>(int, int, int);
template int longrow_max_slots<double>(int, int, int);
template int launch_longrow<float, true>(hipStream_t, const float *, const float *, const float *, const float *,
                                         int *, float *, int64_t, int, int, int, double *, int *, int *);
template int launch_longrow<float, false>(hipStream_t, const float *, const float *, const float *, const float *,
                                          int *, float *, int64_t, int, int, int, double *, int *, int *);
template int launch_longrow<double, true>(hipStream_t, const double *, const double *, const double *,
                                          const double *, int *, double *, int64_t, int, int, int, double *, int *,
                                          int *);
template int launch_longrow<double, false>(hipStream_t, const double *, const double *, const double *,
                                           const double *, int *, double *, int64_t, int, int, int, double *, int *,
                                           int *);

}  // namespace kmhip
