// Fused distance + argmin ("assign") and full distance ("transform") kernels.
//
// Replaces, in one pass over the data and without an n x k buffer, the
// reference sequence make_self_dots(C) -> all_dots -> matmul|cublas gemm ->
// absolute_value -> make_new_labels
// (src/gpu/kmeans/kmeans_labels.cu:183-244, kmeans_labels.h:187-244,360-392).
// Kept from the reference: dist = |(xx + cc) - 2 x.c| with xx + cc rounded
// first, strict '<' argmin, lowest index on ties, start value FLT_MAX, label -1
// when nothing is below it.
#include <type_traits>

#include "kmeans_common.h"
#include "mfma_traits.h"

namespace kmhip {

static constexpr int WG = 256;  // threads per workgroup (4 wavefronts)

// Row stride (in values) of a block of rows staged in LDS for one-thread-per-row access.
// Odd, so that thread t reading row t is conflict-free, and never 2^m - 1: with 31 or 63
// the staged kernels ran 1.6x slower than with their neighbours (measured: d = 30, 31, 62, 63).
__host__ __device__ static inline int staged_row_stride(int d) {
  int sx = d | 1;
  if (((sx + 1) & sx) == 0) sx += 2;
  return sx;
}

// Squared norm of one centroid row, j ascending, multiply and add rounded separately:
// the value row_norms / post_update would store (kmeans_labels.h:187-199). The fused
// kernels call it when they are given no norm buffer, which spares the Lloyd loop a launch.
template <typename T>
__device__ __forceinline__ T row_sqnorm(const T *__restrict__ x, int d) {
#pragma clang fp contract(off)
  T acc = 0;
  for (int j = 0; j < d; j++) {
    const T v = x[j];
    acc = acc + v * v;
  }
  return acc;
}

// Features [j, j + VW) of a row of d >= VW values that is aligned to its elements only;
// features at or past d come back as zero. The load never leaves the row: a vector that
// would reach past the end is taken from the row's last VW values and shifted down. The
// shift is skipped when no lane of the wavefront needs it.
template <typename T>
__device__ __forceinline__ typename Mfma<T>::vec_t load_row_vector(const T *__restrict__ row, int j,
                                                                   int d) {
  constexpr int VW = Mfma<T>::VW;
  const int jc = min(j, d - VW);
  const int s = j - jc;  // 0: the vector lies inside the row
  const typename Mfma<T>::uvec_t v = *reinterpret_cast<const typename Mfma<T>::uvec_t *>(row + jc);
  typename Mfma<T>::vec_t o;
#pragma unroll
  for (int e = 0; e < VW; e++) o[e] = v[e];
  if (__builtin_amdgcn_ballot_w64(s != 0) != 0) {
#pragma unroll
    for (int e = 0; e < VW; e++) {
      T x = 0;
#pragma unroll
      for (int t = e; t < VW; t++) x = (s == t - e) ? v[t] : x;
      o[e] = x;
    }
  }
  return o;
}

// ---------------------------------------------------------------------------
// VALU variant: one thread per row, a chunk of centroids broadcast from LDS.
// Arithmetic order is j ascending with separate multiply and add, so this
// kernel reproduces a scalar CPU loop bit for bit. It carries the small shapes
// (the reference's own k <= 16 && d <= 64 path) and is the any-shape fallback.
// MODE 0: labels (+ optional mindist).  MODE 1: full distances D[c*ldn + i].
// ---------------------------------------------------------------------------
template <typename T, int DREG, int MODE>
__global__ __launch_bounds__(WG) void assign_valu_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm,
    const T *__restrict__ C, const T *__restrict__ cnorm,
    int *__restrict__ labels, T *__restrict__ mindist, T *__restrict__ D,
    int64_t n, int64_t ldn, int d, int k, int kc) {
#pragma clang fp contract(off)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *Cs = reinterpret_cast<T *>(smem_raw);  // [kc][d]
  T *ccs = Cs + (size_t)kc * d;             // [kc]
  const int tid = threadIdx.x;
  const int64_t row = (int64_t)blockIdx.x * WG + tid;
  const bool valid = row < n;
  const T *x = X + (valid ? row : 0) * (int64_t)d;
  T xr[DREG > 0 ? DREG : 1];
  if (DREG > 0) {
#pragma unroll
    for (int j = 0; j < DREG; j++) xr[j] = (valid && j < d) ? x[j] : (T)0;
  }
  const T xx = valid ? xnorm[row] : (T)0;
  T best = argmin_start<T>();
  int bidx = -1;
  for (int c0 = 0; c0 < k; c0 += kc) {
    const int nc = min(kc, k - c0);
    __syncthreads();
    for (int e = tid; e < nc * d; e += WG) Cs[e] = C[(size_t)c0 * d + e];
    for (int c = tid; c < nc; c += WG) ccs[c] = cnorm[c0 + c];
    __syncthreads();
    if (!valid) continue;
    for (int c = 0; c < nc; c++) {
      const T *cp = Cs + (size_t)c * d;
      T dot = 0;
      if (DREG > 0) {
#pragma unroll
        for (int j = 0; j < DREG; j++)
          if (j < d) dot = dot + xr[j] * cp[j];
      } else {
        for (int j = 0; j < d; j++) dot = dot + x[j] * cp[j];
      }
      T t = xx + ccs[c];
      T dist = fabs(t - (T)2 * dot);
      if (MODE == 1) {
        D[(size_t)(c0 + c) * ldn + row] = dist;
      } else if (dist < best) {
        best = dist;
        bidx = c0 + c;
      }
    }
  }
  if (MODE == 0 && valid) {
    labels[row] = bidx;
    if (mindist) mindist[row] = best;
  }
}

// ---------------------------------------------------------------------------
// VALU Lloyd step for the small shapes (k <= 16, d <= 64): assignment and
// per-centroid accumulation in one pass over the data.
//
// Persistent workgroups walk over blocks of 256 rows. A block is fetched with
// coalesced 16-byte loads into registers while the previous
// block is being processed, then written to LDS with an odd row stride so that
// thread t reading row t is conflict-free. Every thread runs the same scalar
// loop as assign_valu_kernel on its row (j ascending, multiply and add rounded
// separately: bit-identical to a CPU loop); the centroid values have a
// wavefront-uniform address and are read straight from global memory, which
// lets them travel through the scalar path instead of LDS. The thread then
// adds its row into the double-precision per-centroid sums of the workgroup.
// Sums and counts go to the workgroup's slot psums[blockIdx.x][k][d],
// pcounts[blockIdx.x][k].
// This is the HBM-bound regime: 2*k*d flop per row against d*s bytes.
// This kernel: d == DREG (4, 8, 16, 32 or 64), the row held in registers and the loops
// over d unrolled; the data must be 16-byte aligned.
// ---------------------------------------------------------------------------
template <typename T, int VEC>
struct BlockLoad {  // VEC is Mfma<T>::VW (one 16-byte load) or 1
  typedef typename Mfma<T>::vec_t type;
};
template <typename T>
struct BlockLoad<T, 1> {
  typedef T type;
};
// Layout of the per-centroid sums of the two fused kernels in LDS: `ncopy` copies (1, 2 or 4),
// copy (lane / 16) % ncopy for the lanes of a wavefront, [copy][centroid][sxs] doubles, sxs =
// d rounded up to 16 (d itself below 16). A lane adds its row starting at feature lane % 16,
// so at any moment the 16 lanes of a group add 16 consecutive features, and with a centroid
// stride of 0 or 16 (mod 32) doubles those are 16 different bank pairs whatever the labels
// are; the groups of a wavefront add into copies of their own. Measured on the LDS pipe
// alone (8 labels, 16 features): 6.7 lane additions per clock and CU against 2.6 for one
// copy with an odd centroid stride (7.6 with no conflict at all).
__host__ __device__ static inline int sums_stride(int d) { return d < 16 ? d : (d + 15) / 16 * 16; }

template <typename T, int DREG, bool SUMS>
__global__ __launch_bounds__(WG) void lloyd_valu_fused_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm, const T *__restrict__ C,
    const T *__restrict__ cnorm, int *__restrict__ labels, T *__restrict__ mindist,
    double *__restrict__ psums, int *__restrict__ pcounts, int64_t n, int k,
    T *__restrict__ D, int64_t ldn, int ncopy) {
#pragma clang fp contract(off)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  constexpr int d = DREG;
  // D (assignment-only form): write every distance to D[c * ldn + row] instead of labels
  const bool full = !SUMS && D != nullptr;
  constexpr int VEC = Mfma<T>::VW;
  // Rows are staged with a stride of d + one 16-byte vector: every staged vector and every
  // row start stays 16-byte aligned (one ds_write_b128 per fetched vector, d / VEC
  // ds_read_b128 per row), and the 8 lanes such an access serves per clock fall on
  // different banks for every d here (d = VEC needs no padding: the rows are lane-linear).
  constexpr int SXT = DREG == VEC ? DREG : DREG + VEC;
  constexpr int sxs = DREG;  // = sums_stride(DREG): DREG is a power of two
  // SUMS false: assignment only (predict, final relabel, inertia): no sums, no counts
  const int kq = (k + 3) & ~3;
  double *sums = reinterpret_cast<double *>(smem_raw);                      // [ncopy][k][sxs]
  int *cnt = reinterpret_cast<int *>(sums + (SUMS ? (size_t)ncopy * k * sxs : 0));  // [kq]
  T *ccs = reinterpret_cast<T *>(cnt + (SUMS ? kq : 0));                    // [kq] centroid norms
  T *Xs = ccs + kq;                                                         // [WG][SXT], 16-byte aligned
  typedef typename BlockLoad<T, VEC>::type ld_t;
  constexpr int NLD = DREG / VEC;  // 16-byte vectors per row = loads per thread and block
  const int tid = threadIdx.x;
  if (SUMS) {
    for (int e = tid; e < ncopy * k * sxs; e += WG) sums[e] = 0.0;
    for (int c = tid; c < k; c += WG) cnt[c] = 0;
  }
  // vector tid + i*WG of the block is vector tid % NLD of row tid / NLD + i * (WG / NLD)
  const int st_off = (tid / NLD) * SXT + (tid % NLD) * VEC;
  ld_t pre[NLD];
  // Loads are never predicated: indices past the end of the data set are
  // clamped instead, which keeps the loop free of divergent branches and lets
  // the fetched block stay in flight across the processing of the current one.
  auto fetch = [&](int64_t base) {
    const int64_t last = (n - base) * d / VEC - 1;  // last load of the data set
    const ld_t *src = reinterpret_cast<const ld_t *>(X + base * (int64_t)d);
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      const int64_t e = tid + i * WG;
      // (every row is read once per pass: a load that does not displace cached lines measured
      // 6.0 against 5.5 TB/s in a plain streaming kernel)
      pre[i] = __builtin_nontemporal_load(&src[e < last ? e : last]);
    }
  };
  const int64_t stride = (int64_t)gridDim.x * WG;
  int64_t base = (int64_t)blockIdx.x * WG;
  if (base >= n) return;  // the grid never exceeds the number of blocks
  fetch(base);
  // centroid norms while the first block travels (visible after the barrier below)
  for (int c = tid; c < k; c += WG) ccs[c] = cnorm ? cnorm[c] : row_sqnorm<T>(C + (size_t)c * d, d);
  const int l16 = tid & 15;
  double *const my_sums = sums + (size_t)((tid >> 4) & (ncopy - 1)) * k * sxs;
  for (; base < n; base += stride) {
    const int rows = (int)min<int64_t>(WG, n - base);
    __syncthreads();  // the previous block has been consumed
#pragma unroll
    for (int i = 0; i < NLD; i++)  // rows past the end of a last, partial block hold clamped copies
      *reinterpret_cast<ld_t *>(Xs + st_off + i * (WG / NLD) * SXT) = pre[i];
    __syncthreads();
    // the next block travels while this one is processed: no other vector
    // load is issued below, so nothing waits for these until the next round
    fetch(base + stride < n ? base + stride : base);
    const int64_t row = base + tid;
    if (tid < rows) {
      const T *xrow = Xs + tid * SXT;
      T xr[DREG];
#pragma unroll
      for (int q = 0; q < NLD; q++) {
        const ld_t v = *reinterpret_cast<const ld_t *>(xrow + q * VEC);
#pragma unroll
        for (int e = 0; e < VEC; e++) xr[q * VEC + e] = v[e];
      }
      // the row's squared norm, j ascending, multiply and add rounded separately: the value
      // row_norms stores (kmeans_labels.h:187-199), without reading it back from memory
      T xx = 0;
#pragma unroll
      for (int j = 0; j < DREG; j++) xx = xx + xr[j] * xr[j];
      T best = argmin_start<T>();
      int bidx = -1;
#pragma unroll 2
      for (int c = 0; c < k; c++) {
        const T *cp = C + (size_t)c * d;
        T dot = 0;
#pragma unroll
        for (int j = 0; j < DREG; j++) dot = dot + xr[j] * cp[j];
        const T t = xx + ccs[c];
        const T dist = fabs(t - (T)2 * dot);
        if (full) D[(size_t)c * ldn + row] = dist;
        if (dist < best) {
          best = dist;
          bidx = c;
        }
      }
      if (!full) {
        labels[row] = bidx;
        if (mindist) mindist[row] = best;
      }
      if (SUMS && bidx >= 0) {
        double *srow = my_sums + (size_t)bidx * sxs;
#pragma unroll 4
        for (int q = 0; q < d; q++) {
          const int j = (l16 + q) & (d - 1);
          unsafeAtomicAdd(srow + j, (double)xrow[j]);
        }
        atomicAdd(&cnt[bidx], 1);
      }
    }
  }
  if (!SUMS) return;
  __syncthreads();
  double *dst = psums + (size_t)blockIdx.x * k * d;
  for (int e = tid; e < k * d; e += WG) {
    const int c = e / d, j = e - c * d;
    double v = sums[(size_t)c * sxs + j];
    for (int cp = 1; cp < ncopy; cp++) v += sums[((size_t)cp * k + c) * sxs + j];  // copy order
    dst[e] = v;
  }
  int *cdst = pcounts + (size_t)blockIdx.x * k;
  for (int c = tid; c < k; c += WG) cdst[c] = cnt[c];
}

// ---------------------------------------------------------------------------
// The same Lloyd step for a feature count that is not one of the register sizes
// above. Two things differ.
// Loop order: features outside, centroids inside, one running dot product per
// centroid in registers (KREG of them), the row read from its staged copy in LDS
// one value at a time and the centroid values, whose addresses are
// wavefront-uniform, through the scalar path. Nothing is unrolled over d, so no
// guard sits in the inner loop; every dot product still adds its terms with j
// ascending, multiply and add rounded separately.
// Staging: a block of 256 rows is one contiguous run of 256*d values that starts
// on a 16-byte boundary whatever d is, so it is fetched as a flat array of
// 16-byte vectors (VEC values each); a vector may straddle two rows, which only
// matters for the LDS offset of its values. The last, partial block of the data
// set is fetched value by value.
// DMAX bounds d (it sizes the register prefetch of the next block); d >= VEC.
// ---------------------------------------------------------------------------
template <typename T, int DMAX, int VEC, int KREG, bool SUMS>
__global__ __launch_bounds__(WG) void lloyd_valu_anyd_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm, const T *__restrict__ C,
    const T *__restrict__ cnorm, int *__restrict__ labels, T *__restrict__ mindist,
    double *__restrict__ psums, int *__restrict__ pcounts, int64_t n, int d, int k,
    T *__restrict__ D, int64_t ldn, int ncopy) {
#pragma clang fp contract(off)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const bool full = !SUMS && D != nullptr;  // as in lloyd_valu_fused_kernel
  const int sx = staged_row_stride(d);
  const int pad = sx - d;                                        // 0 or 1
  const int sxs = sums_stride(d);
  double *sums = reinterpret_cast<double *>(smem_raw);           // [ncopy][k][sxs]; SUMS false: none
  int *cnt = reinterpret_cast<int *>(sums + (SUMS ? (size_t)ncopy * k * sxs : 0));  // [k]
  T *ccs = reinterpret_cast<T *>(cnt + (SUMS ? k + (k & 1) : 0));          // [k]
  T *Xs = ccs + k + (k & 1);                                     // [WG][sx]
  typedef typename BlockLoad<T, VEC>::type ld_t;
  constexpr int NLD = (DMAX + VEC - 1) / VEC;
  const int tid = threadIdx.x;
  if (SUMS) {
    for (int e = tid; e < ncopy * k * sxs; e += WG) sums[e] = 0.0;
    for (int c = tid; c < k; c += WG) cnt[c] = 0;
  }
  const int nld = (d + VEC - 1) / VEC;  // loads per thread and block
  const int nvec = WG / VEC * d;        // vectors in a full block
  // el / d for el < 256 * 64 and d >= 2 as one multiply-high (exact while el * d < 2^32)
  const unsigned dinv = d > 1 ? 0xFFFFFFFFu / (unsigned)d + 1u : 0u;
  auto row_of = [&](int el) -> int { return d > 1 ? (int)__umulhi((unsigned)el, dinv) : el; };
  ld_t pre[NLD];
  T pre_xx = 0, pre_tail = 0;
  // Complete vectors of the block that starts at row `base`: all of them, except in the
  // last, partial block of the data set, whose final values may not fill a vector.
  auto block_vectors = [&](int64_t base) -> int {
    const int64_t left = n - base;
    return left >= WG ? nvec : (int)(left * d / VEC);
  };
  // Loads are never predicated per lane (indices are clamped instead), so the fetched
  // block stays in flight across the processing of the current one. The one exception
  // is the handful of values behind the last complete vector of the data set.
  auto fetch = [&](int64_t base) {
    const int vlim = block_vectors(base);  // >= 1: d >= VEC
    const T *xb = X + base * (int64_t)d;
    const ld_t *src = reinterpret_cast<const ld_t *>(xb);
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      const int e = tid + i * WG;
      if (i < nld) pre[i] = __builtin_nontemporal_load(&src[e < vlim ? e : vlim - 1]);
    }
    if (VEC > 1 && vlim < nvec) {
      const int64_t el = (int64_t)vlim * VEC + tid;
      if (tid < VEC && el < (n - base) * d) pre_tail = xb[el];
    }
    const int64_t r = base + tid;
    pre_xx = xnorm[r < n ? r : n - 1];
  };
  const int64_t stride = (int64_t)gridDim.x * WG;
  int64_t base = (int64_t)blockIdx.x * WG;
  if (base >= n) return;  // the grid never exceeds the number of blocks
  fetch(base);
  // centroid norms while the first block travels (visible after the barrier below)
  for (int c = tid; c < k; c += WG) ccs[c] = cnorm ? cnorm[c] : row_sqnorm<T>(C + (size_t)c * d, d);
  // entry c of the register set reads centroid min(c, k-1): in bounds, unused past k
  int coff[KREG];
#pragma unroll
  for (int c = 0; c < KREG; c++) coff[c] = (c < k ? c : k - 1) * d;
  const int jrot = (tid & 15) % d;  // sums_stride: the 16 lanes of a group add 16 consecutive features
  double *const my_sums = sums + (size_t)((tid >> 4) & (ncopy - 1)) * k * sxs;
  for (; base < n; base += stride) {
    const int rows = (int)min<int64_t>(WG, n - base);
    __syncthreads();  // the previous block has been consumed
    const int vlim = block_vectors(base);
    // Value el of the block lives at LDS offset el + (el / d) * pad. The offsets are
    // recomputed for every block from a copy of the thread index the optimiser cannot see
    // through: hoisted out of the loop they would occupy a register per staged value.
    int tv = tid;
    asm volatile("" : "+v"(tv));
    if (VEC == 1 || pad == 0 || d % VEC == 0) {  // no vector is split by padding slots
#pragma unroll
      for (int i = 0; i < NLD; i++) {
        const int e = tv + i * WG;
        if (i < nld && e < vlim) {
          const int el = e * VEC;
          const int off = el + row_of(el) * pad;
          if constexpr (VEC == 1) {
            Xs[off] = pre[i];
          } else {
#pragma unroll
            for (int q = 0; q < VEC; q++) Xs[off + q] = pre[i][q];
          }
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NLD; i++) {
        const int e = tv + i * WG;
        if (i < nld && e < vlim) {
          if constexpr (VEC > 1) {
            const int el = e * VEC;
            const int r = row_of(el);
            const int off = el + r * pad;
            const int inrow = (r + 1) * d - el;  // values of this vector in its first row
#pragma unroll
            for (int q = 0; q < VEC; q++) Xs[off + q + (q >= inrow ? pad : 0)] = pre[i][q];
          }
        }
      }
    }
    if (VEC > 1 && vlim < nvec) {  // values behind the last complete vector of the data set
      const int el = vlim * VEC + tid;
      if (tid < VEC && el < rows * d) Xs[el + row_of(el) * pad] = pre_tail;
    }
    const T xx = pre_xx;
    __syncthreads();
    fetch(base + stride < n ? base + stride : base);
    const int64_t row = base + tid;
    if (tid < rows) {
      const T *xrow = Xs + tid * sx;
      T dot[KREG];
#pragma unroll
      for (int c = 0; c < KREG; c++) dot[c] = 0;
      int j = 0;
      for (; j + 4 <= d; j += 4) {
        const T x0 = xrow[j], x1 = xrow[j + 1], x2 = xrow[j + 2], x3 = xrow[j + 3];
#pragma unroll
        for (int c = 0; c < KREG; c++) {
          const T *cp = C + coff[c] + j;
          dot[c] = dot[c] + x0 * cp[0];
          dot[c] = dot[c] + x1 * cp[1];
          dot[c] = dot[c] + x2 * cp[2];
          dot[c] = dot[c] + x3 * cp[3];
        }
      }
      for (; j < d; j++) {
        const T x0 = xrow[j];
#pragma unroll
        for (int c = 0; c < KREG; c++) dot[c] = dot[c] + x0 * C[coff[c] + j];
      }
      T best = argmin_start<T>();
      int bidx = -1;
#pragma unroll
      for (int c = 0; c < KREG; c++) {
        if (c < k) {
          const T t = xx + ccs[c];
          const T dist = fabs(t - (T)2 * dot[c]);
          if (full) D[(size_t)c * ldn + row] = dist;
          if (dist < best) {
            best = dist;
            bidx = c;
          }
        }
      }
      if (!full) {
        labels[row] = bidx;
        if (mindist) mindist[row] = best;
      }
      if (SUMS && bidx >= 0) {
        double *srow = my_sums + (size_t)bidx * sxs;
        int jj = jrot;  // rotated start, as in lloyd_valu_fused_kernel
        for (int q = 0; q < d; q++) {
          unsafeAtomicAdd(srow + jj, (double)xrow[jj]);
          jj = (jj + 1 == d) ? 0 : jj + 1;
        }
        atomicAdd(&cnt[bidx], 1);
      }
    }
  }
  if (!SUMS) return;
  __syncthreads();
  double *dst = psums + (size_t)blockIdx.x * k * d;
  for (int e = tid; e < k * d; e += WG) {
    const int c = e / d, jx = e - c * d;
    double v = sums[(size_t)c * sxs + jx];
    for (int cp = 1; cp < ncopy; cp++) v += sums[((size_t)cp * k + c) * sxs + jx];  // copy order
    dst[e] = v;
  }
  int *cdst = pcounts + (size_t)blockIdx.x * k;
  for (int c = tid; c < k; c += WG) cdst[c] = cnt[c];
}

// Three-input unsigned minimum as ONE instruction. Written as inline assembly
// because the optimiser otherwise re-associates a chain of them into pairs of
// two-input minima and spends 12 instead of 8 instructions on 16 keys.
__device__ __forceinline__ unsigned umin3(unsigned a, unsigned b, unsigned c) {
  unsigned r;
  asm("v_min3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// centroid row of accumulator v (runtime v) of the 32x32 float tile
__device__ __forceinline__ int key_row(unsigned v, int g) {
  return (int)((v >> 2) * 8 + (unsigned)g * 4 + (v & 3));
}

// float32 products on the bfloat16 matrix pipe. A float is the exact sum of three
// bfloat16 values (8 significant bits each: the float rounded to bfloat16, the remainder
// rounded to bfloat16, and what is left of it, which has at most 8 significant bits; every
// subtraction is exact), so x * c is the exact sum of the nine products of their parts, each
// of which a float holds exactly (16 bits). v_mfma_f32_32x32x16_bf16 adds such products
// into float accumulators: the result carries float rounding of the running sum only, as
// the float32 instruction's does. On gfx950 the instruction runs at 16 times the float32
// rate (nine of them per 16 features take 288 cycles where eight v_mfma_f32_32x32x2_f32
// take 512). The parts are rounded to nearest (v_cvt_pk_bf16_f32), not cut off: the
// remainders then carry either sign, and the products the 6-product form leaves out cancel
// on average instead of adding up to a bias of the distances (cut-off parts all have the
// sign of the float they come from; measured on 6000 x 200 blobs far from the origin, the
// sum of the minimum distances came out 1.6e-5 too large).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
// two floats rounded to bfloat16 in one register: a in bits 0-15, b in bits 16-31
__device__ __forceinline__ unsigned cvt_pk_bf16(float a, float b) {
  const floatx2 f = {a, b};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
}
// The three parts of two floats, each pair packed like cvt_pk_bf16 packs it: 11 vector
// instructions (three conversions, four unpackings, four subtractions).
struct Bf16x3Pair {
  unsigned h, m, l;
};
__device__ __forceinline__ Bf16x3Pair split_pair_bf16x3(float a, float b) {
  Bf16x3Pair p;
  p.h = cvt_pk_bf16(a, b);
  const float ra = a - __uint_as_float(p.h << 16), rb = b - __uint_as_float(p.h & 0xFFFF0000u);
  p.m = cvt_pk_bf16(ra, rb);
  p.l = cvt_pk_bf16(ra - __uint_as_float(p.m << 16), rb - __uint_as_float(p.m & 0xFFFF0000u));
  return p;
}
__device__ __forceinline__ floatx16 mma_bf16(uintx4 a, uintx4 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// ---------------------------------------------------------------------------
// MFMA row-stationary variant (d <= DP, all centroids resident in LDS).
//
// A workgroup is persistent: it stages -2*C once into LDS, already permuted
// into A-operand order so that every later read is one conflict-free 16-byte
// load per lane, then walks over row tiles. Each wavefront keeps ROWT tiles of
// MT data rows in registers (plain 16-byte global loads, never through LDS)
// and sweeps all centroid tiles over them: accumulators start at xx + cc, the
// matrix core adds -2 x.c, and the epilogue folds |acc| into a per-lane running
// (min, index). Lane groups holding different centroid subsets of the same row
// are merged with one (f32) or two (f64) cross-lane exchanges per row tile.
// ---------------------------------------------------------------------------
//
// FUSE: the workgroup also keeps per-centroid sums and counts of the rows it
// labels in LDS (row stride DP+1 words so that different centroids start on
// different banks) and writes them to its own slot psums[blockIdx.x][k][d],
// pcounts[blockIdx.x][k] when it has walked all its row tiles: the centroid
// update then needs no second pass over the data.
// LOAD: how a lane fetches its feature slice of a data row. 1: d == DP and 16-byte aligned
// data: 16-byte loads of the slice as it lies in memory. 2: any d >= the vector width, data
// aligned to its elements: 16-byte loads that stay inside the row (padded features are
// zero, or finite values meeting zeros on the centroid side).
// 0: d below the vector width: scalar loads, zero padded.
// SPLIT (float32 only; 0, 6 or 9): the dot products run on the bfloat16 matrix pipe as that
// many products of bfloat16 parts per feature pair (see split_pair_bf16x3). 9: every product
// exact. 6: the three smallest (below 2^-24 of |x||c|) left out. The centroid parts are
// staged in LDS in operand order, [tile][16-feature step][part][lane] 16 bytes each; the
// data rows are split in registers once per row tile.
template <typename T, int DP, int ROWT, int LOAD, bool FUSE, int NW, bool EXACT = false, int SPLIT = 0>
__global__ __launch_bounds__(NW * 64) void assign_rowstat_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm,
    const T *__restrict__ C, const T *__restrict__ cnorm,
    int *__restrict__ labels, T *__restrict__ mindist, int64_t n, int d, int k,
    int kp, double *__restrict__ psums, int *__restrict__ pcounts, int c_off, int merge,
    int sets, int kps, int kset) {
  constexpr int TPB = NW * 64;
  typedef Mfma<T> M;
  constexpr int MT = M::MT, KL = M::KL, NACC = M::NACC, VW = M::VW;
  constexpr int DCH = DP / KL;  // features per lane group
  constexpr int NV = DCH / VW;  // 16-byte vectors per lane per tile
  static_assert(DCH % VW == 0, "DP must be a multiple of KL*VW");
  typedef typename M::acc_t acc_t;
  typedef typename M::vec_t vec_t;
  constexpr bool VECLOAD = LOAD == 1;
  // float32 argmin on integer keys (16-ulp resolution) unless the exact compare chain is asked for
  constexpr bool KEYS = sizeof(T) == 4 && !EXACT;
  static_assert(SPLIT == 0 || (sizeof(T) == 4 && NV % 2 == 0 && LOAD != 0 && (SPLIT == 6 || SPLIT == 9)),
                "bfloat16 parts: float32, whole 16-feature steps, vector loads");
  constexpr int NS = NV / 2;  // (SPLIT) 16-feature steps: two of a lane's vectors each

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *Cs = reinterpret_cast<T *>(smem_raw);  // [KT][NV][64][VW], see cs_slot
  // (SPLIT: [KT][NS][3][64] vectors of 8 bfloat16, 6 bytes per element instead of 4)
  T *ccs = SPLIT ? reinterpret_cast<T *>(smem_raw + (size_t)kp * DP * 6) : Cs + (size_t)kp * DP;  // [kp]
  constexpr int SD = DP + 1;
  // (FUSE) sums in double: ds_add_f64 is the fast LDS floating-point atomic on gfx950
  double *sums = reinterpret_cast<double *>(ccs + kp + (kp & 1));  // [k][SD], 8-byte aligned
  int *cnt = reinterpret_cast<int *>(sums + (size_t)k * SD);       // [k]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane % MT;
  const int g = lane / MT;
  const int KT = kp / MT;
  // Feature j lies in 16-byte vector j / VW of its row, and the vectors are dealt to the
  // KL lane groups in turn: vector v belongs to lane group v % KL and is that group's
  // step v / KL. A row of d < DP features thus fills the first nq steps of every lane
  // group; the steps after them hold nothing and are skipped, matrix work included.
  const int nq = LOAD == 1 ? NV : ((d + VW - 1) / VW + KL - 1) / KL;
  auto cs_slot = [&](int c, int j) -> size_t {  // place of centroid c, feature j in Cs
    const int t = c / MT, i = c - t * MT, v = j / VW;
    return ((size_t)(t * NV + v / KL) * 64 + (v % KL) * MT + i) * VW + (j - v * VW);
  };

  if (FUSE) {
    for (int e = tid; e < k * SD; e += TPB) sums[e] = 0.0;
    for (int c = tid; c < k; c += TPB) cnt[c] = 0;
  }

  if constexpr (SPLIT != 0) {
    // one (centroid, step, lane group) per thread and turn: its 8 features, times -2
    // (exact), split into three parts and stored as the lane's operand of that step
    for (int e = tid; e < kp * NS * KL; e += TPB) {
      const int c = e / (NS * KL), rem = e - c * (NS * KL), st = rem / KL, gg = rem - st * KL;
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int f = ((2 * st + j / VW) * KL + gg) * VW + j % VW;
        v[j] = (c < k && f < d) ? -2.0f * (float)C[(size_t)c * d + f] : 0.0f;
      }
      uintx4 ph, pm, pl;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const Bf16x3Pair pr = split_pair_bf16x3(v[2 * w], v[2 * w + 1]);
        ph[w] = pr.h;
        pm[w] = pr.m;
        pl[w] = pr.l;
      }
      const int t = c / MT, i = c - t * MT;
      uintx4 *dst = reinterpret_cast<uintx4 *>(smem_raw) + (size_t)((t * NS + st) * 3) * 64 + gg * MT + i;
      dst[0] = ph;
      dst[64] = pm;
      dst[128] = pl;
    }
  } else if (VECLOAD) {
    // d == DP: 16-byte loads, four in flight per thread, one 16-byte LDS store each
    constexpr int VPR = DP / VW;  // vectors per centroid row
    const int nvec = k * VPR;
    constexpr int U = 4;
    for (int e0 = tid; e0 < nvec; e0 += U * TPB) {
      vec_t v[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int e = min(e0 + u * TPB, nvec - 1);
        v[u] = reinterpret_cast<const vec_t *>(C)[e];
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int e = e0 + u * TPB;
        if (e < nvec) {
          const int c = e / VPR, j = (e - c * VPR) * VW;
          reinterpret_cast<vec_t *>(Cs)[cs_slot(c, j) / VW] = v[u] * (T)-2;
        }
      }
    }
    // centroid rows k .. kp-1 of the last tile: zeros
    for (int e = k * VPR + tid; e < kp * VPR; e += TPB) {
      const int c = e / VPR, j = (e - c * VPR) * VW;
      vec_t z;
#pragma unroll
      for (int q = 0; q < VW; q++) z[q] = 0;
      reinterpret_cast<vec_t *>(Cs)[cs_slot(c, j) / VW] = z;
    }
  } else {
    for (int e = tid; e < kp * DP; e += TPB) {
      const int c = e / DP, j = e - c * DP;
      const T v = (c < k && j < d) ? (T)-2 * C[(size_t)c * d + j] : (T)0;
      Cs[cs_slot(c, j)] = v;
    }
  }
  // Stacked model (sets > 1): `sets` independent centroid sets laid end to end, each padded
  // to kps rows (a multiple of the tile height) of which the first kset are centroids; a
  // padding row's norm is +inf, so it can never win. One set: kps = kp, kset = k.
  for (int c = tid; c < kp; c += TPB)
    ccs[c] = (c < k && (c % kps) < kset && cnorm) ? cnorm[c] : pos_inf<T>();
  __syncthreads();
  if (cnorm == nullptr) {
    // No norm buffer given: take the norms from the staged centroids. A staged value is
    // -2c; halving it is exact, so the sum below (j ascending, multiply and add rounded
    // separately) is bit for bit what row_norms / post_update would have stored.
#pragma clang fp contract(off)
    for (int c = tid; c < k; c += TPB) {
      if ((c % kps) >= kset) continue;
      T acc = 0;
      for (int j = 0; j < d; j++) {
        const T v = SPLIT ? C[(size_t)c * d + j] : (T)-0.5 * Cs[cs_slot(c, j)];
        acc = acc + v * v;
      }
      ccs[c] = acc;
    }
    __syncthreads();
  }

  constexpr int ROWS_PER_WAVE = ROWT * MT;
  // The rows of the next tile are fetched while the current tile is swept, so
  // the only exposed memory latency is that of the first tile.
  T xn[ROWT][DCH];
  T xxn[ROWT];
  T pmn[ROWT];
  int pln[ROWT];
#pragma unroll
  for (int rt = 0; rt < ROWT; rt++) {
    pmn[rt] = 0;
    pln[rt] = -1;
  }
  auto fetch_rows = [&](int64_t wrow0) {
#pragma unroll
    for (int rt = 0; rt < ROWT; rt++) {
      // rows past the end re-read the last row; their results are never stored
      const int64_t row = min(wrow0 + rt * MT + r, n - 1);
      if (VECLOAD) {
        const vec_t *src = reinterpret_cast<const vec_t *>(X + row * (int64_t)DP);
#pragma unroll
        for (int q = 0; q < NV; q++) {
          vec_t v = src[q * KL + g];
#pragma unroll
          for (int e = 0; e < VW; e++) xn[rt][q * VW + e] = v[e];
        }
      } else if (LOAD == 2) {
        const T *src = X + row * (int64_t)d;
#pragma unroll
        for (int q = 0; q < NV; q++) {
          // (steps from nq on are never used, but their loads are issued all the same,
          // clamped into the row: a branch here would make every load wait for the last)
          const int f0 = (q * KL + g) * VW;
          vec_t v;
          if (d % VW == 0) {
            // no vector straddles the end of the row: one that lies past it re-reads the
            // row's last vector (finite x * 0 from the zero-padded centroid side adds
            // nothing, and the padded columns of the fused sums are never written back)
            const typename M::uvec_t u = *reinterpret_cast<const typename M::uvec_t *>(src + min(f0, d - VW));
#pragma unroll
            for (int e = 0; e < VW; e++) v[e] = u[e];
          } else {
            v = load_row_vector<T>(src, f0, d);
          }
#pragma unroll
          for (int e = 0; e < VW; e++) xn[rt][q * VW + e] = v[e];
        }
      } else {
        const T *src = X + row * (int64_t)d;
#pragma unroll
        for (int s = 0; s < DCH; s++) {
          const int j = ((s / VW) * KL + g) * VW + s % VW;
          xn[rt][s] = j < d ? src[j] : (T)0;
        }
      }
      xxn[rt] = xnorm[row];
      if (!FUSE && merge) {  // the row's result from the earlier chunks travels with the prefetch
        pmn[rt] = mindist[row];
        pln[rt] = labels[row];
      }
    }
  };
  // Row tiles of ROWS_PER_WAVE rows are dealt out one per workgroup before the next
  // wavefront slot gets any: wavefront w of workgroup b takes tiles w*G + b, then every
  // G*NW-th after it. In the last, partial round the remaining tiles thus spread over all
  // CUs and SIMDs instead of filling the first few workgroups, whose four wavefronts per
  // SIMD would share one matrix pipe while the rest of the chip idles.
  const int64_t tile_stride = (int64_t)gridDim.x * NW;
  const int64_t row_stride = tile_stride * ROWS_PER_WAVE;
  const int64_t wrow_first = ((int64_t)wave * gridDim.x + blockIdx.x) * ROWS_PER_WAVE;
  if (wrow_first < n) fetch_rows(wrow_first);
  for (int64_t wrow0 = wrow_first; wrow0 < n; wrow0 += row_stride) {
    T x[ROWT][DCH];
    T xx[ROWT];
    T pm[ROWT];
    int pl[ROWT];
#pragma unroll
    for (int rt = 0; rt < ROWT; rt++) {
#pragma unroll
      for (int s = 0; s < DCH; s++) x[rt][s] = xn[rt][s];
      xx[rt] = xxn[rt];
      pm[rt] = pmn[rt];
      pl[rt] = pln[rt];
    }
    if (wrow0 + row_stride < n) fetch_rows(wrow0 + row_stride);
    // (SPLIT) the row tile's three bfloat16 parts, packed in operand order
    uintx4 xh[SPLIT ? ROWT : 1][SPLIT ? NS : 1], xm[SPLIT ? ROWT : 1][SPLIT ? NS : 1],
        xl[SPLIT ? ROWT : 1][SPLIT ? NS : 1];
    if constexpr (SPLIT != 0) {
#pragma unroll
      for (int rt = 0; rt < ROWT; rt++) {
#pragma unroll
        for (int st = 0; st < NS; st++) {
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const Bf16x3Pair pr =
                split_pair_bf16x3((float)x[rt][2 * st * VW + 2 * w], (float)x[rt][2 * st * VW + 2 * w + 1]);
            xh[rt][st][w] = pr.h;
            xm[rt][st][w] = pr.m;
            xl[rt][st][w] = pr.l;
          }
        }
      }
    }
    T best[ROWT];
    int bidx[ROWT];
    unsigned bkey[ROWT];  // float32 path: running minimum key and its tile
    int btile[ROWT];
    auto tile_mma = [&](acc_t (&acc)[ROWT], int t) {
#pragma unroll
      for (int v = 0; v < NACC; v++) {
        const T cc = ccs[t * MT + M::acc_row(v, g)];
#pragma unroll
        for (int rt = 0; rt < ROWT; rt++) acc[rt][v] = xx[rt] + cc;
      }
      if constexpr (SPLIT != 0) {
        const uintx4 *ap = reinterpret_cast<const uintx4 *>(smem_raw) + (size_t)t * NS * 3 * 64 + lane;
#pragma unroll
        for (int st = 0; st < NS; st++) {
          if (LOAD == 1 || 2 * st < nq) {
            const uintx4 ah = ap[(st * 3 + 0) * 64], am = ap[(st * 3 + 1) * 64], al = ap[(st * 3 + 2) * 64];
            // smallest products first
#pragma unroll
            for (int rt = 0; rt < ROWT; rt++) {
              if constexpr (SPLIT == 9) {
                acc[rt] = mma_bf16(al, xl[rt][st], acc[rt]);
                acc[rt] = mma_bf16(al, xm[rt][st], acc[rt]);
                acc[rt] = mma_bf16(am, xl[rt][st], acc[rt]);
              }
              acc[rt] = mma_bf16(al, xh[rt][st], acc[rt]);
              acc[rt] = mma_bf16(ah, xl[rt][st], acc[rt]);
              acc[rt] = mma_bf16(am, xm[rt][st], acc[rt]);
              acc[rt] = mma_bf16(am, xh[rt][st], acc[rt]);
              acc[rt] = mma_bf16(ah, xm[rt][st], acc[rt]);
              acc[rt] = mma_bf16(ah, xh[rt][st], acc[rt]);
            }
          }
        }
        return;
      }
      const vec_t *ap = reinterpret_cast<const vec_t *>(Cs) + (size_t)t * NV * 64 + lane;
#pragma unroll
      for (int q = 0; q < NV; q++) {
        if (LOAD == 1 || q < nq) {  // (no early exit: the loop must unroll, x lives in registers)
          const vec_t a = ap[q * 64];
#pragma unroll
          for (int e = 0; e < VW; e++) {
#pragma unroll
            for (int rt = 0; rt < ROWT; rt++)
              acc[rt] = M::mma(a[e], x[rt][q * VW + e], acc[rt]);
          }
        }
      }
    };
    auto tile_argmin = [&](const acc_t (&acc)[ROWT], int t) {
      if constexpr (KEYS) {
        // float32 MFMA shares the SIMD's FP32 datapath with ordinary vector
        // instructions, so every epilogue instruction costs matrix time. The
        // argmin is therefore done on integer keys: |acc| with its four lowest
        // mantissa bits replaced by the accumulator number v. Keys of one tile are
        // reduced with 3-input unsigned minima (positive floats order like
        // unsigned integers), the winner is compared once per tile with the
        // running key. Distances are thus compared at a resolution of 16 ulp
        // (1.9e-6 relative); within one 16-ulp bucket the lowest centroid index wins:
        // inside a tile through the index bits, across tiles because a later tile must
        // be below the running key's bucket (index bits ignored) to replace it.
#pragma unroll
        for (int rt = 0; rt < ROWT; rt++) {
          unsigned key[NACC];
#pragma unroll
          for (int v = 0; v < NACC; v++)
            key[v] = (__float_as_uint(acc[rt][v]) & 0x7FFFFFF0u) | (unsigned)v;
          unsigned m = umin3(key[0], key[1], key[2]);
#pragma unroll
          for (int v = 3; v + 1 < NACC; v += 2) m = umin3(m, key[v], key[v + 1]);
          if ((NACC & 1) == 0) m = min(m, key[NACC - 1]);
          if ((m | 15u) < bkey[rt]) {
            bkey[rt] = m;
            btile[rt] = t;
          }
        }
      } else {
        // the compare chain: the running best keeps the accumulator's sign (magnitudes are
        // compared through operand modifiers), the winner is remembered as its accumulator
        // number, and the tile is noted once per tile
        int loc[ROWT];
#pragma unroll
        for (int rt = 0; rt < ROWT; rt++) loc[rt] = -1;
#pragma unroll
        for (int v = 0; v < NACC; v++) {
#pragma unroll
          for (int rt = 0; rt < ROWT; rt++) {
            const T a = acc[rt][v];
            if (fabs(a) < fabs(best[rt])) {
              best[rt] = a;
              loc[rt] = v;
            }
          }
        }
#pragma unroll
        for (int rt = 0; rt < ROWT; rt++) {
          if (loc[rt] >= 0) {
            btile[rt] = t;
            bidx[rt] = loc[rt];
          }
        }
      }
    };
    // (Software-pipelining tile t's matrix work against tile t-1's argmin with a second
    // accumulator set measured no faster: the two do not overlap on this hardware, and
    // the extra registers cost occupancy.)
    const int tps = KT / sets;  // tiles per centroid set
    for (int set = 0; set < sets; set++) {
#pragma unroll
      for (int rt = 0; rt < ROWT; rt++) {
        best[rt] = argmin_start<T>();
        bidx[rt] = -1;
        bkey[rt] = 0x7F7FFFF0u;  // FLT_MAX with the index bits cleared
        btile[rt] = -1;
      }
      // The sweep over the centroid tiles at the highest wave priority, everything around it
      // (next rows, labels, the sums in LDS) at the lowest: a wavefront in its sweep is then
      // served before one that is between sweeps (10M x 32, k = 256: 1.391 -> 1.357 ms per fused
      // step, 1M x 64, k = 64: 0.115 -> 0.105 ms, double 10M x 32: 2.743 -> 2.704 ms; priority 1
      // gave two thirds of that, raising it around the matrix instructions only a third).
      __builtin_amdgcn_s_setprio(3);
      for (int t = set * tps; t < (set + 1) * tps; t++) {
        acc_t acc[ROWT];
        tile_mma(acc, t);
        tile_argmin(acc, t);
      }
      __builtin_amdgcn_s_setprio(0);
      if constexpr (KEYS) {
#pragma unroll
        for (int rt = 0; rt < ROWT; rt++) {
          best[rt] = __uint_as_float(bkey[rt] & 0xFFFFFFF0u);
          bidx[rt] = btile[rt] < 0 ? -1 : btile[rt] * MT + key_row(bkey[rt] & 15u, g);
        }
      } else {
#pragma unroll
        for (int rt = 0; rt < ROWT; rt++) {
          best[rt] = fabs(best[rt]);
          if (btile[rt] >= 0) bidx[rt] = btile[rt] * MT + M::acc_row(bidx[rt], g);
        }
      }
#pragma unroll
      for (int rt = 0; rt < ROWT; rt++) {
#pragma unroll
        for (int off = MT; off < 64; off <<= 1) {
          const T ob = __shfl_xor(best[rt], off, 64);
          const int oi = __shfl_xor(bidx[rt], off, 64);
          argmin_merge(best[rt], bidx[rt], ob, oi);
        }
        const int64_t row = wrow0 + rt * MT + r;
        if (g == 0 && row < n) {
          // A model too large for LDS is swept in chunks of centroids, one launch each:
          // C and cnorm then point at the chunk, c_off is its first centroid, and from the
          // second chunk on (merge) the row's result so far is read back and kept unless
          // this chunk is strictly closer (earlier chunks hold the lower indices).
          // (a set's labels count from its own first centroid and go to its own [n] block)
          T bv = best[rt];
          int bi = bidx[rt] < 0 ? -1 : bidx[rt] + c_off - set * kps;
          if (!FUSE && merge) argmin_merge(bv, bi, pm[rt], pl[rt]);  // (a fused step is never chunked)
          labels[(int64_t)set * n + row] = bi;
          if (mindist) mindist[(int64_t)set * n + row] = bv;
        }
        if (FUSE && row < n && bidx[rt] >= 0) {
          double *srow = sums + (size_t)bidx[rt] * SD;
#pragma unroll
          for (int q = 0; q < NV; q++) {
            if (LOAD == 1 || q < nq) {
#pragma unroll
              for (int e = 0; e < VW; e++) {
                const int f = (q * KL + g) * VW + e;  // the feature this register holds
                if (LOAD == 1 || f < d) unsafeAtomicAdd(srow + f, (double)x[rt][q * VW + e]);
              }
            }
          }
          if (g == 0) atomicAdd(&cnt[bidx[rt]], 1);
        }
      }
    }  // centroid sets
  }
  if (FUSE) {
    __syncthreads();
    double *dst = psums + (size_t)blockIdx.x * k * d;
    for (int e = tid; e < k * d; e += TPB) {
      const int c = e / d, j = e - c * d;
      dst[e] = sums[(size_t)c * SD + j];
    }
    int *cdst = pcounts + (size_t)blockIdx.x * k;
    for (int c = tid; c < k; c += TPB) cdst[c] = cnt[c];
  }
}

// ---------------------------------------------------------------------------
// MFMA tiled variant (any d, any k). A workgroup owns BR = 128 data rows and
// walks over centroid blocks of BC = 128; for each block it runs the d-loop in
// steps of BK features with both operand tiles staged through LDS in operand
// order (double buffered, next stage's global loads in flight during the
// current stage's matrix work). The four wavefronts split the block 2 x 2, each
// holding (BC/2/MT) x (BR/2/MT) result tiles in accumulators.
// MODE 0: running argmin kept in registers across centroid blocks, halves
// merged through LDS at the end.  MODE 1: one centroid block per workgroup, the
// distances stored to D[c*ldn + i].
//
// Preconditions (the engine's buffers satisfy them): C holds round_up(k, BC)
// rows and cnorm round_up(k, BC) entries, the entries past k being +inf, so the
// loads need no bounds test on the centroid axis; rows past n re-read row n-1.
// A feature tail (d not a multiple of BK, DTAIL) is zero on the centroid side (on both
// sides when d is not a multiple of the vector width); its loads stay inside the operand
// row (VECLOAD: 16-byte loads for any d >= the vector width, rows aligned to their
// elements only).
// ---------------------------------------------------------------------------
// BCW = wavefronts along the centroid axis (2 or 4): the workgroup has 2*BCW
// wavefronts and covers 64*BCW centroids. Data-row blocks are private to a
// workgroup and come from HBM/MALL every time they are re-read, centroid blocks
// are shared by all workgroups and hit L2, so for large k the wider centroid
// block (BCW = 4) halves the expensive traffic.
// The centroids' bfloat16 parts for the tiled kernel, written as the LDS images it stages:
// for centroid block cb (bc centroids) and stage st (16 features) a block of bc*16*6 bytes,
// [32-centroid tile][part][lane group * 32 + centroid] vectors of 8 bfloat16, the lane
// group's features in the order the row side deals them out (16-byte vectors of the stage in
// turn: vector 0 and 2 to lane group 0, 1 and 3 to lane group 1). Rows past k and features
// past d are zero, so the tiled kernel needs no bounds on this operand.
__global__ void split_centroids_kernel(const float *__restrict__ C, uintx4 *__restrict__ out, int k,
                                       int d, int bc, int nstage, int nblocks) {
  const int tiles = bc / 32;
  const int64_t total = (int64_t)nblocks * nstage * tiles * 64;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int slot = (int)(e & 63);
    int64_t rest = e >> 6;
    const int t = (int)(rest % tiles);
    rest /= tiles;
    const int st = (int)(rest % nstage);
    const int cb = (int)(rest / nstage);
    const int gg = slot >> 5, i = slot & 31;
    const int c = cb * bc + t * 32 + i;
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int f = st * 16 + ((j >> 2) * 2 + gg) * 4 + (j & 3);
      v[j] = (c < k && f < d) ? C[(size_t)c * d + f] : 0.0f;
    }
    uintx4 ph, pm, pl;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      const Bf16x3Pair pr = split_pair_bf16x3(v[2 * w], v[2 * w + 1]);
      ph[w] = pr.h;
      pm[w] = pr.m;
      pl[w] = pr.l;
    }
    uintx4 *dst = out + (((size_t)cb * nstage + st) * tiles + t) * 3 * 64 + slot;
    dst[0] = ph;
    dst[64] = pm;
    dst[128] = pl;
  }
}

template <typename T, int BCW, bool WIDE = false, int SPLIT = 0>
struct TiledCfg {
  static constexpr int TPB = 2 * BCW * 64;
  // WIDE: every wavefront holds twice as many centroid tiles (a 256-centroid block for four
  // wavefronts) at half the stage depth: the same matrix work per stage and barrier, half as
  // many passes over the workgroup's row slice.
  static constexpr int BC = 64 * BCW * (WIDE ? 2 : 1);
  // 128 rows for both precisions: with 64 rows the double kernel issued only 32 MFMAs per
  // staged tile pair and its staging instructions weighed twice as much (2M x 256, k = 1024
  // double: 0.75 -> 0.81 of peak with 128 rows, a few spilled registers included)
  static constexpr int BR = 128;
  // features per stage. The 64-centroid form serves bandwidth-bound shapes (k <= 64): half
  // the stage depth halves its LDS image, so twice as many workgroups keep loads in flight
  // (500k x 784, k = 10: 0.62 -> 0.49 ms; a quarter of the depth was slower again).
  // SPLIT (float32 dot products as products of bfloat16 parts, see split_pair_bf16x3): a stage is
  // one 16-feature step of the bfloat16 instruction; its three parts per element take 6 bytes
  // of LDS where the float takes 4.
  static constexpr int BK = SPLIT ? 16 : (sizeof(T) == 4 ? 32 : 16) / (BCW == 1 || WIDE ? 2 : 1);
  static constexpr size_t OPERAND_BYTES = (size_t)2 * (BC + BR) * BK * (SPLIT ? 6 : sizeof(T));
  // two copies of a block's centroid norms behind the operand stages
  static constexpr size_t LDS_BYTES = OPERAND_BYTES + (size_t)2 * BC * sizeof(T);
};

template <typename T, int MODE, bool VECLOAD, bool DTAIL, int BCW, bool EXACT = false, bool WIDE = false,
          int SPLIT = 0>
__global__ __launch_bounds__(2 * BCW * 64, BCW == 4 ? 1 : 2) void assign_tiled_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm,
    const T *__restrict__ C, const T *__restrict__ cnorm,
    int *__restrict__ labels, T *__restrict__ mindist, T *__restrict__ D,
    int64_t n, int64_t ldn, int d, int k, const uintx4 *__restrict__ Cparts) {
  typedef Mfma<T> M;
  typedef TiledCfg<T, BCW, WIDE, SPLIT> Cfg;
  static_assert(SPLIT == 0 || (sizeof(T) == 4 && VECLOAD && (SPLIT == 6 || SPLIT == 9)),
                "bfloat16 parts: float32 rows fetched as vectors");
  constexpr int MT = M::MT, KL = M::KL, NACC = M::NACC, VW = M::VW;
  constexpr int BC = Cfg::BC, BR = Cfg::BR, BK = Cfg::BK, WG = Cfg::TPB;
  constexpr int DCH = BK / KL;       // features per lane group per stage
  constexpr int NV = DCH / VW;       // 16-byte vectors per lane per tile per stage
  constexpr int CT = BC / BCW / MT;  // centroid tiles per wavefront
  constexpr int RT = BR / 2 / MT;    // row tiles per wavefront
  constexpr int TILE_ELEMS = MT * BK;               // one operand tile, one stage
  constexpr int A_ELEMS = (BC / MT) * TILE_ELEMS;   // = BC*BK
  constexpr int B_ELEMS = (BR / MT) * TILE_ELEMS;
  constexpr int VEC_PER_ROW = BK / VW;              // 16-byte vectors per operand row per stage
  constexpr int ROWS_PER_PASS = WG / VEC_PER_ROW;   // operand rows one pass of the workgroup covers
  constexpr int A_VECS = BC / ROWS_PER_PASS;        // vectors each thread stages for A
  constexpr int B_VECS = BR / ROWS_PER_PASS;
  typedef typename M::acc_t acc_t;
  typedef typename M::vec_t vec_t;
  typedef typename M::uvec_t uvec_t;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *As = reinterpret_cast<T *>(smem_raw);  // [2][A_ELEMS]
  T *Bs = As + 2 * A_ELEMS;                 // [2][B_ELEMS]
  // after the main loop the same memory is reused for the cross-wave merge
  // SPLIT: [2][tile][16-feature step][part][64 lanes] vectors of 8 bfloat16 for either operand
  constexpr int NSB = SPLIT ? NV / 2 : 1;  // 16-feature steps per stage
  constexpr int A_BYTES = BC * BK * 6, B_BYTES = BR * BK * 6;
  unsigned char *Ab = smem_raw, *Bb = smem_raw + 2 * A_BYTES;
  // The accumulators start at zero and -(xx + cc)/2 is added when a block is complete, as in
  // assign_tiled_dma_kernel and for its reason (the partial sums of the dot product are then
  // rounded at their own size: 1.5 times less rounding noise in the minimum distance at 256
  // float32 features); the two kernels add the same products in the same order and close a
  // block with the same expression, so a shape gives the same bits through either, whatever
  // its alignment or the tiled_direct option. The block's norms wait in LDS for the epilogue.
  T *cns = reinterpret_cast<T *>(smem_raw + Cfg::OPERAND_BYTES);  // [2][BC]
  static_assert(BC <= WG, "one thread per centroid of a block fetches its norm");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wc = wave % BCW;  // which part of the centroid block
  const int wr = wave / BCW;  // which half of the row block
  const int r = lane % MT;
  const int g = lane / MT;
  // MODE 0: one workgroup per row block. MODE 1: one per (row block, centroid block) pair
  // on a linear grid with the centroid block running fastest: workgroups that are resident
  // together then share a handful of row blocks (which stay in L2) instead of all reading
  // different ones (500k x 784, k = 4096, 100,000 rows: 5.94 -> 5.64 ms against the row
  // block running fastest; L2-sized patches of both measured the same as this order).
  const int ncb = MODE == 1 ? (k + BC - 1) / BC : 1;
  const int64_t rt_id = MODE == 1 ? (int64_t)blockIdx.x / ncb : (int64_t)blockIdx.x;
  const int cb_id = MODE == 1 ? (int)((int64_t)blockIdx.x - rt_id * ncb) : 0;
  const int64_t row0 = rt_id * BR;
  const int nstage = (d + BK - 1) / BK;
  // A stage is NV steps of KL vectors (KL * VW features). Where d is not a whole number of
  // stages (DTAIL) the d-steps are dealt evenly over the stages, the first `srem` stages one
  // step longer than the rest, instead of leaving a short last stage: staging a stage costs
  // the same whatever it holds, and a stage with a full share of matrix instructions hides
  // more of it. Measured against whole stages and a short last one, same box, alternating
  // runs: float32 3M x 100, k = 1000 (4, 4, 4, 1 -> 4, 3, 3, 3 steps) 5.77 -> 5.70 ms, 261k x
  // 298, k = 1000 1.528 -> 1.507 ms, 200k x 780, k = 4096 11.47 -> 11.32 ms; with one test per
  // step (`q >= nq_st`) for every stage instead of a second one for "last stage" the double
  // kernels gained more than the dealing explains (1M x 100, k = 1000 4.05 -> 3.69 ms, 500k x
  // 250, k = 1024 4.54 -> 4.24 ms, the same steps per stage before and after). The
  // bfloat16-parts kernels keep whole stages: theirs is a single step.
  constexpr int SF = KL * VW;
  constexpr bool EVEN = DTAIL && SPLIT == 0;
  const int nsteps = (d + SF - 1) / SF;
  const int sbase = EVEN ? nsteps / nstage : NV;
  const int srem = EVEN ? nsteps - sbase * nstage : 0;
  auto stage_off = [&](int st) { return EVEN ? SF * (st * sbase + min(st, srem)) : st * BK; };
  // steps of stage st that hold features
  auto stage_nq = [&](int st) {
    if (EVEN) return sbase + (st < srem ? 1 : 0);
    // whole stages, the last one ceil(rest / VW) vectors, KL per step
    return st + 1 < nstage ? NV : ((d - (nstage - 1) * BK + VW - 1) / VW + KL - 1) / KL;
  };

  // staging role of this thread: operand row rr0 + q*ROWS_PER_PASS, features
  // [jj, jj+VW) of the stage. The 16-byte vector lands in LDS at tile rr/MT,
  // lane group jj/DCH, slot jj%DCH (operand order).
  const int rr0 = tid / VEC_PER_ROW;
  const int jj = (tid - rr0 * VEC_PER_ROW) * VW;
  int lds_off[A_VECS > B_VECS ? A_VECS : B_VECS];
#pragma unroll
  for (int q = 0; q < (A_VECS > B_VECS ? A_VECS : B_VECS); q++) {
    const int rr = rr0 + q * ROWS_PER_PASS;
    // the stage's 16-byte vectors are dealt to the KL lane groups in turn (vector v:
    // lane group v % KL, step v / KL), so a short last stage fills the first steps of
    // every lane group and the steps after them can be skipped
    const int t = rr / MT, i = rr - t * MT, gg = (jj / VW) % KL, s = (jj / VW) / KL * VW;
    // The 8 threads that stage one operand row write 8 different (vector, lane group)
    // combinations; unswizzled they land 1 KB apart, i.e. on the same banks. XOR-ing the
    // combination number into the low 3 bits of the lane slot spreads them over all
    // banks; a reader of vector q applies the same XOR, and since it reads all 64 slots
    // of the vector its access stays a conflict-free permutation.
    const int slot = (gg * MT + i) ^ (((s / VW) * KL + gg) & 7);
    lds_off[q] = ((t * NV + s / VW) * 64 + slot) * VW;
    if constexpr (SPLIT != 0) {
      // byte offset of the high part: lane group step sf = s / VW is half sf % 2 of the
      // 16-feature step sf / 2; the middle and low parts follow 1 KB and 2 KB behind. (The 64
      // threads of a wavefront write 16 consecutive lane slots of 2 lane groups and both
      // halves: every bank equally often, no swizzle needed.)
      const int sf = s / VW;
      lds_off[q] = ((((t * NSB + sf / 2) * 3) * 64 + gg * MT + i) * 16) + (sf % 2) * 8;
    }
  }
  int rd_slot[NV];  // this lane's (swizzled) slot when it reads vector q of a tile
#pragma unroll
  for (int q = 0; q < NV; q++) rd_slot[q] = lane ^ ((q * KL + g) & 7);
  const T *xrow[B_VECS];
#pragma unroll
  for (int q = 0; q < B_VECS; q++)
    xrow[q] = X + min(row0 + rr0 + q * ROWS_PER_PASS, n - 1) * (int64_t)d;

  // The accumulators hold -1/2 of the reference's value: they start at -(xx + cc)/2 and the
  // matrix cores add +x.c with the centroids staged as they are, which spares the staging of
  // every tile a multiplication by -2. Halving and doubling are exact, so every accumulator
  // is bit for bit -1/2 of (xx + cc) - 2 x.c accumulated in the same order; the comparisons
  // are unaffected and the distance that leaves the kernel is 2 |acc|. (They start at zero
  // and -(xx + cc)/2 joins them in the epilogue.)
  T xx[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++)
    xx[rt] = (T)-0.5 * xnorm[min(row0 + (wr * RT + rt) * MT + r, n - 1)];
  T best[RT];
  int bidx[RT];
  unsigned bkey[RT];
  int bblk[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {
    best[rt] = (T)0.5 * argmin_start<T>();  // the start value FLT_MAX on the accumulators' scale
    bidx[rt] = -1;
    bkey[rt] = 0x7EFFFFF0u;  // FLT_MAX / 2 with the index bits cleared
    bblk[rt] = -1;  // first centroid of the tile the best key came from
  }

  vec_t areg[A_VECS], breg[B_VECS];
  // SPLIT: the centroid parts come ready-made from Cparts (split_centroids_kernel), one LDS
  // image of A_BYTES per (centroid block, stage), copied as it lies
  constexpr int A_PVECS = SPLIT ? A_BYTES / 16 / WG : 1;
  static_assert(!SPLIT || A_BYTES % (16 * WG) == 0, "whole 16-byte vectors per thread");
  uintx4 apreg[A_PVECS];
  // Only the last d-step can reach past the feature count: the guards live in a second
  // instance of the loader (tail_tag true) used for that step alone.
  auto gload = [&](int c0, int st, auto tail_tag) {
    constexpr bool TAILSTEP = DTAIL && decltype(tail_tag)::value;
    const int j = stage_off(st) + jj;
    // VECLOAD: 16-byte loads at element-aligned addresses; in the tail step through
    // load_row_vector, which stays inside the row and returns zero past feature d
    auto fetch = [&](const T *src, bool zero_past_d) -> vec_t {
      vec_t v;
      if (VECLOAD) {
        if (TAILSTEP && d % VW == 0) {
          // no vector straddles the end of the row: one past it re-reads the last one and
          // is zeroed on the centroid side only (finite x * 0 adds nothing)
          const uvec_t u = *reinterpret_cast<const uvec_t *>(src + min(j, d - VW));
#pragma unroll
          for (int e = 0; e < VW; e++) v[e] = (zero_past_d && j >= d) ? (T)0 : u[e];
        } else if (TAILSTEP) {
          v = load_row_vector<T>(src, j, d);
        } else {
          // (EVEN: the vectors past a stage's own steps belong to the next stage and are not
          // used; near the end of the row they are fetched from inside it all the same)
          const uvec_t u = *reinterpret_cast<const uvec_t *>(src + (EVEN ? min(j, d - VW) : j));
#pragma unroll
          for (int e = 0; e < VW; e++) v[e] = u[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < VW; e++) v[e] = (j + e < d) ? src[min(j + e, d - 1)] : (T)0;
      }
      return v;
    };
    if constexpr (SPLIT != 0) {
      const uintx4 *cp = Cparts + ((size_t)(c0 / BC) * nstage + st) * (A_BYTES / 16) + tid;
#pragma unroll
      for (int q = 0; q < A_PVECS; q++) apreg[q] = cp[q * WG];
    } else {
      const T *cbase = C + (size_t)(c0 + rr0) * d;
#pragma unroll
      for (int q = 0; q < A_VECS; q++)
        areg[q] = fetch(cbase + (size_t)q * ROWS_PER_PASS * d, true);
    }
#pragma unroll
    for (int q = 0; q < B_VECS; q++) breg[q] = fetch(xrow[q], false);
  };
  // (SPLIT) the three bfloat16 parts of a staged vector, 8 bytes each
  auto store_parts = [&](unsigned char *dst, const vec_t &v) {
    if constexpr (SPLIT != 0) {
      typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
      uintx2 ph, pm, pl;
#pragma unroll
      for (int w = 0; w < 2; w++) {
        const Bf16x3Pair pr = split_pair_bf16x3((float)v[2 * w], (float)v[2 * w + 1]);
        ph[w] = pr.h;
        pm[w] = pr.m;
        pl[w] = pr.l;
      }
      *reinterpret_cast<uintx2 *>(dst) = ph;
      *reinterpret_cast<uintx2 *>(dst + 1024) = pm;
      *reinterpret_cast<uintx2 *>(dst + 2048) = pl;
    }
  };
  auto lstore = [&](int buf) {
    if constexpr (SPLIT != 0) {
#pragma unroll
      for (int q = 0; q < A_PVECS; q++)
        reinterpret_cast<uintx4 *>(Ab + buf * A_BYTES)[q * WG + tid] = apreg[q];
#pragma unroll
      for (int q = 0; q < B_VECS; q++) store_parts(Bb + buf * B_BYTES + lds_off[q], breg[q]);
      return;
    }
#pragma unroll
    for (int q = 0; q < A_VECS; q++)
      *reinterpret_cast<vec_t *>(As + buf * A_ELEMS + lds_off[q]) = areg[q];
#pragma unroll
    for (int q = 0; q < B_VECS; q++)
      *reinterpret_cast<vec_t *>(Bs + buf * B_ELEMS + lds_off[q]) = breg[q];
  };

  // MODE 1 has no dependency between centroid blocks: each workgroup takes a single
  // block, which keeps a short batch of rows (a transform of 100,000 rows is
  // 782 row tiles on 512 workgroup slots) from ending in a half-empty last round.
  const int c_begin = MODE == 1 ? cb_id * BC : 0;
  const int c_end = MODE == 1 ? min(k, c_begin + BC) : k;
  for (int c0 = c_begin; c0 < c_end; c0 += BC) {
    acc_t acc[CT][RT];
    // the copy of the norms this block's epilogue reads; the other copy may still be
    // read by wavefronts in the epilogue of the block before. Visible to everybody after the
    // barriers below.
    const T *cn = cns + (((c0 - c_begin) / BC) & 1) * BC;
    if (tid < BC) cns[(((c0 - c_begin) / BC) & 1) * BC + tid] = cnorm[c0 + tid];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
#pragma unroll
        for (int v = 0; v < NACC; v++) acc[ct][rt][v] = (T)0;
      }
    }
    if (DTAIL && nstage == 1) gload(c0, 0, std::true_type{});
    else gload(c0, 0, std::false_type{});
    __syncthreads();  // previous block's readers are done with buffer 0
    lstore(0);
    __syncthreads();
    for (int st = 0; st < nstage; st++) {
      const int buf = st & 1;
      if (st + 2 < nstage || (!DTAIL && st + 1 < nstage)) gload(c0, st + 1, std::false_type{});
      else if (st + 1 < nstage) gload(c0, st + 1, std::true_type{});
      // The stage's matrix instructions (and the operand reads between them) at the highest
      // wave priority, its staging at the lowest: the instruction arbiter then serves a
      // wavefront that is in its matrix phase before one that is storing its next tile, so
      // the matrix pipe waits less often for an issue slot (2M x 256, k = 1024: 8.27 -> 8.19 ms,
      // 500k x 784, k = 4096: 25.84 -> 25.58 ms; priority 1 gave half of that).
      __builtin_amdgcn_s_setprio(3);
      if constexpr (SPLIT != 0) {
        const uintx4 *ap = reinterpret_cast<const uintx4 *>(Ab + buf * A_BYTES) + lane;
        const uintx4 *bp = reinterpret_cast<const uintx4 *>(Bb + buf * B_BYTES) + lane;
#pragma unroll
        for (int sb = 0; sb < NSB; sb++) {
          uintx4 bh[RT], bm[RT], bl[RT];
#pragma unroll
          for (int rt = 0; rt < RT; rt++) {
            const int o = (((wr * RT + rt) * NSB + sb) * 3) * 64;
            bh[rt] = bp[o];
            bm[rt] = bp[o + 64];
            bl[rt] = bp[o + 128];
          }
#pragma unroll
          for (int ct = 0; ct < CT; ct++) {
            const int o = (((wc * CT + ct) * NSB + sb) * 3) * 64;
            const uintx4 ah = ap[o], am = ap[o + 64], al = ap[o + 128];
            // smallest products first
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
              if constexpr (SPLIT == 9) {
                acc[ct][rt] = mma_bf16(al, bl[rt], acc[ct][rt]);
                acc[ct][rt] = mma_bf16(al, bm[rt], acc[ct][rt]);
                acc[ct][rt] = mma_bf16(am, bl[rt], acc[ct][rt]);
              }
              acc[ct][rt] = mma_bf16(al, bh[rt], acc[ct][rt]);
              acc[ct][rt] = mma_bf16(ah, bl[rt], acc[ct][rt]);
              acc[ct][rt] = mma_bf16(am, bm[rt], acc[ct][rt]);
              acc[ct][rt] = mma_bf16(am, bh[rt], acc[ct][rt]);
              acc[ct][rt] = mma_bf16(ah, bm[rt], acc[ct][rt]);
              acc[ct][rt] = mma_bf16(ah, bh[rt], acc[ct][rt]);
            }
          }
        }
      }
      const vec_t *ap = reinterpret_cast<const vec_t *>(As + buf * A_ELEMS);
      const vec_t *bp = reinterpret_cast<const vec_t *>(Bs + buf * B_ELEMS);
      const int nq_st = DTAIL ? stage_nq(st) : NV;
      // Whole stages are one basic block of matrix instructions and operand reads: the
      // compiler's interleaving strategy for such blocks spreads the reads between the matrix
      // instructions instead of bunching them in front (256-centroid block, 500k x 784,
      // k = 4096: 25.71 -> 24.51 ms, 200k x 784: 11.32 -> 10.94 ms; the 128-centroid block and the
      // double kernels measured the same with and without it, the per-step blocks of the DTAIL
      // kernels do not benefit).
      if constexpr (!DTAIL && SPLIT == 0 && sizeof(T) == 4) __builtin_amdgcn_iglp_opt(0);
#pragma unroll
      for (int q = 0; q < (SPLIT ? 0 : NV); q++) {
        if (DTAIL && q >= nq_st) continue;  // nothing of this stage there
        vec_t a[CT], b[RT];
#pragma unroll
        for (int ct = 0; ct < CT; ct++) a[ct] = ap[((wc * CT + ct) * NV + q) * 64 + rd_slot[q]];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) b[rt] = bp[((wr * RT + rt) * NV + q) * 64 + rd_slot[q]];
#pragma unroll
        for (int e = 0; e < VW; e++) {
#pragma unroll
          for (int ct = 0; ct < CT; ct++) {
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
              acc[ct][rt] = M::mma(a[ct][e], b[rt][e], acc[ct][rt]);
          }
        }
      }
      __builtin_amdgcn_s_setprio(0);
      if (st + 1 < nstage) {
        lstore(buf ^ 1);  // the other buffer was last read one stage ago
        __syncthreads();
      }
    }
    // epilogue for this centroid block
    if (MODE == 1) {
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
#pragma unroll
        for (int v = 0; v < NACC; v++) {
          const int c = c0 + (wc * CT + ct) * MT + M::acc_row(v, g);
          const T cc = cn[c - c0];
#pragma unroll
          for (int rt = 0; rt < RT; rt++) {
            const int64_t row = row0 + (wr * RT + rt) * MT + r;
            const T a = acc[ct][rt][v] + fma((T)-0.5, cc, xx[rt]);
            if (c < k && row < n) D[(size_t)c * ldn + row] = (T)2 * fabs(a);
          }
        }
      }
    } else if constexpr (sizeof(T) == 4 && !EXACT) {
      // integer keys as in the row-stationary kernel (4 index bits, 16 ulp; a later tile
      // or block replaces the running key only from a lower bucket)
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
        T ccv[NACC];
#pragma unroll
        for (int v = 0; v < NACC; v++) ccv[v] = cn[(wc * CT + ct) * MT + M::acc_row(v, g)];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
          unsigned key[NACC];
#pragma unroll
          for (int v = 0; v < NACC; v++) {
            const float a = (float)(acc[ct][rt][v] + fma((T)-0.5, ccv[v], xx[rt]));
            key[v] = (__float_as_uint(a) & 0x7FFFFFF0u) | (unsigned)v;
          }
          unsigned m = umin3(key[0], key[1], key[2]);
#pragma unroll
          for (int v = 3; v + 1 < NACC; v += 2) m = umin3(m, key[v], key[v + 1]);
          if ((NACC & 1) == 0) m = min(m, key[NACC - 1]);
          if ((m | 15u) < bkey[rt]) {
            bkey[rt] = m;
            bblk[rt] = c0 + (wc * CT + ct) * MT;
          }
        }
      }
    } else {
      // The compare chain, three vector instructions per distance: the running best keeps
      // the accumulator's sign (the comparison takes both magnitudes through operand
      // modifiers), and the winner is remembered as its place inside the block, a small
      // constant, with the block itself noted once per block. Accumulators are visited in
      // ascending centroid order, so the strict '<' keeps the lowest index on ties.
      int loc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; rt++) loc[rt] = -1;
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
#pragma unroll
        for (int v = 0; v < NACC; v++) {
          const T cc = cn[(wc * CT + ct) * MT + M::acc_row(v, g)];
#pragma unroll
          for (int rt = 0; rt < RT; rt++) {
            const T a = acc[ct][rt][v] + fma((T)-0.5, cc, xx[rt]);
            if (fabs(a) < fabs(best[rt])) {
              best[rt] = a;
              loc[rt] = ct * NACC + v;
            }
          }
        }
      }
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        if (loc[rt] >= 0) {
          bblk[rt] = c0;
          bidx[rt] = loc[rt];
        }
      }
    }
  }
  if (MODE == 0) {
    if constexpr (sizeof(T) == 4 && !EXACT) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        best[rt] = __uint_as_float(bkey[rt] & 0xFFFFFFF0u);
        bidx[rt] = bblk[rt] < 0 ? -1 : bblk[rt] + key_row(bkey[rt] & 15u, g);
      }
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        best[rt] = fabs(best[rt]);
        if (bblk[rt] >= 0)
          bidx[rt] = bblk[rt] + (wc * CT + bidx[rt] / NACC) * MT + M::acc_row(bidx[rt] % NACC, g);
      }
    }
    // lane groups of one wavefront, then the two wavefronts sharing the rows
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
#pragma unroll
      for (int off = MT; off < 64; off <<= 1) {
        const T ob = __shfl_xor(best[rt], off, 64);
        const int oi = __shfl_xor(bidx[rt], off, 64);
        argmin_merge(best[rt], bidx[rt], ob, oi);
      }
    }
    __syncthreads();  // all waves are past their last LDS operand read
    T *mb = reinterpret_cast<T *>(smem_raw);                   // [BCW-1][BR]
    int *mi = reinterpret_cast<int *>(mb + (BCW - 1) * BR);    // [BCW-1][BR]
    if (wc > 0 && g == 0) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const int lr = (wr * RT + rt) * MT + r;
        mb[(wc - 1) * BR + lr] = best[rt];
        mi[(wc - 1) * BR + lr] = bidx[rt];
      }
    }
    __syncthreads();
    if (wc == 0 && g == 0) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const int lr = (wr * RT + rt) * MT + r;
#pragma unroll
        for (int w = 0; w < BCW - 1; w++)
          argmin_merge(best[rt], bidx[rt], mb[w * BR + lr], mi[w * BR + lr]);
        const int64_t row = row0 + lr;
        if (row < n) {
          labels[row] = bidx[rt];
          if (mindist) mindist[row] = (T)2 * best[rt];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Tiled kernel, operands staged by the memory system itself.
//
// The same tiling as assign_tiled_kernel for the shapes that need none of its special cases
// (rows and centroids whole numbers of stages, 16-byte aligned rows, float32 instructions or
// float64): here no operand passes through a register on its way to LDS. gfx950's
// global_load_lds_dwordx4 lets every lane name a 16-byte source and writes the 64 vectors of a
// wavefront to 64 consecutive 16-byte LDS slots, which is exactly one [tile][vector][lane]
// block of the operand-order layout when lane (group g, row i) asks for vector q * KL + g of
// the stage from row i of the tile. The stages form a ring of NBUF buffers and the loads run
// NBUF - 1 stages ahead of the matrix instructions; a wavefront waits for its own loads of a
// stage with s_waitcnt vmcnt (the loads of later stages stay in flight), the workgroup's
// barrier then covers everybody else's, and the loads of the stage NBUF - 1 ahead are
// issued right behind the barrier, into the buffer the stage before this one was read from.
// All (centroid block, stage) pairs of a workgroup run as one pipeline, so a new centroid
// block starts with its first stages already in LDS.
//
// The accumulators start at zero and -(xx + cc)/2 is added when a block is complete (the order
// of a GEMM with beta = 1, which is what the reference runs, kmeans_labels.cu:158-165): the
// partial sums of the dot product are then rounded at their own size instead of at the size
// of xx + cc, which measured 1.5 times less rounding noise in the minimum distance at 256
// features than accumulators that start at -(xx + cc)/2.
// ---------------------------------------------------------------------------
template <typename T, int BCW, bool WIDE, int BK, int NBUF>
struct DmaCfg {
  typedef Mfma<T> M;
  static constexpr int TPB = 2 * BCW * 64;
  static constexpr int BC = 64 * BCW * (WIDE ? 2 : 1);
  static constexpr int BR = 128;
  static constexpr int STAGE_ELEMS = (BC + BR) * BK;
  // ring of stages + two copies of the block's centroid norms
  static constexpr size_t LDS_BYTES = ((size_t)NBUF * STAGE_ELEMS + 2 * BC) * sizeof(T);
};

// One direct-to-LDS load: every lane's 16 bytes (4 for the narrow form) from its own global
// address, the wavefront's 64 results to consecutive LDS slots starting at `lds` (the same
// address in every lane). The builtin exists for the gfx950 target only; the host pass of the
// compiler, which has to see the kernel's body to emit its launch stub, gets an empty function.
__device__ __forceinline__ void dma_to_lds_16(const void *gsrc, void *lds) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_global_load_lds(gsrc, (__attribute__((address_space(3))) void *)(lds), 16, 0, 0);
#else
  (void)gsrc;
  (void)lds;
#endif
}
// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters at
// "do not wait")
#define KM_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14))

template <typename T, int MODE, int BCW, bool EXACT, bool WIDE, int BK, int NBUF, bool SPREAD>
__global__ __launch_bounds__(2 * BCW * 64, 2) void assign_tiled_dma_kernel(
    const T *__restrict__ X, const T *__restrict__ xnorm,
    const T *__restrict__ C, const T *__restrict__ cnorm,
    int *__restrict__ labels, T *__restrict__ mindist, T *__restrict__ D,
    int64_t n, int64_t ldn, int d, int k) {
  typedef Mfma<T> M;
  typedef DmaCfg<T, BCW, WIDE, BK, NBUF> Cfg;
  constexpr int MT = M::MT, KL = M::KL, NACC = M::NACC, VW = M::VW;
  constexpr int BC = Cfg::BC, BR = Cfg::BR, NWAVE = Cfg::TPB / 64;
  constexpr int NV = BK / KL / VW;   // 16-byte vectors per lane per tile per stage
  constexpr int CT = BC / BCW / MT;  // centroid tiles per wavefront
  constexpr int RT = BR / 2 / MT;    // row tiles per wavefront
  constexpr int TILE_ELEMS = MT * BK;
  constexpr int A_TILES = BC / MT, B_TILES = BR / MT;
  constexpr int A_TPW = A_TILES / NWAVE, B_TPW = B_TILES / NWAVE;  // tiles a wavefront fetches
  constexpr int A_ELEMS = A_TILES * TILE_ELEMS;  // the A part of a stage
  constexpr int STAGE_ELEMS = Cfg::STAGE_ELEMS;
  static_assert(A_TILES % NWAVE == 0 && B_TILES % NWAVE == 0, "tiles are dealt evenly to the wavefronts");
  static_assert(BK % (KL * VW) == 0 && NBUF >= 2 && NBUF <= 4, "whole vectors per lane group");
  constexpr int LPW = (A_TPW + B_TPW) * NV;  // loads per wavefront and stage
  constexpr int AHEAD = NBUF - 1;
  static_assert((AHEAD - 1) * LPW < 64, "vmcnt is a 6-bit counter");
  typedef typename M::acc_t acc_t;
  typedef typename M::vec_t vec_t;

  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wc = wave % BCW;
  const int wr = wave / BCW;
  const int r = lane % MT;
  const int g = lane / MT;
  T *ring = reinterpret_cast<T *>(smem_raw);   // [NBUF][A tiles | B tiles]
  T *cns = ring + (size_t)NBUF * STAGE_ELEMS;  // [2][BC]: squared norms of the current block's centroids
  const int ncb = (k + BC - 1) / BC;
  const int64_t rt_id = MODE == 1 ? (int64_t)blockIdx.x / ncb : (int64_t)blockIdx.x;
  const int cb_id = MODE == 1 ? (int)((int64_t)blockIdx.x - rt_id * ncb) : 0;
  const int64_t row0 = rt_id * BR;
  const int nstage = d / BK;
  const int c_begin = MODE == 1 ? cb_id * BC : 0;
  const int nblk = MODE == 1 ? 1 : ncb;
  const int total = nblk * nstage;  // stages of this workgroup's pipeline

  // What this lane fetches: vector g (+ q * KL) of the stage from row r of each tile the
  // wavefront is responsible for, as a byte offset from a base that is the same for the whole
  // workgroup (the block's first centroid, the workgroup's first row): the loads then take
  // their address as scalar base + 32-bit lane offset and cost no vector arithmetic.
  unsigned aoff[A_TPW], boff[B_TPW];
#pragma unroll
  for (int t = 0; t < A_TPW; t++)
    aoff[t] = (unsigned)((((wave * A_TPW + t) * MT + r) * (size_t)d + g * VW) * sizeof(T));
#pragma unroll
  for (int t = 0; t < B_TPW; t++) {
    const int64_t row = min(row0 + (wave * B_TPW + t) * MT + r, n - 1);  // clamped: stays inside X
    boff[t] = (unsigned)(((row - row0) * (int64_t)d + g * VW) * sizeof(T));
  }
  const char *const xbase = reinterpret_cast<const char *>(X + row0 * (int64_t)d);
  // the pipeline's fetch position: stage ist of block iblk goes to ring slot ibuf
  int iblk = 0, ist = 0, ibuf = 0, issued = 0;
  // The burst form takes the tiles one after the other, the NV vectors of a tile in a row:
  // they ask for adjacent pieces of the same 32 (16) rows, i.e. of the same cache lines.
  // vector q of every tile the wavefront fetches (the order the 256-centroid block of a fit
  // prefers when the loads are spread over the stage: 500k x 784, k = 4096 23.7 against 24.5 ms)
  auto issue_part = [&](int q) {
    T *dst = ring + (size_t)ibuf * STAGE_ELEMS;
    const char *abase = reinterpret_cast<const char *>(C + ((size_t)(c_begin + iblk * BC) * d + (size_t)ist * BK));
    const char *bbase = xbase + (size_t)ist * BK * sizeof(T);
#pragma unroll
    for (int t = 0; t < A_TPW; t++)
      dma_to_lds_16(abase + q * KL * VW * sizeof(T) + aoff[t], dst + ((wave * A_TPW + t) * NV + q) * 64 * VW);
#pragma unroll
    for (int t = 0; t < B_TPW; t++)
      dma_to_lds_16(bbase + q * KL * VW * sizeof(T) + boff[t],
                    dst + A_ELEMS + ((wave * B_TPW + t) * NV + q) * 64 * VW);
  };
  auto issue_done = [&]() {
    issued++;
    ibuf = ibuf + 1 == NBUF ? 0 : ibuf + 1;
    if (++ist == nstage) {
      ist = 0;
      iblk++;
    }
  };
  // all of a stage's loads, tile by tile
  auto issue_all = [&]() {
    T *dst = ring + (size_t)ibuf * STAGE_ELEMS;
    const char *abase = reinterpret_cast<const char *>(C + ((size_t)(c_begin + iblk * BC) * d + (size_t)ist * BK));
    const char *bbase = xbase + (size_t)ist * BK * sizeof(T);
#pragma unroll
    for (int t = 0; t < A_TPW; t++) {
#pragma unroll
      for (int q = 0; q < NV; q++)
        dma_to_lds_16(abase + q * KL * VW * sizeof(T) + aoff[t], dst + ((wave * A_TPW + t) * NV + q) * 64 * VW);
    }
#pragma unroll
    for (int t = 0; t < B_TPW; t++) {
#pragma unroll
      for (int q = 0; q < NV; q++)
        dma_to_lds_16(bbase + q * KL * VW * sizeof(T) + boff[t],
                      dst + A_ELEMS + ((wave * B_TPW + t) * NV + q) * 64 * VW);
    }
  };
  auto issue = [&]() {
    issue_all();
    issue_done();
  };

  T xxh[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++)
    xxh[rt] = (T)-0.5 * xnorm[min(row0 + (wr * RT + rt) * MT + r, n - 1)];
  T best[RT];
  int bidx[RT];
  unsigned bkey[RT];
  int bblk[RT];
#pragma unroll
  for (int rt = 0; rt < RT; rt++) {
    best[rt] = (T)0.5 * argmin_start<T>();  // the start value FLT_MAX on the accumulators' scale
    bidx[rt] = -1;
    bkey[rt] = 0x7EFFFFF0u;  // FLT_MAX / 2 with the index bits cleared
    bblk[rt] = -1;
  }

#pragma unroll
  for (int a = 0; a < AHEAD; a++)
    if (issued < total) issue();
  // the row norms are in their registers before the loop starts (the loads above, issued
  // after them, stay in flight): no wait for them can end up inside the pipeline
#pragma unroll
  for (int rt = 0; rt < RT; rt++) asm volatile("" : "+v"(xxh[rt]));

  int buf = 0, done = 0;
  for (int blk = 0; blk < nblk; blk++) {
    const int c0 = c_begin + blk * BC;
    // This block's centroid norms for the epilogue, fetched the same way (64 lanes x 16 bytes
    // cover the block); they have landed and are visible to everybody at the latest after the
    // second barrier below. The copy of the block before stays readable for wavefronts that
    // are still in its epilogue.
    T *cn = cns + (blk & 1) * BC;
    static_assert(BC / VW <= 64, "one wavefront fetches the block's norms");
    if (wave == 0 && lane < BC / VW) dma_to_lds_16(cnorm + c0 + lane * VW, cn);
    acc_t acc[CT][RT];
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
#pragma unroll
        for (int v = 0; v < NACC; v++) acc[ct][rt][v] = (T)0;
      }
    }
    for (int st = 0; st < nstage; st++) {
      // this wavefront's loads of the stage have landed (those of the AHEAD - 1 stages after it
      // may still be under way), then everybody's
      if (AHEAD > 1 && issued - done >= AHEAD) KM_WAIT_VMCNT((AHEAD - 1) * LPW);
      else KM_WAIT_VMCNT(0);
      __syncthreads();
      const bool more = issued < total;  // the next stage to fetch goes into the slot read one stage ago
      // SPREAD: a part of the next stage's loads in front of every step's matrix instructions
      // instead of all of them in front of the stage.
      if constexpr (!SPREAD) {
        if (more) issue_all();
      }
      __builtin_amdgcn_s_setprio(3);
      const vec_t *ap = reinterpret_cast<const vec_t *>(ring + (size_t)buf * STAGE_ELEMS) + lane;
      const vec_t *bp = ap + A_ELEMS / VW;
      if constexpr (sizeof(T) == 4) __builtin_amdgcn_iglp_opt(0);
#pragma unroll
      for (int q = 0; q < NV; q++) {
        if constexpr (SPREAD) {
          if (more) issue_part(q);
        }
        vec_t a[CT], b[RT];
#pragma unroll
        for (int ct = 0; ct < CT; ct++) a[ct] = ap[((wc * CT + ct) * NV + q) * 64];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) b[rt] = bp[((wr * RT + rt) * NV + q) * 64];
#pragma unroll
        for (int e = 0; e < VW; e++) {
#pragma unroll
          for (int ct = 0; ct < CT; ct++) {
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
              acc[ct][rt] = M::mma(a[ct][e], b[rt][e], acc[ct][rt]);
          }
        }
      }
      __builtin_amdgcn_s_setprio(0);
      if (more) issue_done();
      done++;
      buf = buf + 1 == NBUF ? 0 : buf + 1;
    }
    if (nstage < NBUF) {  // too few waits since the norms were asked for: wait for them here
      KM_WAIT_VMCNT(0);
      __syncthreads();
    }
    // epilogue of the block: a = x.c - (xx + cc)/2, i.e. -1/2 of the reference's value with its
    // rounding order ((xx + cc) first, then the product term); -(xx + cc)/2 as one fused
    // multiply-add of exact terms, i.e. rounded once like xx + cc itself
    if (MODE == 1) {
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
#pragma unroll
        for (int v = 0; v < NACC; v++) {
          const int cl = (wc * CT + ct) * MT + M::acc_row(v, g);
          const T cc = cn[cl];
#pragma unroll
          for (int rt = 0; rt < RT; rt++) {
            const int64_t row = row0 + (wr * RT + rt) * MT + r;
            const T a = acc[ct][rt][v] + fma((T)-0.5, cc, xxh[rt]);
            if (c0 + cl < k && row < n) D[(size_t)(c0 + cl) * ldn + row] = (T)2 * fabs(a);
          }
        }
      }
    } else if constexpr (sizeof(T) == 4 && !EXACT) {
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
        T ccv[NACC];
#pragma unroll
        for (int v = 0; v < NACC; v++) ccv[v] = cn[(wc * CT + ct) * MT + M::acc_row(v, g)];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
          unsigned key[NACC];
#pragma unroll
          for (int v = 0; v < NACC; v++)
            key[v] = (__float_as_uint(acc[ct][rt][v] + fmaf(-0.5f, ccv[v], xxh[rt])) & 0x7FFFFFF0u) | (unsigned)v;
          unsigned m = umin3(key[0], key[1], key[2]);
#pragma unroll
          for (int v = 3; v + 1 < NACC; v += 2) m = umin3(m, key[v], key[v + 1]);
          if ((NACC & 1) == 0) m = min(m, key[NACC - 1]);
          if ((m | 15u) < bkey[rt]) {
            bkey[rt] = m;
            bblk[rt] = c0 + (wc * CT + ct) * MT;
          }
        }
      }
    } else {
      int loc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; rt++) loc[rt] = -1;
#pragma unroll
      for (int ct = 0; ct < CT; ct++) {
#pragma unroll
        for (int v = 0; v < NACC; v++) {
          const T cc = cn[(wc * CT + ct) * MT + M::acc_row(v, g)];
#pragma unroll
          for (int rt = 0; rt < RT; rt++) {
            const T a = acc[ct][rt][v] + fma((T)-0.5, cc, xxh[rt]);
            if (fabs(a) < fabs(best[rt])) {
              best[rt] = a;
              loc[rt] = ct * NACC + v;
            }
          }
        }
      }
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        if (loc[rt] >= 0) {
          bblk[rt] = c0;
          bidx[rt] = loc[rt];
        }
      }
    }
  }
  if (MODE == 0) {
    if constexpr (sizeof(T) == 4 && !EXACT) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        best[rt] = __uint_as_float(bkey[rt] & 0xFFFFFFF0u);
        bidx[rt] = bblk[rt] < 0 ? -1 : bblk[rt] + key_row(bkey[rt] & 15u, g);
      }
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        best[rt] = fabs(best[rt]);
        if (bblk[rt] >= 0)
          bidx[rt] = bblk[rt] + (wc * CT + bidx[rt] / NACC) * MT + M::acc_row(bidx[rt] % NACC, g);
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
#pragma unroll
      for (int off = MT; off < 64; off <<= 1) {
        const T ob = __shfl_xor(best[rt], off, 64);
        const int oi = __shfl_xor(bidx[rt], off, 64);
        argmin_merge(best[rt], bidx[rt], ob, oi);
      }
    }
    __syncthreads();  // all waves are past their last LDS operand read
    T *mb = reinterpret_cast<T *>(smem_raw);                   // [BCW-1][BR]
    int *mi = reinterpret_cast<int *>(mb + (BCW - 1) * BR);    // [BCW-1][BR]
    if (wc > 0 && g == 0) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const int lr = (wr * RT + rt) * MT + r;
        mb[(wc - 1) * BR + lr] = best[rt];
        mi[(wc - 1) * BR + lr] = bidx[rt];
      }
    }
    __syncthreads();
    if (wc == 0 && g == 0) {
#pragma unroll
      for (int rt = 0; rt < RT; rt++) {
        const int lr = (wr * RT + rt) * MT + r;
#pragma unroll
        for (int w = 0; w < BCW - 1; w++)
          argmin_merge(best[rt], bidx[rt], mb[w * BR + lr], mi[w * BR + lr]);
        const int64_t row = row0 + lr;
        if (row < n) {
          labels[row] = bidx[rt];
          if (mindist) mindist[row] = (T)2 * best[rt];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
const char *assign_variant_name(int variant) {
  switch (variant) {
    case ASSIGN_VALU: return "valu";
    case ASSIGN_ROWSTAT: return "mfma_rowstat";
    case ASSIGN_TILED: return "mfma_tiled";
    case ASSIGN_LONGROW: return "wave_row";
    default: return "auto";
  }
}


template <typename T>
static int rowstat_dp(int d) {
  const int maxdp = sizeof(T) == 4 ? 128 : 64;
  for (int dp = 8; dp <= maxdp; dp *= 2)
    if (d <= dp) return dp;
  return 0;
}
// split != 0: the staged centroids are three bfloat16 parts per element (6 bytes)
template <typename T>
static size_t rowstat_lds(int d, int k, int split = 0) {
  const int MT = Mfma<T>::MT;
  const int kp = (k + MT - 1) / MT * MT;
  return (size_t)kp * rowstat_dp<T>(d) * (split ? 6 : sizeof(T)) + (size_t)kp * sizeof(T);
}

static const size_t ROWSTAT_LDS_MAX = 96 * 1024;
// centroids per chunk of a chunked row-stationary sweep (a multiple of the MFMA tile)
template <typename T>
static int rowstat_chunk(int d, int k, int split = 0) {
  if (rowstat_lds<T>(d, k, split) <= ROWSTAT_LDS_MAX) return k;
  const int MT = Mfma<T>::MT;
  const size_t per = (size_t)rowstat_dp<T>(d) * (split ? 6 : sizeof(T)) + sizeof(T);
  const int kc_max = (int)(ROWSTAT_LDS_MAX / per) / MT * MT;
  const int chunks = (k + kc_max - 1) / kc_max;
  const int kc = ((k + chunks - 1) / chunks + MT - 1) / MT * MT;  // balanced
  return kc;
}

template <typename T>
int pick_assign_variant(int requested, int64_t n, int d, int k) {
  const int dp = rowstat_dp<T>(d);
  const bool rowstat_ok = dp != 0 && rowstat_lds<T>(d, k) <= ROWSTAT_LDS_MAX;
  // any model can be swept in LDS-sized chunks of centroids (one launch per chunk)
  if (requested == ASSIGN_ROWSTAT) return dp != 0 ? ASSIGN_ROWSTAT : -1;
  if (requested == ASSIGN_VALU || requested == ASSIGN_TILED) return requested;
  if (requested == ASSIGN_LONGROW) return longrow_applies<T>(d, k) ? ASSIGN_LONGROW : -1;
  // the reference switches to its hand-written small kernel at k<=16 && d<=64
  // (kmeans_labels.cu:140,207); same boundary here
  if (k <= 16 && d <= 64) return ASSIGN_VALU;
  // Up to four centroids and rows beyond 64 features: the one-pass kernel of longrow_kernels.hip is
  // ahead of the matrix-core kernels on every such shape (2M x 128, k = 4: 0.34 against 0.62 ms per
  // step, 2M x 72: 0.32 against 0.37; float64 1M x 128: 0.26 against 0.52, 1M x 200: 0.33 against 0.86).
  if (k <= 4 && longrow_applies<T>(d, k)) return ASSIGN_LONGROW;
  if (rowstat_ok) return ASSIGN_ROWSTAT;
  // Short rows with a large model: the tiled kernel's d-loop has one or two stages and
  // cannot hide its loads; chunked row-stationary sweeps re-read X once per chunk, which
  // is cheap next to the matrix work of 700+ centroids. Longer rows only when they fill the
  // register slice exactly (measured, chunked vs tiled: 2M x 128 f32 k=2048 0.83 vs 0.78 of
  // peak, 4M x 64 f64 k=2048 0.78 vs 0.68; with d = 96 padded to 128 it is 0.58 vs 0.71).
  if (dp != 0 && (dp * (int)sizeof(T) <= 256 || d == dp)) return ASSIGN_ROWSTAT;
  // Long rows and a handful of centroids: the tiled kernel would pad the model to 64 centroids
  // and need a second pass over the rows for the sums; one wavefront along the features of
  // four rows reads them once.
  // (float64, whose exchanges between lanes cost twice the float32 ones: 5 to 8 centroids from 96
  // features on, 1M x 96, k = 8: 0.33 against 0.40 ms, 1M x 128: 0.35 against 0.52; 9 to 16 from 224 on,
  // 1M x 128, k = 16: 0.66 against 0.53, 1M x 192: 0.86 against 0.85, 1M x 252, k = 12: 0.82 against 1.03,
  // 500k x 256, k = 8: 0.30 against 0.64; float32 from the first shape the row-stationary kernel does
  // not take: 1M x 132, k = 8: 0.27 against 0.37 ms, 500k x 784, k = 10: 0.51 against 0.86 ms)
  if (longrow_applies<T>(d, k) && (sizeof(T) == 4 || d >= (k <= 8 ? 96 : 224))) return ASSIGN_LONGROW;
  return ASSIGN_TILED;
}

template <typename T, int MODE>
static int launch_valu(hipStream_t s, const T *X, const T *xnorm, const T *C,
                       const T *cnorm, int *labels, T *mindist, T *D, int64_t n,
                       int64_t ldn, int d, int k) {
  // centroid chunk: as many whole centroids as fit in 48 KB
  int kc = (int)((48 * 1024) / ((size_t)(d + 1) * sizeof(T)));
  if (kc < 1) return H2O4GPU_KMEANS_EARG;  // d beyond 12K features
  if (kc > k) kc = k;
  const size_t lds = (size_t)kc * (d + 1) * sizeof(T);
  const dim3 grid((unsigned)((n + WG - 1) / WG));
#define KM_VALU(DREG)                                                          \
  hipLaunchKernelGGL((assign_valu_kernel<T, DREG, MODE>), grid, dim3(WG), lds, \
                     s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn, d, k, kc)
  if (d <= 4) KM_VALU(4);
  else if (d <= 8) KM_VALU(8);
  else if (d <= 16) KM_VALU(16);
  else if (d <= 32) KM_VALU(32);
  else if (d <= 64) KM_VALU(64);
  else KM_VALU(0);
#undef KM_VALU
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template <typename T>
static size_t rowstat_fused_lds(int d, int k, int split = 0) {
  const int dp = rowstat_dp<T>(d);
  return rowstat_lds<T>(d, k, split) + 8 + (size_t)k * (dp + 1) * sizeof(double) + (size_t)k * sizeof(int);
}
static const size_t ROWSTAT_FUSED_LDS_MAX = 150 * 1024;
// The number of bfloat16 products (0, 6 or 9) a row-stationary launch of this shape runs
// with when `split` is asked for: float32 rows of whole 16-feature steps whose staged parts
// (half as large again as the floats) still fit.
template <typename T>
static int rowstat_split(int split, int d, int k, bool fused) {
  if (sizeof(T) != 4 || (split != 6 && split != 9)) return 0;
  if (rowstat_dp<T>(d) < 16 || rowstat_dp<T>(d) > 64 || d < Mfma<T>::VW) return 0;
  if (fused ? rowstat_fused_lds<T>(d, k, split) > ROWSTAT_FUSED_LDS_MAX
            : rowstat_lds<T>(d, k, split) > ROWSTAT_LDS_MAX)
    return 0;  // (an assignment-only sweep is cut into chunks that fit before it gets here)
  return split;
}

// Persistent grid of the row-stationary kernels: as many workgroups as stay
// resident (two 4-wave workgroups per CU while two LDS images fit, otherwise
// one 8-wave workgroup per CU), never more than there are row tiles.
static bool rowstat_two_per_cu(size_t lds) { return lds <= (size_t)80 * 1024; }

template <typename T, int DP, int ROWT, bool FUSE, int NW, int SPLIT = 0>
static int launch_rowstat_nw(hipStream_t s, const T *X, const T *xnorm, const T *C,
                             const T *cnorm, int *labels, T *mindist, int64_t n, int d,
                             int k, int num_cu, double *psums, int *pcounts, int *slots,
                             size_t lds, int c_off, int merge, bool exact, const StackShape &st) {
  const int MT = Mfma<T>::MT;
  const int kp = (k + MT - 1) / MT * MT;
  const int sets = st.sets > 1 ? st.sets : 1;
  const int kps = sets > 1 ? st.kps : kp, kset = sets > 1 ? st.kset : k;
  if (sets > 1 && (kps % MT != 0 || (int64_t)sets * kps != k || kset > kps || c_off != 0 || merge))
    return H2O4GPU_KMEANS_EARG;
  // (row tiles go round the workgroups before a second wavefront of any gets one, so a
  // small data set spreads over as many CUs as it has tiles)
  const int rows_per_wave = ROWT * MT;
  const int64_t tiles = (n + rows_per_wave - 1) / rows_per_wave;
  int64_t grid = (int64_t)num_cu * (NW == 4 ? 2 : 1);
  if (grid > tiles) grid = tiles;
  if (grid < 1) grid = 1;
  if (slots) *slots = (int)grid;
  const bool xal = (reinterpret_cast<uintptr_t>(X) & 15) == 0;
  const bool vec = (d == DP) && xal && ((reinterpret_cast<uintptr_t>(C) & 15) == 0);
  const bool padvec = !vec && d >= Mfma<T>::VW;
#define KM_RS_LAUNCH_X(LOAD, EXACT)                                                           \
  do {                                                                                        \
    auto kern = assign_rowstat_kernel<T, DP, ROWT, LOAD, FUSE, NW, EXACT, SPLIT>;             \
    KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds));                    \
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), lds, s, X, xnorm, C, cnorm, \
                       labels, mindist, n, d, k, kp, psums, pcounts, c_off, merge, sets, kps, \
                       kset);                                                                 \
  } while (0)
  // the exact-compare form exists for the float32 assignment-only kernels
#define KM_RS_LAUNCH(LOAD)                                       \
  do {                                                           \
    if constexpr (SPLIT != 0) {                                  \
      if constexpr (LOAD != 0) KM_RS_LAUNCH_X(LOAD, false);      \
      else return H2O4GPU_KMEANS_EARG;                           \
    } else if constexpr (!FUSE && sizeof(T) == 4) {              \
      if (exact) KM_RS_LAUNCH_X(LOAD, true);                     \
      else KM_RS_LAUNCH_X(LOAD, false);                          \
    } else {                                                     \
      KM_RS_LAUNCH_X(LOAD, false);                               \
    }                                                            \
  } while (0)
  if (vec) KM_RS_LAUNCH(1);
  else if (padvec) KM_RS_LAUNCH(2);
  else KM_RS_LAUNCH(0);
#undef KM_RS_LAUNCH
#undef KM_RS_LAUNCH_X
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template <typename T, int DP, int ROWT, bool FUSE>
static int launch_rowstat_dp(hipStream_t s, const T *X, const T *xnorm,
                             const T *C, const T *cnorm, int *labels,
                             T *mindist, int64_t n, int d, int k, int num_cu,
                             double *psums, int *pcounts, int *slots, int c_off, int merge,
                             bool exact, const StackShape &st) {
  const size_t lds = FUSE ? rowstat_fused_lds<T>(d, k) : rowstat_lds<T>(d, k);
  // Shapes whose register use fits 128 VGPRs run one 16-wavefront workgroup per CU, which
  // measured ahead of two 4-wave workgroups everywhere it applies (float32 10M x 32 and
  // 8M x 16: 5-12 %; 1M x 64, k = 64: 12 %; float64 8M x 16: 8 %).
  constexpr bool wide = (sizeof(T) == 4 && (DP <= 32 || (DP == 64 && ROWT == 1))) ||
                        (sizeof(T) == 8 && ((DP <= 32 && ROWT <= 2) || (DP == 64 && ROWT == 1)));
  if (!wide && rowstat_two_per_cu(lds))
    return launch_rowstat_nw<T, DP, ROWT, FUSE, 4>(s, X, xnorm, C, cnorm, labels, mindist, n, d,
                                                   k, num_cu, psums, pcounts, slots, lds, c_off, merge, exact, st);
  // one workgroup per CU: as many wavefronts as the register budget allows
  if constexpr (wide)
    return launch_rowstat_nw<T, DP, ROWT, FUSE, 16>(s, X, xnorm, C, cnorm, labels, mindist, n, d,
                                                    k, num_cu, psums, pcounts, slots, lds, c_off, merge, exact, st);
  else
    return launch_rowstat_nw<T, DP, ROWT, FUSE, 8>(s, X, xnorm, C, cnorm, labels, mindist, n, d,
                                                   k, num_cu, psums, pcounts, slots, lds, c_off, merge, exact, st);
}

// The float32 shapes on the bfloat16 matrix pipe: the three parts of a row tile take half
// as many registers again as the floats, so one row tile per wavefront.
template <bool FUSE, int SPLIT>
static int launch_rowstat_split(hipStream_t s, const float *X, const float *xnorm, const float *C,
                                const float *cnorm, int *labels, float *mindist, int64_t n, int d,
                                int k, int num_cu, double *psums, int *pcounts, int *slots,
                                int c_off, int merge, const StackShape &st) {
  const size_t lds = FUSE ? rowstat_fused_lds<float>(d, k, SPLIT) : rowstat_lds<float>(d, k, SPLIT);
#define KM_SPLIT_CASE(DP, ROWT, NW)                                                              \
  case DP:                                                                                       \
    return launch_rowstat_nw<float, DP, ROWT, FUSE, NW, SPLIT>(s, X, xnorm, C, cnorm, labels,    \
                                                               mindist, n, d, k, num_cu, psums,  \
                                                               pcounts, slots, lds, c_off, merge, false, st)
  switch (rowstat_dp<float>(d)) {
    KM_SPLIT_CASE(16, 1, 16);
    KM_SPLIT_CASE(32, 1, 16);
    KM_SPLIT_CASE(64, 1, 8);
  }
#undef KM_SPLIT_CASE
  return H2O4GPU_KMEANS_EARG;
}

template <typename T, bool FUSE>
struct RowstatDispatch;
#define KM_ROWSTAT_CASE(T, DP, ROWT)                                                  \
  case DP:                                                                            \
    return launch_rowstat_dp<T, DP, ROWT, FUSE>(s, X, xnorm, C, cnorm, labels, mindist, \
                                                n, d, k, num_cu, psums, pcounts, slots, c_off, merge, exact, st)
template <bool FUSE>
struct RowstatDispatch<float, FUSE> {
  static int run(hipStream_t s, const float *X, const float *xnorm, const float *C,
                 const float *cnorm, int *labels, float *mindist, int64_t n, int d,
                 int k, int num_cu, double *psums, int *pcounts, int *slots, int c_off = 0,
                 int merge = 0, bool exact = false, const StackShape &st = StackShape(),
                 int split = 0) {
    if (!exact) {
      split = rowstat_split<float>(split, d, k, FUSE);
      if (split == 9)
        return launch_rowstat_split<FUSE, 9>(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu,
                                             psums, pcounts, slots, c_off, merge, st);
      if (split == 6)
        return launch_rowstat_split<FUSE, 6>(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu,
                                             psums, pcounts, slots, c_off, merge, st);
    }
    switch (rowstat_dp<float>(d)) {
      KM_ROWSTAT_CASE(float, 8, 2);
      KM_ROWSTAT_CASE(float, 16, 2);
      KM_ROWSTAT_CASE(float, 32, 2);
      KM_ROWSTAT_CASE(float, 64, 1);  // one row tile: fits 16 wavefronts per CU
      KM_ROWSTAT_CASE(float, 128, 1);
    }
    return H2O4GPU_KMEANS_EARG;
  }
};
template <bool FUSE>
struct RowstatDispatch<double, FUSE> {
  static int run(hipStream_t s, const double *X, const double *xnorm, const double *C,
                 const double *cnorm, int *labels, double *mindist, int64_t n, int d,
                 int k, int num_cu, double *psums, int *pcounts, int *slots, int c_off = 0,
                 int merge = 0, bool exact = false, const StackShape &st = StackShape(),
                 int split = 0) {
    (void)split;  // float32 only
    switch (rowstat_dp<double>(d)) {
      // two row tiles keep these within 128 registers, i.e. 16 wavefronts per CU
      KM_ROWSTAT_CASE(double, 8, 2);
      KM_ROWSTAT_CASE(double, 16, 2);
      KM_ROWSTAT_CASE(double, 32, 2);
      KM_ROWSTAT_CASE(double, 64, 1);
    }
    return H2O4GPU_KMEANS_EARG;
  }
};
#undef KM_ROWSTAT_CASE

static bool valu_fused_applies(int d, int k) { return k <= 16 && d <= 64; }
// LDS of the two fused kernels for a shape: `reg` = the register variant (d one of 4, 8, 16,
// 32, 64 and 16-byte aligned rows), otherwise the any-d variant.
template <typename T>
static size_t valu_fused_lds(int d, int k, bool sums, bool reg, int ncopy) {
  const int vw = Mfma<T>::VW;
  const size_t sum_bytes = sums ? (size_t)ncopy * k * sums_stride(d) * sizeof(double) : 0;
  if (reg) {
    const int kq = (k + 3) & ~3;
    const int sxt = d == vw ? d : d + vw;
    return sum_bytes + (sums ? (size_t)kq * sizeof(int) : 0) + (size_t)kq * sizeof(T) +
           (size_t)WG * sxt * sizeof(T);
  }
  const int sx = staged_row_stride(d);
  return sum_bytes + (sums ? ((size_t)k + 1) * sizeof(int) : 0) + ((size_t)k + 1) * sizeof(T) +
         (size_t)WG * sx * sizeof(T) + 16;
}
// Copies of the sums (see sums_stride): as many of 4, 2, 1 as leave the workgroups per CU that
// one copy allows (by LDS; at most 8 are used).
template <typename T>
static int valu_fused_copies(int d, int k, bool reg) {
  auto per_cu = [&](int nc) {
    const int v = (int)((160 * 1024) / valu_fused_lds<T>(d, k, true, reg, nc));
    return v > 8 ? 8 : v;
  };
  for (int nc = 4; nc > 1; nc >>= 1)
    if (per_cu(nc) >= per_cu(1) && per_cu(nc) >= 1) return nc;
  return 1;
}
static int valu_fused_grid(int64_t n, int resident, int num_cu) {
  int per_cu = resident;  // what a CU holds at once of this kernel instance
  if (per_cu > 8) per_cu = 8;
  if (per_cu < 1) per_cu = 1;
  int64_t grid = (int64_t)num_cu * per_cu;
  const int64_t blocks = (n + WG - 1) / WG;
  if (grid > blocks) grid = blocks;
  return (int)(grid < 1 ? 1 : grid);
}

// Fused assign + accumulate is offered where the row-stationary kernel applies
// and centroids plus the double-precision sums fit in one CU's LDS, and for the
// small shapes the VALU kernel serves.
template <typename T>
int fused_slots(int requested_variant, int64_t n, int d, int k, int num_cu) {
  const int v = pick_assign_variant<T>(requested_variant, n, d, k);
  if (v == ASSIGN_VALU && valu_fused_applies(d, k)) return 8 * num_cu;
  if (v == ASSIGN_LONGROW) return longrow_max_slots<T>(d, k, num_cu);
  if (v != ASSIGN_ROWSTAT) return 0;
  const size_t lds = rowstat_fused_lds<T>(d, k);
  if (lds > ROWSTAT_FUSED_LDS_MAX) return 0;
  return 2 * num_cu;  // upper bound of the grid = number of partial slots
}

// SUMS false: the same kernels without sums and counts (psums, pcounts, slots unused).
template <typename T, bool SUMS>
static int launch_valu_fused(hipStream_t s, const T *X, const T *xnorm, const T *C,
                             const T *cnorm, int *labels, T *mindist, int64_t n, int d, int k,
                             int num_cu, double *psums, int *pcounts, int *slots, T *D = nullptr,
                             int64_t ldn = 0) {
  int grid = 1;
  const int vw = Mfma<T>::VW;
  const bool aligned = (reinterpret_cast<uintptr_t>(X) & 15) == 0;
  const bool reg = aligned && (d == 4 || d == 8 || d == 16 || d == 32 || d == 64) && d >= vw;
  const int ncopy = SUMS ? valu_fused_copies<T>(d, k, reg) : 1;
  const size_t lds = valu_fused_lds<T>(d, k, SUMS, reg, ncopy);
  // the grid is what the device holds at once of the chosen instance (its registers count too)
#define KM_VF_SETUP(kern)                                                                      \
  KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds));                       \
  grid = valu_fused_grid(n, resident_blocks_per_cu(reinterpret_cast<const void *>(kern), WG, lds), num_cu); \
  if (slots) *slots = grid
  // d is one of the register sizes: the row lives in registers
#define KM_VF(DREG)                                                                        \
  do {                                                                                     \
    auto kern = lloyd_valu_fused_kernel<T, DREG, SUMS>;                                    \
    KM_VF_SETUP(kern);                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WG), lds, s, X, xnorm, C, cnorm, labels,     \
                       mindist, psums, pcounts, n, k, D, ldn, ncopy);                      \
  } while (0)
  // any other d: dot products in registers, KREG >= k of them
#define KM_VA_LAUNCH(DMAX, VEC, KREG)                                                      \
  do {                                                                                     \
    auto kern = lloyd_valu_anyd_kernel<T, DMAX, VEC, KREG, SUMS>;                          \
    KM_VF_SETUP(kern);                                                                     \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WG), lds, s, X, xnorm, C, cnorm, labels,     \
                       mindist, psums, pcounts, n, d, k, D, ldn, ncopy);                   \
  } while (0)
#define KM_VA_K(DMAX, VEC)                       \
  do {                                           \
    if (k <= 4) KM_VA_LAUNCH(DMAX, VEC, 4);      \
    else if (k <= 8) KM_VA_LAUNCH(DMAX, VEC, 8); \
    else KM_VA_LAUNCH(DMAX, VEC, 16);            \
  } while (0)
#define KM_VA(DMAX)                                         \
  do {                                                      \
    if (aligned && d >= vw) KM_VA_K(DMAX, Mfma<T>::VW);     \
    else KM_VA_K(DMAX, 1);                                  \
  } while (0)
  if (reg && d == 4) KM_VF(4);
  else if (reg && d == 8) KM_VF(8);
  else if (reg && d == 16) KM_VF(16);
  else if (reg && d == 32) KM_VF(32);
  else if (reg && d == 64) KM_VF(64);
  else if (d <= 16) KM_VA(16);
  else if (d <= 32) KM_VA(32);
  else if (d <= 48) KM_VA(48);
  else KM_VA(64);
#undef KM_VA
#undef KM_VA_K
#undef KM_VA_LAUNCH
#undef KM_VF
#undef KM_VF_SETUP
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template <typename T>
int launch_assign_accumulate(hipStream_t s, int variant, const T *X, const T *xnorm, const T *C,
                             const T *cnorm, int *labels, T *mindist, int64_t n, int d,
                             int k, int num_cu, double *psums, int *pcounts, int *slots,
                             int *used, StackShape st, int split) {
  // cnorm == nullptr: the kernel computes the centroid norms from C itself
  if (n <= 0 || d < 1 || k < 1) return H2O4GPU_KMEANS_EARG;
  const int v = pick_assign_variant<T>(variant, n, d, k);
  if (used) *used = v;
  if (st.sets > 1 && v != ASSIGN_ROWSTAT) return H2O4GPU_KMEANS_EARG;
  if (v == ASSIGN_VALU && valu_fused_applies(d, k))
    return launch_valu_fused<T, true>(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu,
                                      psums, pcounts, slots);
  if (v == ASSIGN_LONGROW)
    return launch_longrow<T, true>(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu, psums, pcounts,
                                   slots);
  if (v != ASSIGN_ROWSTAT) return H2O4GPU_KMEANS_EARG;
  return RowstatDispatch<T, true>::run(s, X, xnorm, C, cnorm, labels, mindist, n, d, k,
                                       num_cu, psums, pcounts, slots, 0, 0, false, st, split);
}

// The kernel whose operands are staged by direct-to-LDS loads: rows and centroids whole
// numbers of BK-feature stages and 16-byte aligned. Returns 1 when the shape is not its.
template <typename T, int MODE, int BCW, bool WIDE, int BK, int NBUF, bool SPREAD>
static int launch_tiled_dma(hipStream_t s, const T *X, const T *xnorm, const T *C, const T *cnorm,
                            int *labels, T *mindist, T *D, int64_t n, int64_t ldn, int d, int k,
                            bool exact) {
  typedef DmaCfg<T, BCW, WIDE, BK, NBUF> Cfg;
  const uintptr_t bits = reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(C) |
                         reinterpret_cast<uintptr_t>(cnorm);
  if (d % BK != 0 || (bits & 15) != 0 || ((size_t)d * sizeof(T)) % 16 != 0) return 1;
  const int64_t row_tiles = (n + Cfg::BR - 1) / Cfg::BR;
  const int64_t tiles = MODE == 1 ? row_tiles * ((k + Cfg::BC - 1) / Cfg::BC) : row_tiles;
  if (tiles > 2147483647ll) return H2O4GPU_KMEANS_EARG;
  const size_t lds = Cfg::LDS_BYTES;
#define KM_DMA_X(EXACT)                                                                      \
  do {                                                                                       \
    auto kern = assign_tiled_dma_kernel<T, MODE, BCW, EXACT, WIDE, BK, NBUF, SPREAD>;        \
    KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds));                   \
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(Cfg::TPB), lds, s, X, xnorm, C,     \
                       cnorm, labels, mindist, D, n, ldn, d, k);                             \
  } while (0)
  if (d >= 128) exact = true;  // as in launch_tiled_bcw
  if constexpr (MODE == 0 && sizeof(T) == 4) {
    if (exact) KM_DMA_X(true);
    else KM_DMA_X(false);
  } else {
    KM_DMA_X(false);
  }
#undef KM_DMA_X
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template <typename T, int MODE, int BCW, bool WIDE = false, int SPLIT = 0>
static int launch_tiled_bcw(hipStream_t s, const T *X, const T *xnorm, const T *C,
                            const T *cnorm, int *labels, T *mindist, T *D, int64_t n,
                            int64_t ldn, int d, int k, bool exact, void *cparts = nullptr,
                            bool direct = true) {
  typedef TiledCfg<T, BCW, WIDE, SPLIT> Cfg;
  const size_t lds = Cfg::LDS_BYTES;
  if constexpr (SPLIT != 0) {
    // the centroids' parts, once per launch, as the LDS images the kernel stages
    if (!cparts) return H2O4GPU_KMEANS_EARG;
    const int nstage = (d + Cfg::BK - 1) / Cfg::BK, nblocks = (k + Cfg::BC - 1) / Cfg::BC;
    const int64_t items = (int64_t)nblocks * nstage * (Cfg::BC / 32) * 64;
    hipLaunchKernelGGL(split_centroids_kernel, dim3((unsigned)std::min<int64_t>((items + 255) / 256, 4096)),
                       dim3(256), 0, s, reinterpret_cast<const float *>(C), static_cast<uintx4 *>(cparts), k,
                       d, Cfg::BC, nstage, nblocks);
  }
  if constexpr (SPLIT == 0 && BCW == 2) if (direct) {
    // Stage depth, ring size and issue order per shape, each measured against the others and
    // against the kernel that stages through registers in alternating runs on one machine:
    // 128-centroid block, float32: 32 features, 2 buffers (2M x 256, k = 1024: 8.16 against 8.20 ms;
    // 16 features with 3 buffers 8.28); 256-centroid block in a fit: 16 features, 2 buffers, loads
    // spread over the stage (500k x 784, k = 4096: 23.9 against 24.6 ms; in one go 24.4); its
    // transform: in one go (100,000 rows: 5.46 against 5.59 ms; spread 5.57); float64: 16
    // features, 2 buffers (2M x 256, k = 1024: 15.8 against 16.1 ms; 3 buffers 17.6).
    int rc = 1;
    if constexpr (sizeof(T) == 8)
      rc = launch_tiled_dma<T, MODE, BCW, WIDE, 16, 2, false>(s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn,
                                                              d, k, exact);
    else if constexpr (!WIDE)
      rc = launch_tiled_dma<T, MODE, BCW, WIDE, 32, 2, false>(s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn,
                                                              d, k, exact);
    else
      rc = launch_tiled_dma<T, MODE, BCW, WIDE, 16, 2, MODE == 0>(s, X, xnorm, C, cnorm, labels, mindist, D, n,
                                                                  ldn, d, k, exact);
    if (rc != 1) return rc;
  }
  const int64_t row_tiles = (n + Cfg::BR - 1) / Cfg::BR;
  const int64_t tiles = MODE == 1 ? row_tiles * ((k + Cfg::BC - 1) / Cfg::BC) : row_tiles;
  if (tiles > 2147483647ll) return H2O4GPU_KMEANS_EARG;
  const dim3 grid((unsigned)tiles, 1u);
  const bool vec = d >= Mfma<T>::VW;  // 16-byte loads need element alignment only
  const bool tail = (d % Cfg::BK) != 0;
#define KM_TILED_X(VEC, TAIL, EXACT)                                                         \
  do {                                                                                       \
    auto kern = assign_tiled_kernel<T, MODE, VEC, TAIL, BCW, EXACT, WIDE, SPLIT>;            \
    KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds));                   \
    hipLaunchKernelGGL(kern, grid, dim3(Cfg::TPB), lds, s, X, xnorm, C, cnorm, labels,       \
                       mindist, D, n, ldn, d, k, static_cast<const uintx4 *>(cparts));       \
  } while (0)
  // From 128 features on the float32 argmin compares the distances themselves: the
  // epilogue is then about one per cent of the matrix work (2M x 256, k = 1024: 8.30 ->
  // 8.37 ms; 500k x 784, k = 4096: 26.5 -> 26.9 ms), and on data whose distances are
  // close to whole numbers the 16-ulp keys flipped four times as many near-tie rows.
  if (d >= 128) exact = true;
#define KM_TILED(VEC, TAIL)                                      \
  do {                                                           \
    if constexpr (MODE == 0 && sizeof(T) == 4) {                 \
      if (exact) KM_TILED_X(VEC, TAIL, true);                    \
      else KM_TILED_X(VEC, TAIL, false);                         \
    } else {                                                     \
      KM_TILED_X(VEC, TAIL, false);                              \
    }                                                            \
  } while (0)
  if (vec && !tail) KM_TILED(true, false);
  else if (vec) KM_TILED(true, true);
  else if constexpr (SPLIT == 0) KM_TILED(false, true);
  else return H2O4GPU_KMEANS_EARG;
#undef KM_TILED
#undef KM_TILED_X
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// The shapes of the tiled kernel that take the bfloat16-parts option: float32 rows fetched
// as 16-byte vectors, more than 64 centroids (below that the kernel waits for memory, not
// for the matrix pipe).
template <typename T>
static int tiled_split(int split, int d, int k) {
  if (sizeof(T) != 4 || (split != 6 && split != 9)) return 0;
  if (d < Mfma<T>::VW || k <= 64) return 0;
  return split;
}

// Bytes of device scratch the tiled kernel needs for the centroids' parts (0: the option
// does not apply to the shape).
// (with the parts the 256-centroid block is ahead whenever it has the centroids to fill it:
// 2M x 256, k = 1024 5.87 -> 5.37 ms, 500k x 784, k = 4096 14.96 -> 13.52 ms)
static bool tiled_split_wide(int k) { return k > 128; }
template <typename T>
size_t tiled_split_scratch_bytes(int split, int d, int k) {
  if (tiled_split<T>(split, d, k) == 0) return 0;
  const int bc = tiled_split_wide(k) ? 256 : 128;
  return (size_t)((k + bc - 1) / bc) * bc * ((d + 15) / 16) * 16 * 6;
}
template size_t tiled_split_scratch_bytes<float>(int, int, int);
template size_t tiled_split_scratch_bytes<double>(int, int, int);

template <typename T, int MODE>
static int launch_tiled(hipStream_t s, const T *X, const T *xnorm, const T *C,
                        const T *cnorm, int *labels, T *mindist, T *D, int64_t n,
                        int64_t ldn, int d, int k, bool exact = false, int split = 0,
                        SplitScratch scratch = SplitScratch()) {
  const bool direct = !scratch.through_registers;
  if constexpr (sizeof(T) == 4) {
    const bool wide = tiled_split_wide(k);
    const size_t need = tiled_split_scratch_bytes<T>(split, d, k);
    void *split_scratch = scratch.ptr;
    switch (need > 0 && scratch.ptr && scratch.bytes >= need ? split : 0) {
#define KM_TILED_SPLIT(SP)                                                                         \
  case SP:                                                                                         \
    if (wide)                                                                                      \
      return launch_tiled_bcw<T, MODE, 2, true, SP>(s, X, xnorm, C, cnorm, labels, mindist, D, n,  \
                                                    ldn, d, k, exact, split_scratch);              \
    return launch_tiled_bcw<T, MODE, 2, false, SP>(s, X, xnorm, C, cnorm, labels, mindist, D, n,   \
                                                   ldn, d, k, exact, split_scratch)
      KM_TILED_SPLIT(6);
      KM_TILED_SPLIT(9);
#undef KM_TILED_SPLIT
    }
  }
  // Measured at 2M x 256, k = 1024 and 500k x 784, k = 4096: two 4-wave workgroups per CU
  // (BCW = 2) beat one 8-wave workgroup with the wider centroid block (BCW = 4) by 5-10 %,
  // so the 128-centroid form is used for large models. Up to 64 centroids a 64-wide block
  // (two wavefronts) halves the matrix work spent on padding; such shapes are bandwidth-bound.
  if (k <= 64)
    return launch_tiled_bcw<T, MODE, 1>(s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn, d, k, exact);
  // A float32 model beyond one XCD's 4 MB of L2 (500k x 784, k = 4096: 12.8 MB): the centroid
  // stream misses L2 as well as the row slices, and the 256-centroid block, which passes over
  // a workgroup's row slice half as often, is ahead (26.9 -> 26.3 ms, 53 -> 30 GB through the
  // L2 miss path); while the model fits L2 it is behind (2M x 256, k = 1024: 8.37 -> 8.53 ms).
  if constexpr (sizeof(T) == 4) {
    if ((size_t)k * d * sizeof(T) > ((size_t)4 << 20))
      return launch_tiled_bcw<T, MODE, 2, true>(s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn, d, k, exact,
                                                nullptr, direct);
    // With the operands staged by direct loads the 256-centroid block is ahead for models that
    // stay in L2 as well (2M x 256, k = 1024: 7.95 against 8.11 ms in alternating runs): half as
    // many bytes fetched and read back from LDS per matrix instruction. Taken whenever its
    // padding of the model costs nothing (or next to nothing) over the 128-centroid block's.
    const uintptr_t bits = reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(C) |
                           reinterpret_cast<uintptr_t>(cnorm);
    const int64_t pad256 = ((int64_t)k + 255) / 256 * 256, pad128 = ((int64_t)k + 127) / 128 * 128;
    if (direct && MODE == 0 && d % 16 == 0 && (bits & 15) == 0 && pad256 * 50 <= pad128 * 51)
      return launch_tiled_bcw<T, MODE, 2, true>(s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn, d, k, exact,
                                                nullptr, true);
  }
  return launch_tiled_bcw<T, MODE, 2>(s, X, xnorm, C, cnorm, labels, mindist, D, n, ldn, d, k, exact, nullptr,
                                      direct);
}

template <typename T>
int launch_assign(hipStream_t s, int variant, const T *X, const T *xnorm,
                  const T *C, const T *cnorm, int *labels, T *mindist, int64_t n,
                  int d, int k, int num_cu, int *used, bool exact, StackShape st, int split,
                  SplitScratch split_scratch) {
  if (n <= 0) return 0;
  if (d < 1 || k < 1) return H2O4GPU_KMEANS_EARG;
  const int v = pick_assign_variant<T>(variant, n, d, k);
  if (v < 0) return H2O4GPU_KMEANS_EARG;
  if (used) *used = v;
  if (st.sets > 1) {  // stacked sets: the row-stationary kernel with the whole model in LDS
    if (v != ASSIGN_ROWSTAT || rowstat_chunk<T>(d, k) < k || !mindist) return H2O4GPU_KMEANS_EARG;
    return RowstatDispatch<T, false>::run(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu,
                                          nullptr, nullptr, nullptr, 0, 0, exact, st, split);
  }
  switch (v) {
    case ASSIGN_VALU:
      // The staged kernels of the fused step, minus the sums: the one-thread-per-row
      // kernel with its strided loads takes two to three times as long (8M x 32, k = 8:
      // 0.68 vs 0.23 ms) except for rows of a few values, where staging does not pay.
      if (valu_fused_applies(d, k) && (d >= 8 || d * sizeof(T) == 32))
        return launch_valu_fused<T, false>(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu,
                                           nullptr, nullptr, nullptr);
      return launch_valu<T, 0>(s, X, xnorm, C, cnorm, labels, mindist, nullptr, n, n, d, k);
    case ASSIGN_ROWSTAT: {
      // (the staged bfloat16 parts are half as large again as the floats: smaller chunks)
      const int split_dp = rowstat_dp<T>(d);
      const bool split_ok = sizeof(T) == 4 && (split == 6 || split == 9) && !exact && split_dp >= 16 &&
                            split_dp <= 64 && d >= Mfma<T>::VW;
      const int kc = rowstat_chunk<T>(d, k, split_ok ? split : 0);
      if (kc < k && !mindist) {  // merging chunks needs the running minimum in memory
        if (used) *used = ASSIGN_TILED;
        return launch_tiled<T, 0>(s, X, xnorm, C, cnorm, labels, mindist, nullptr, n, n, d, k, exact, split,
                                  split_scratch);
      }
      for (int c0 = 0; c0 < k; c0 += kc)
        KM_TRY((RowstatDispatch<T, false>::run(s, X, xnorm, C + (size_t)c0 * d, cnorm + c0, labels,
                                               mindist, n, d, min(kc, k - c0), num_cu, nullptr,
                                               nullptr, nullptr, c0, c0 > 0, exact, StackShape(),
                                               split)));
      return 0;
    }
    case ASSIGN_TILED:
      return launch_tiled<T, 0>(s, X, xnorm, C, cnorm, labels, mindist, nullptr, n, n, d, k, exact, split,
                                split_scratch);
    case ASSIGN_LONGROW:
      return launch_longrow<T, false>(s, X, xnorm, C, cnorm, labels, mindist, n, d, k, num_cu, nullptr,
                                      nullptr, nullptr);
  }
  return H2O4GPU_KMEANS_EARG;
}

template <typename T>
int launch_transform(hipStream_t s, const T *X, const T *xnorm, const T *C,
                     const T *cnorm, T *D, int64_t n, int64_t ldn, int d, int k,
                     int num_cu, int split, SplitScratch split_scratch) {
  if (n <= 0) return 0;
  if (d < 1 || k < 1) return H2O4GPU_KMEANS_EARG;
  if (k <= 16 && d <= 64) {
    // the staged kernels of the small-shape Lloyd step (coalesced 16-byte loads of the rows,
    // scalar-order arithmetic) with every distance stored; rows of a few values keep the
    // one-thread-per-row kernel, as in launch_assign
    if (valu_fused_applies(d, k) && (d >= 8 || d * sizeof(T) == 32))
      return launch_valu_fused<T, false>(s, X, xnorm, C, cnorm, nullptr, nullptr, n, d, k, num_cu,
                                         nullptr, nullptr, nullptr, D, ldn);
    return launch_valu<T, 1>(s, X, xnorm, C, cnorm, nullptr, nullptr, D, n, ldn, d, k);
  }
  return launch_tiled<T, 1>(s, X, xnorm, C, cnorm, nullptr, nullptr, D, n, ldn, d, k, false, split,
                            split_scratch);
}

template <typename T>
int assign_split_products(int variant, int split, int64_t n, int d, int k, bool fused) {
  const int v = pick_assign_variant<T>(variant, n, d, k);
  if (v == ASSIGN_TILED) return fused ? 0 : tiled_split<T>(split, d, k);
  if (v != ASSIGN_ROWSTAT) return 0;
  if (fused) return rowstat_split<T>(split, d, k, true);
  const int dp = rowstat_dp<T>(d);
  if (sizeof(T) != 4 || (split != 6 && split != 9) || dp < 16 || dp > 64 || d < Mfma<T>::VW) return 0;
  const int kc = rowstat_chunk<T>(d, k, split);  // (a chunked sweep runs every chunk the same way)
  return rowstat_split<T>(split, d, kc < k ? kc : k, false);
}
template int assign_split_products<float>(int, int, int64_t, int, int, bool);
template int assign_split_products<double>(int, int, int64_t, int, int, bool);

template int fused_slots<float>(int, int64_t, int, int, int);
template int fused_slots<double>(int, int64_t, int, int, int);
template int launch_assign_accumulate<float>(hipStream_t, int, const float *, const float *,
                                             const float *, const float *, int *, float *,
                                             int64_t, int, int, int, double *, int *, int *,
                                             int *, StackShape, int);
template int launch_assign_accumulate<double>(hipStream_t, int, const double *, const double *,
                                              const double *, const double *, int *, double *,
                                              int64_t, int, int, int, double *, int *, int *,
                                              int *, StackShape, int);
template int pick_assign_variant<float>(int, int64_t, int, int);
template int pick_assign_variant<double>(int, int64_t, int, int);
template int launch_assign<float>(hipStream_t, int, const float *, const float *,
                                  const float *, const float *, int *, float *,
                                  int64_t, int, int, int, int *, bool, StackShape, int, SplitScratch);
template int launch_assign<double>(hipStream_t, int, const double *, const double *,
                                   const double *, const double *, int *, double *,
                                   int64_t, int, int, int, int *, bool, StackShape, int, SplitScratch);
template int launch_transform<float>(hipStream_t, const float *, const float *,
                                     const float *, const float *, float *, int64_t,
                                     int64_t, int, int, int, int, SplitScratch);
template int launch_transform<double>(hipStream_t, const double *, const double *,
                                      const double *, const double *, double *,
                                      int64_t, int64_t, int, int, int, int, SplitScratch);

}  // namespace kmhip
