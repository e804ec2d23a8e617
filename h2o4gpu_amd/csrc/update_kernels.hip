// Row norms, centroid update and reductions.
//
// The centroid update replaces the reference's find_centroids
// (src/gpu/kmeans/kmeans_centroids.h:108-189: copy old centroids, sort (label,
// index) pairs, zero, 30-block run-length accumulate with global atomics,
// revert empties, scale) by
//   pass 1  accumulate : every workgroup owns a contiguous block of rows and a
//           chunk of centroids, keeps that chunk's sums and counts in LDS and
//           writes them to its own slot of a partials buffer (no global
//           atomics, no sort);
//   pass 2  finalize   : sums the slots in slot order, applies the reference's
//           rules (count < 1 keeps the old centroid; mean = sum * (1/count)),
//           and emits per-block partials of sum((old-new)^2);
//   pass 3  post_update: centroid norms for the next assign and the ordered
//           sum of the shift partials.
#include "kmeans_common.h"

namespace kmhip {

static constexpr int WG = 256;

// Sums are kept in double in LDS for both precisions and added with ds_add_f64:
// measured on gfx950, ds_add_f32 retires about 0.33 lane-operations per clock
// per CU whatever the address pattern, ds_add_f64 about 8. As a side effect a
// float32 column whose values span fewer than ~14 binades is summed exactly, so
// the result does not depend on the order in which wavefronts arrive.
__device__ __forceinline__ void lds_add(double *p, double v) { unsafeAtomicAdd(p, v); }

// 2 or 4 consecutive row values as one load. The types are aligned to their elements
// only: a row of d values starts wherever it starts, and gfx950 serves such a load with
// one instruction.
template <typename T, int VEC>
struct VecOf;
template <> struct VecOf<float, 4> { typedef float type __attribute__((ext_vector_type(4), aligned(4))); };
template <> struct VecOf<float, 2> { typedef float type __attribute__((ext_vector_type(2), aligned(4))); };
template <> struct VecOf<double, 2> { typedef double type __attribute__((ext_vector_type(2), aligned(8))); };

template <typename T, int VEC>
struct RowVec {
  typedef typename VecOf<T, VEC>::type type;
};
template <typename T>
struct RowVec<T, 1> {
  typedef T type;
};
template <typename T, int VEC>
__device__ __forceinline__ typename RowVec<T, VEC>::type load_vec(const T *p) {
  return *reinterpret_cast<const typename RowVec<T, VEC>::type *>(p);
}
// ---------------------------------------------------------------------------
// out[i] = sum_j X[i][j]^2, j ascending, multiply and add rounded separately
// (what self_dots does, kmeans_labels.h:187-199). One thread per row; used once
// per fit on the data and on k rows per iteration.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WG) void row_norms_kernel(const T *__restrict__ X,
                                                      T *__restrict__ out,
                                                      int64_t n, int d) {
#pragma clang fp contract(off)
  const int64_t i = (int64_t)blockIdx.x * WG + threadIdx.x;
  if (i >= n) return;
  const T *x = X + i * (int64_t)d;
  T acc = 0;
  for (int j = 0; j < d; j++) {
    const T v = x[j];
    acc = acc + v * v;
  }
  out[i] = acc;
}

// Same result, but a group of LPR lanes cooperates on a row so that global
// loads are coalesced; the partial products are exchanged and then added in j
// order by one lane, which keeps the sum bit-identical to the scalar loop.
// Used for the large one-off pass over the data (d <= 64 * VEC).
template <typename T, int LPR>
__global__ __launch_bounds__(WG) void row_norms_coalesced_kernel(
    const T *__restrict__ X, T *__restrict__ out, int64_t n, int d) {
#pragma clang fp contract(off)
  constexpr int ROWS = WG / LPR;
  __shared__ T sq[ROWS][LPR + 1];
  const int sub = threadIdx.x / LPR, col = threadIdx.x % LPR;
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;
  const int64_t row = row0 + sub;
  T acc = 0;
  for (int j0 = 0; j0 < d; j0 += LPR) {
    const int j = j0 + col;
    T v = (row < n && j < d) ? X[row * (int64_t)d + j] : (T)0;
    sq[sub][col] = v * v;
    __syncthreads();
    if (col == 0) {
      const int lim = min(LPR, d - j0);
      for (int e = 0; e < lim; e++) acc = acc + sq[sub][e];
    }
    __syncthreads();
  }
  if (col == 0 && row < n) out[row] = acc;
}

// Same result for short rows (d <= 64) of a large matrix: a block of 256 rows is one
// contiguous run of 256*d values, fetched as a flat array of 16-byte vectors (the block
// starts on a 16-byte boundary whatever d is; VEC = 1 for data that is not 16-byte aligned)
// into LDS with an odd row stride, and every thread then sums its own row in j order.
template <typename T, int VEC>
__global__ __launch_bounds__(WG) void row_norms_staged_kernel(const T *__restrict__ X,
                                                             T *__restrict__ out, int64_t n, int d) {
#pragma clang fp contract(off)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *Xs = reinterpret_cast<T *>(smem_raw);  // [WG][sx]
  typedef typename RowVec<T, VEC>::type ld_t;
  int sx = d | 1;
  if (((sx + 1) & sx) == 0) sx += 2;  // never 2^m - 1 (measured slow as an LDS row stride)
  const int pad = sx - d;
  const int tid = threadIdx.x;
  const unsigned dinv = d > 1 ? 0xFFFFFFFFu / (unsigned)d + 1u : 0u;  // el / d by multiply-high
  auto row_of = [&](int el) -> int { return d > 1 ? (int)__umulhi((unsigned)el, dinv) : el; };
  for (int64_t base = (int64_t)blockIdx.x * WG; base < n; base += (int64_t)gridDim.x * WG) {
    const int rows = (int)min<int64_t>(WG, n - base);
    const T *xb = X + base * (int64_t)d;
    const int total = rows * d;     // values of this block
    const int nvec = total / VEC;   // complete vectors
    __syncthreads();                // the previous block has been consumed
    for (int e = tid; e < nvec; e += WG) {
      const ld_t v = *reinterpret_cast<const ld_t *>(xb + (size_t)e * VEC);
      const int el = e * VEC;
      if constexpr (VEC == 1) {
        Xs[el + row_of(el) * pad] = v;
      } else {
#pragma unroll
        for (int q = 0; q < VEC; q++) Xs[el + q + row_of(el + q) * pad] = v[q];
      }
    }
    if (tid < total - nvec * VEC) {  // values behind the last complete vector of the data set
      const int el = nvec * VEC + tid;
      Xs[el + row_of(el) * pad] = xb[el];
    }
    __syncthreads();
    if (tid < rows) {
      const T *x = Xs + tid * sx;
      T acc = 0;
      for (int j = 0; j < d; j++) {
        const T v = x[j];
        acc = acc + v * v;
      }
      out[base + tid] = acc;
    }
  }
}

template <typename T>
int launch_row_norms(hipStream_t s, const T *X, T *out, int64_t n, int d) {
  if (n <= 0) return 0;
  if (d >= 4 && d <= 64 && n * (int64_t)d >= (1 << 22)) {
    int sx = d | 1;
    if (((sx + 1) & sx) == 0) sx += 2;
    const size_t lds = (size_t)WG * sx * sizeof(T);
    int64_t grid = (n + WG - 1) / WG;
    if (grid > 256 * 8) grid = 256 * 8;
    constexpr int VW = 16 / sizeof(T);
    if ((reinterpret_cast<uintptr_t>(X) & 15) == 0)
      hipLaunchKernelGGL((row_norms_staged_kernel<T, VW>), dim3((unsigned)grid), dim3(WG), lds, s, X, out,
                         n, d);
    else
      hipLaunchKernelGGL((row_norms_staged_kernel<T, 1>), dim3((unsigned)grid), dim3(WG), lds, s, X, out,
                         n, d);
    KM_HIP_TRY(hipGetLastError());
    return 0;
  }
  // (a thread per row is enough for a handful of short rows; long rows always go
  // through the cooperative kernel, a single thread would walk them serially)
  if (d >= 8 && (n * (int64_t)d >= 65536 || d >= 64)) {
    if (d <= 16) {
      constexpr int LPR = 16;
      hipLaunchKernelGGL((row_norms_coalesced_kernel<T, LPR>),
                         dim3((unsigned)((n + WG / LPR - 1) / (WG / LPR))), dim3(WG), 0,
                         s, X, out, n, d);
    } else if (d <= 32) {
      constexpr int LPR = 32;
      hipLaunchKernelGGL((row_norms_coalesced_kernel<T, LPR>),
                         dim3((unsigned)((n + WG / LPR - 1) / (WG / LPR))), dim3(WG), 0,
                         s, X, out, n, d);
    } else {
      constexpr int LPR = 64;
      hipLaunchKernelGGL((row_norms_coalesced_kernel<T, LPR>),
                         dim3((unsigned)((n + WG / LPR - 1) / (WG / LPR))), dim3(WG), 0,
                         s, X, out, n, d);
    }
  } else {
    hipLaunchKernelGGL((row_norms_kernel<T>), dim3((unsigned)((n + WG - 1) / WG)),
                       dim3(WG), 0, s, X, out, n, d);
  }
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// ---------------------------------------------------------------------------
// pass 1: accumulate
// grid (row_blocks, k_chunks). LDS: sums[kc][d] + counts[kc].
// A wavefront reads 64 labels at a time, then serves the matching rows one
// group at a time: LPR lanes (each VEC consecutive features per step) per row,
// 64/LPR rows in flight. With a single centroid chunk every row matches and
// the ballot is skipped.
// ---------------------------------------------------------------------------
// adds elements first .. VEC-1 of v to dst[first .. VEC-1]
template <typename T, int VEC, bool RAGGED>
__device__ __forceinline__ void lds_add_vec(double *dst, typename RowVec<T, VEC>::type v, int first) {
  if constexpr (VEC == 1) {
    lds_add(dst, (double)v);
  } else {
#pragma unroll
    for (int e = 0; e < VEC; e++)
      if (!RAGGED || e >= first) lds_add(dst + e, (double)v[e]);
  }
}

// RAGGED: d is not a multiple of VEC (d >= VEC). The vector that would reach past the end
// of the row is fetched from the row's last VEC values instead, and only the elements the
// lane is responsible for (from `first` on) are added.
template <typename T, int VEC, bool RAGGED>
__device__ __forceinline__ void add_row_slice(double *srow, const T *xrow, int col,
                                              int lpr, int d) {
  // lanes col, col+lpr, ... each take VEC consecutive features; four loads are issued
  // before the first add (a load past the end of the row is clamped into it and unused;
  // eight in flight measured slower: short rows then mostly fetch clamped duplicates)
  constexpr int U = 4;
  const int step = lpr * VEC;
  for (int j0 = col * VEC; j0 < d; j0 += U * step) {
    typename RowVec<T, VEC>::type v[U];
    int jc[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      jc[u] = VEC > 1 ? min(j0 + u * step, d - VEC) : min(j0 + u * step, d - 1);
      v[u] = load_vec<T, VEC>(xrow + jc[u]);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int j = j0 + u * step;
      if (j < d) lds_add_vec<T, VEC, RAGGED>(srow + jc[u], v[u], j - jc[u]);
    }
  }
}

// sd = LDS row stride of the sums (>= d): chosen odd-ish by the host so that
// rows of different centroids do not all start on the same bank.
template <typename T, int VEC, bool RAGGED, int TPB>
__global__ __launch_bounds__(TPB) void accumulate_kernel(
    const T *__restrict__ X, const int *__restrict__ labels,
    double *__restrict__ psums, int *__restrict__ pcounts, int64_t n, int d, int k,
    int kc, int64_t rows_per_block, int lpr, int sd) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  double *sums = reinterpret_cast<double *>(smem_raw);         // [kc][sd]
  int *cnt = reinterpret_cast<int *>(sums + (size_t)kc * sd);  // [kc]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int k0 = blockIdx.y * kc;
  const int nk = min(kc, k - k0);
  for (int e = tid; e < nk * sd; e += TPB) sums[e] = 0.0;
  for (int c = tid; c < nk; c += TPB) cnt[c] = 0;
  __syncthreads();

  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int64_t r1 = min(n, r0 + rows_per_block);
  const int rps = 64 / lpr;  // rows served per wavefront step
  const int sub = lane / lpr, col = lane % lpr;
  const bool single_chunk = gridDim.y == 1;
  const bool narrow = d <= lpr * VEC;  // one vector per lane covers a row
  constexpr int U = 8;

  for (int64_t g0 = r0 + (int64_t)wave * 64; g0 < r1; g0 += (TPB / 64) * 64) {
    const int64_t myrow = g0 + lane;
    int lab = -1;
    if (myrow < r1) lab = labels[myrow] - k0;
    const bool match = lab >= 0 && lab < nk;
    if (match) atomicAdd(&cnt[lab], 1);
    if (single_chunk && narrow) {
      // all loads of U row groups are issued before the first LDS add
      const bool has = col * VEC < d;
      const int jc = RAGGED ? min(col * VEC, d - VEC) : col * VEC;  // see add_row_slice
      const int first = col * VEC - jc;
      for (int b = 0; b < 64; b += rps * U) {
        typename RowVec<T, VEC>::type v[U];
        int l[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          const int src = b + u * rps + sub;
          l[u] = src < 64 ? __shfl(lab, src & 63, 64) : -1;
          const int64_t row = g0 + src;
          if (!(l[u] >= 0 && l[u] < nk && row < r1 && has)) l[u] = -1;
          v[u] = load_vec<T, VEC>(X + (l[u] >= 0 ? row : r0) * (int64_t)d + (has ? jc : 0));
        }
#pragma unroll
        for (int u = 0; u < U; u++)
          if (l[u] >= 0) lds_add_vec<T, VEC, RAGGED>(sums + (size_t)l[u] * sd + jc, v[u], first);
      }
    } else if (single_chunk) {
      for (int b = 0; b < 64; b += rps) {
        const int src = b + sub;
        const int l = __shfl(lab, src, 64);
        const int64_t row = g0 + src;
        if (l >= 0 && l < nk && row < r1)
          add_row_slice<T, VEC, RAGGED>(sums + (size_t)l * sd, X + row * (int64_t)d, col, lpr, d);
      }
    } else {
      unsigned long long mask = __ballot(match);
      while (mask) {
        // take up to rps set bits; sub-group `sub` serves the sub-th of them
        int src = -1;
        unsigned long long m = mask;
        for (int q = 0; q < rps; q++) {
          if (!m) break;
          const int b = __ffsll((long long)m) - 1;
          if (q == sub) src = b;
          m &= m - 1;
        }
        mask = m;
        const int l = __shfl(lab, src < 0 ? 0 : src, 64);
        if (src >= 0) {
          const int64_t row = g0 + src;
          add_row_slice<T, VEC, RAGGED>(sums + (size_t)l * sd, X + row * (int64_t)d, col, lpr, d);
        }
      }
    }
  }
  __syncthreads();
  double *dst = psums + ((size_t)blockIdx.x * k + k0) * d;
  for (int e = tid; e < nk * d; e += TPB) {
    const int c = e / d, j = e - c * d;
    dst[e] = sums[(size_t)c * sd + j];
  }
  int *cdst = pcounts + (size_t)blockIdx.x * k + k0;
  for (int c = tid; c < nk; c += TPB) cdst[c] = cnt[c];
}

// LDS row stride of the sums (in doubles): odd, so that the rows of different
// centroids start on different banks.
static int update_lds_stride(int d) { return d | 1; }
static constexpr size_t UPDATE_LDS_MAX = 150 * 1024;
static constexpr int KM_MAX_LDS_CHUNKS = 8;

template <typename T>
UpdatePlan plan_update(int64_t n, int d, int k, int num_cu) {
  UpdatePlan p;
  p.sd = update_lds_stride(d);
  const size_t per_centroid = (size_t)p.sd * sizeof(double) + sizeof(int);
  // As few balanced chunks of centroids as a CU's LDS allows (one 1024-thread workgroup
  // per CU when a chunk is large). Every chunk scans all labels and reads the rows that
  // fall into it, so X is read once in total.
  int kc = (int)(UPDATE_LDS_MAX / per_centroid);
  if (kc < 1) kc = 1;
  if (kc > k) kc = k;
  p.k_chunks = (k + kc - 1) / kc;
  kc = (k + p.k_chunks - 1) / p.k_chunks;  // balanced chunks
  p.kc = kc;
  p.lds_bytes = (size_t)kc * per_centroid;
  p.vec = sizeof(T) == 4 ? (d >= 4 ? 4 : (d >= 2 ? 2 : 1)) : (d >= 2 ? 2 : 1);  // see launch_accumulate
  // enough workgroups to cover the machine a few times, but bounded so the
  // partials buffer (row_blocks * k * d) stays small next to the data
  // (fewer when a workgroup's LDS image leaves room for only one or two per CU)
  // An LDS image above 40 KB leaves room for at most three 4-wave workgroups per CU: one
  // 16-wave workgroup per CU then keeps more loads in flight (500k x 784, k = 10, 63 KB:
  // 0.48 -> 0.43 ms); below that, four 4-wave workgroups per CU.
  const bool wide = p.lds_bytes > 40 * 1024;
  p.threads = wide ? 1024 : 256;
  const int per_cu = wide ? 1 : 4;
  int64_t want = (int64_t)num_cu * per_cu / p.k_chunks;
  if (want < 1) want = 1;
  int64_t max_by_rows = (n + 1023) / 1024;  // at least 1024 rows per block
  if (max_by_rows < 1) max_by_rows = 1;
  if (want > max_by_rows) want = max_by_rows;
  // partials traffic 2*rb*k*d should stay below ~1/8 of the data n*d
  int64_t max_by_bytes = n / ((int64_t)16 * k);
  if (max_by_bytes < 1) max_by_bytes = 1;
  if (want > max_by_bytes) want = max_by_bytes;
  p.row_blocks = (int)want;
  return p;
}

template <typename T, int VEC, bool RAGGED>
static int launch_accumulate_vec(hipStream_t s, const UpdatePlan &p, const T *X,
                                 const int *labels, double *psums, int *pcounts,
                                 int64_t n, int d, int k) {
  const int64_t rows_per_block = ((n + p.row_blocks - 1) / p.row_blocks + 63) / 64 * 64;
  int groups = (d + VEC - 1) / VEC;  // lanes wanted per row
  int lpr = 1;
  while (lpr < groups && lpr < 64) lpr <<= 1;
  // workgroup size from the plan: 16 wavefronts when only one workgroup fits a CU
#define KM_ACC_LAUNCH(TPB)                                                                      \
  do {                                                                                          \
    auto kern = accumulate_kernel<T, VEC, RAGGED, TPB>;                                         \
    KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(kern), p.lds_bytes));              \
    hipLaunchKernelGGL(kern, dim3(p.row_blocks, p.k_chunks), dim3(TPB), p.lds_bytes, s, X,      \
                       labels, psums, pcounts, n, d, k, p.kc, rows_per_block, lpr, p.sd);       \
  } while (0)
  if (p.threads == 1024) KM_ACC_LAUNCH(1024);
  else KM_ACC_LAUNCH(256);
#undef KM_ACC_LAUNCH
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// Lanes take 16 bytes of a row each wherever a row holds that much (8 bytes for float rows
// of 2 or 3 values); the rows need element alignment only.
template <>
int launch_accumulate<float>(hipStream_t s, const UpdatePlan &p, const float *X,
                             const int *labels, double *psums, int *pcounts,
                             int64_t n, int d, int k) {
  if (d >= 4 && d % 4 == 0) return launch_accumulate_vec<float, 4, false>(s, p, X, labels, psums, pcounts, n, d, k);
  if (d >= 4) return launch_accumulate_vec<float, 4, true>(s, p, X, labels, psums, pcounts, n, d, k);
  if (d == 2) return launch_accumulate_vec<float, 2, false>(s, p, X, labels, psums, pcounts, n, d, k);
  if (d == 3) return launch_accumulate_vec<float, 2, true>(s, p, X, labels, psums, pcounts, n, d, k);
  return launch_accumulate_vec<float, 1, false>(s, p, X, labels, psums, pcounts, n, d, k);
}
template <>
int launch_accumulate<double>(hipStream_t s, const UpdatePlan &p, const double *X,
                              const int *labels, double *psums, int *pcounts,
                              int64_t n, int d, int k) {
  if (d >= 2 && d % 2 == 0) return launch_accumulate_vec<double, 2, false>(s, p, X, labels, psums, pcounts, n, d, k);
  if (d >= 2) return launch_accumulate_vec<double, 2, true>(s, p, X, labels, psums, pcounts, n, d, k);
  return launch_accumulate_vec<double, 1, false>(s, p, X, labels, psums, pcounts, n, d, k);
}

// ---------------------------------------------------------------------------
// pass 1, large k*d: bucket rows by label, then sum each bucket.
//
// When the per-centroid sums do not fit in LDS the chunked kernel above has to
// scan all labels once per centroid chunk. Instead the rows are ordered by label
// with a stable counting sort and the ordered rows are summed in fixed windows.
// Nothing in it depends on the order in which workgroups or wavefronts run, so the
// sums are the same bit for bit from run to run, in float64 too:
//   histogram : rows per label of every block of rows               [blocks][k]
//   scan      : per label, exclusive sum over the blocks (two levels), bucket
//               sizes, and the exclusive sum of those over the labels
//   scatter   : position of a row = start of its label's bucket + rows of that
//               label in earlier blocks + rows of that label earlier in its own
//               block (each wavefront walks a contiguous quarter of the block in
//               row order and ranks 64 rows at a time with ballots)
//   window sum: a wavefront sums WPOS consecutive positions of the ordered rows in
//               registers, lanes across features, and stores the sum of every run
//               of equal labels to a slot of its own (window + label: the index
//               grows by at least one from each run to the next, so no two runs
//               share a slot and nothing is added atomically)
//   bucket sum: per label, the slots of its windows are added in window order by
//               four strands with a fixed tree.
// Replaces the reference's sort_by_key + calculate_centroids
// (kmeans_centroids.h:40-75, 131), whose atomic adds arrive in no fixed order.
// ---------------------------------------------------------------------------
static constexpr int BUCKET_ROWS_MIN = 4096;  // rows per block of the histogram / scatter
static constexpr int BUCKET_MAX_BLOCKS = 2048;
static constexpr int BUCKET_SEGS = 32;        // block segments of the two-level scan

int64_t bucket_rows_per_block(int64_t n) {
  int64_t rpb = (n + BUCKET_MAX_BLOCKS - 1) / BUCKET_MAX_BLOCKS;
  rpb = (rpb + 255) / 256 * 256;
  return rpb < BUCKET_ROWS_MIN ? BUCKET_ROWS_MIN : rpb;
}
int bucket_blocks(int64_t n) { return (int)((n + bucket_rows_per_block(n) - 1) / bucket_rows_per_block(n)); }
// wavefronts per scatter workgroup: each keeps its own [k] counters in LDS
static int bucket_waves(int k) {
  if ((size_t)4 * k * sizeof(int) <= 128 * 1024) return 4;
  if ((size_t)2 * k * sizeof(int) <= 128 * 1024) return 2;
  return 1;
}
// positions per window of the window sum: 128 once there are enough windows to fill the GPU
int bucket_window(int64_t n) { return n >= (int64_t)1 << 20 ? 128 : 64; }
size_t bucket_partial_slots(int64_t n, int k) { return (size_t)(n / bucket_window(n) + 2) + k; }

__global__ __launch_bounds__(WG) void bucket_hist_kernel(const int *__restrict__ labels,
                                                        int *__restrict__ bh, int64_t n, int k,
                                                        int64_t rpb) {
  extern __shared__ int hist[];  // [k]
  const int tid = threadIdx.x;
  for (int c = tid; c < k; c += WG) hist[c] = 0;
  __syncthreads();
  const int64_t r0 = (int64_t)blockIdx.x * rpb;
  const int64_t r1 = min(n, r0 + rpb);
  for (int64_t i = r0 + tid; i < r1; i += WG) {
    const int l = labels[i];
    if (l >= 0 && l < k) atomicAdd(&hist[l], 1);  // integer counts: order-independent
  }
  __syncthreads();
  int *dst = bh + (size_t)blockIdx.x * k;
  for (int c = tid; c < k; c += WG) dst[c] = hist[c];
}

// Level 1 of the scan over blocks: seg[s][c] = rows of label c in the blocks of segment s.
__global__ __launch_bounds__(WG) void bucket_seg_kernel(const int *__restrict__ bh,
                                                       int *__restrict__ seg, int nb, int k,
                                                       int per_seg) {
  const int c = blockIdx.x * WG + threadIdx.x;
  if (c >= k) return;
  const int b0 = blockIdx.y * per_seg, b1 = min(nb, b0 + per_seg);
  int sum = 0;
  int b = b0;
  for (; b + 4 <= b1; b += 4) {
    const int v0 = bh[(size_t)b * k + c], v1 = bh[(size_t)(b + 1) * k + c];
    const int v2 = bh[(size_t)(b + 2) * k + c], v3 = bh[(size_t)(b + 3) * k + c];
    sum += v0 + v1 + v2 + v3;
  }
  for (; b < b1; b++) sum += bh[(size_t)b * k + c];
  seg[(size_t)blockIdx.y * k + c] = sum;
}
// Level 2: bh[b][c] <- rows of label c in blocks before b; the last segment also leaves the
// bucket size in counts[c].
__global__ __launch_bounds__(WG) void bucket_block_scan_kernel(int *__restrict__ bh,
                                                              const int *__restrict__ seg,
                                                              int *__restrict__ counts, int nb,
                                                              int k, int per_seg) {
  const int c = blockIdx.x * WG + threadIdx.x;
  if (c >= k) return;
  int run = 0;
  for (int s = 0; s < (int)blockIdx.y; s++) run += seg[(size_t)s * k + c];
  const int b0 = blockIdx.y * per_seg, b1 = min(nb, b0 + per_seg);
  int b = b0;
  for (; b + 4 <= b1; b += 4) {
    const int v0 = bh[(size_t)b * k + c], v1 = bh[(size_t)(b + 1) * k + c];
    const int v2 = bh[(size_t)(b + 2) * k + c], v3 = bh[(size_t)(b + 3) * k + c];
    bh[(size_t)b * k + c] = run;
    bh[(size_t)(b + 1) * k + c] = run + v0;
    bh[(size_t)(b + 2) * k + c] = run + v0 + v1;
    bh[(size_t)(b + 3) * k + c] = run + v0 + v1 + v2;
    run += v0 + v1 + v2 + v3;
  }
  for (; b < b1; b++) {
    const int v = bh[(size_t)b * k + c];
    bh[(size_t)b * k + c] = run;
    run += v;
  }
  if (blockIdx.y == gridDim.y - 1) counts[c] = run;
}

// offsets[c] = sum of counts[0..c), *total = sum of all; single workgroup.
__global__ __launch_bounds__(WG) void bucket_scan_kernel(const int *__restrict__ counts,
                                                        int *__restrict__ offsets,
                                                        int *__restrict__ total, int k) {
  __shared__ int part[WG];
  const int tid = threadIdx.x;
  const int per = (k + WG - 1) / WG;
  const int lo = tid * per, hi = min(k, lo + per);
  int s = 0;
  for (int c = lo; c < hi; c++) s += counts[c];
  part[tid] = s;
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int t = 0; t < WG; t++) {
      const int v = part[t];
      part[t] = run;
      run += v;
    }
    *total = run;  // rows that carry a label in [0, k)
  }
  __syncthreads();
  int run = part[tid];
  for (int c = lo; c < hi; c++) {
    offsets[c] = run;
    run += counts[c];
  }
}

// Stable scatter. The workgroup has NWB wavefronts; wavefront w owns rows
// [r0 + w*q, r0 + (w+1)*q) of the block, q = rpb / NWB, and its own counters wh[w][k].
__global__ void bucket_scatter_kernel(const int *__restrict__ labels, const int *__restrict__ bh,
                                      const int *__restrict__ offsets, int *__restrict__ order,
                                      int *__restrict__ order_label, int64_t n, int k, int64_t rpb) {
  extern __shared__ int wh[];  // [NWB][k]
  const int tid = threadIdx.x, tpb = blockDim.x;
  const int nwb = tpb >> 6, wave = tid >> 6, lane = tid & 63;
  for (int e = tid; e < nwb * k; e += tpb) wh[e] = 0;
  __syncthreads();
  const int64_t r0 = (int64_t)blockIdx.x * rpb;
  const int64_t q = rpb / nwb;  // rpb is a multiple of 256
  const int64_t w0 = min(n, r0 + wave * q), w1 = min(n, w0 + q);
  int *mine = wh + (size_t)wave * k;
  for (int64_t i = w0 + lane; i < w1; i += 64) {
    const int l = labels[i];
    if (l >= 0 && l < k) atomicAdd(&mine[l], 1);
  }
  __syncthreads();
  // counters -> first position of (this wavefront, label): bucket start + earlier blocks +
  // earlier wavefronts of this block
  const int *bbase = bh + (size_t)blockIdx.x * k;
  for (int c = tid; c < k; c += tpb) {
    int run = offsets[c] + bbase[c];
    for (int w = 0; w < nwb; w++) {
      const int v = wh[(size_t)w * k + c];
      wh[(size_t)w * k + c] = run;
      run += v;
    }
  }
  __syncthreads();
  // 64 rows at a time, in row order: every lane reads its label's counter, lanes with the
  // same label rank themselves by lane number, the first of them advances the counter
  for (int64_t i0 = w0; i0 < w1; i0 += 64) {
    const int64_t i = i0 + lane;
    const int l = i < w1 ? labels[i] : -1;
    const bool valid = l >= 0 && l < k;
    const int cur = valid ? mine[l] : 0;
    unsigned long long todo = __ballot(valid);
    int pos = -1, cnt = 0;
    bool first = false;
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const int l0 = __shfl(l, leader, 64);
      const unsigned long long same = __ballot(valid && l == l0);
      if (valid && l == l0) {
        pos = cur + __popcll(same & ((1ull << lane) - 1ull));
        cnt = __popcll(same);
        first = lane == leader;
      }
      todo &= ~same;
    }
    if (valid) {
      order[pos] = (int)i;
      order_label[pos] = l;
    }
    if (first) mine[l] = cur + cnt;  // (one lane per label; read again only in the next round)
  }
}

// One wavefront per window of WM*64 consecutive ordered positions; lanes across features
// (VEC each, NVEC vectors per lane cover up to 64*VEC*NVEC features per pass over the rows).
// The sum of every run of equal labels goes to slot (window + label) of P, [slots][d].
template <typename T, int VEC, int NVEC>
__global__ __launch_bounds__(WG) void window_sum_kernel(
    const T *__restrict__ X, const int *__restrict__ order,
    const int *__restrict__ order_label, double *__restrict__ P,
    const int *__restrict__ total, int d, int wm) {
  const int64_t m = *total;
  const int lane = threadIdx.x & 63;
  const int64_t win = (int64_t)blockIdx.x * (WG / 64) + (threadIdx.x >> 6);
  const int64_t wpos0 = win * wm * 64;
  if (wpos0 >= m) return;
  constexpr int SPAN = 64 * VEC * NVEC;
  for (int d0 = 0; d0 < d; d0 += SPAN) {
    double acc[NVEC][VEC];
#pragma unroll
    for (int q = 0; q < NVEC; q++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[q][e] = 0.0;
    // Lane slot q covers features [j, j + VEC). When d is not a multiple of VEC the last
    // such vector would reach past the row: it is fetched from the row's last VEC values
    // instead (offset jc) and only its elements from `first` on belong to this lane.
    int jc[NVEC], first[NVEC];
    bool active[NVEC];
#pragma unroll
    for (int q = 0; q < NVEC; q++) {
      const int j = d0 + (q * 64 + lane) * VEC;
      active[q] = j < d;
      jc[q] = active[q] ? min(j, d - VEC) : 0;
      first[q] = active[q] ? j - jc[q] : 0;
    }
    auto flush = [&](int label) {
      double *dst = P + (size_t)(win + label) * d;
#pragma unroll
      for (int q = 0; q < NVEC; q++) {
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          if (active[q] && e >= first[q]) dst[jc[q] + e] = acc[q][e];
          acc[q][e] = 0.0;
        }
      }
    };
    int cur = -1;
    for (int sub = 0; sub < wm; sub++) {
      const int64_t pos0 = wpos0 + (int64_t)sub * 64;
      if (pos0 >= m) break;
      const int cnt = (int)min<int64_t>(64, m - pos0);
      const int my_row = lane < cnt ? order[pos0 + lane] : 0;
      const int my_lab = lane < cnt ? order_label[pos0 + lane] : -1;
      if (sub == 0) cur = __shfl(my_lab, 0, 64);
      constexpr int U = 4;
      for (int i0 = 0; i0 < cnt; i0 += U) {
        typename RowVec<T, VEC>::type v[U][NVEC];
        int lab[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          const int i = min(i0 + u, cnt - 1);
          const int row = __shfl(my_row, i, 64);
          lab[u] = __shfl(my_lab, i, 64);
          const T *x = X + (int64_t)row * d;
#pragma unroll
          for (int q = 0; q < NVEC; q++) v[u][q] = load_vec<T, VEC>(x + jc[q]);  // inactive: masked below
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
          if (i0 + u >= cnt) break;
          if (lab[u] != cur) {
            flush(cur);
            cur = lab[u];
          }
#pragma unroll
          for (int q = 0; q < NVEC; q++) {
            if (active[q]) {
              if constexpr (VEC == 1) {
                acc[q][0] += (double)v[u][q];
              } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[q][e] += (double)v[u][q][e];
              }
            }
          }
        }
      }
    }
    flush(cur);
  }
}

// gsum[c][j] = sum over the windows of label c's bucket of P[window + c][j], windows in
// ascending order dealt to 4 strands (window w: strand (w - first) % 4), the four strand
// sums then added as ((s0 + s1) + s2) + s3. grid (k, ceil(d / 64)).
__global__ __launch_bounds__(WG) void bucket_sum_kernel(const double *__restrict__ P,
                                                       const int *__restrict__ offsets,
                                                       const int *__restrict__ counts,
                                                       double *__restrict__ gsum, int d, int wpos) {
  __shared__ double part[4][64];
  const int c = blockIdx.x;
  const int f = threadIdx.x & 63, strand = threadIdx.x >> 6;
  const int j = blockIdx.y * 64 + f;
  const int cnt = counts[c], off = offsets[c];
  double s = 0.0;
  if (cnt > 0 && j < d) {
    const int w_first = off / wpos, w_last = (off + cnt - 1) / wpos;
    const double *src = P + (size_t)c * d + j;
    int w = w_first + strand;
    for (; w + 12 <= w_last; w += 16) {
      const double a0 = src[(size_t)w * d], a1 = src[(size_t)(w + 4) * d];
      const double a2 = src[(size_t)(w + 8) * d], a3 = src[(size_t)(w + 12) * d];
      s = s + a0;
      s = s + a1;
      s = s + a2;
      s = s + a3;
    }
    for (; w <= w_last; w += 4) s = s + src[(size_t)w * d];
  }
  part[strand][f] = s;
  __syncthreads();
  if (strand == 0 && j < d) gsum[(size_t)c * d + j] = ((part[0][f] + part[1][f]) + part[2][f]) + part[3][f];
}

size_t bucket_lds_bytes(int k) { return (size_t)bucket_waves(k) * k * sizeof(int); }
bool bucketed_update_applies(int k_chunks, int k, int d) {
  // Measured: up to 8 chunks the LDS kernel is ahead (10M x 32, k = 4096: 0.61 vs 0.83 ms;
  // 8M x 16, k = 8192: 0.40 vs 0.66), from 11 chunks on bucketing is (2M x 256, k = 1024:
  // 0.49 vs 0.62; 500k x 784, k = 256: 0.36 vs 0.52). With a handful of centroids a bucket
  // spans thousands of windows and the per-label sum has no parallelism left, so bucketing
  // is never used while the sums fit LDS.
  (void)d;
  return k_chunks > KM_MAX_LDS_CHUNKS && (size_t)k * sizeof(int) <= 128 * 1024;
}

template <typename T>
int launch_bucketed_accumulate(hipStream_t s, const T *X, const int *labels, int *order,
                               int *order_label, int *offsets, int *block_hist, int *seg_hist,
                               int *total, double *partials, double *gsum, int *counts, int64_t n,
                               int d, int k) {
  const int64_t rpb = bucket_rows_per_block(n);
  const int nb = bucket_blocks(n);
  const int per_seg = (nb + BUCKET_SEGS - 1) / BUCKET_SEGS;
  const int segs = (nb + per_seg - 1) / per_seg;
  const size_t lds1 = (size_t)k * sizeof(int), lds2 = bucket_lds_bytes(k);
  KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(bucket_hist_kernel), lds1));
  KM_TRY(ensure_dynamic_lds(reinterpret_cast<const void *>(bucket_scatter_kernel), lds2));
  const unsigned kblocks = (unsigned)((k + WG - 1) / WG);
  hipLaunchKernelGGL(bucket_hist_kernel, dim3(nb), dim3(WG), lds1, s, labels, block_hist, n, k, rpb);
  hipLaunchKernelGGL(bucket_seg_kernel, dim3(kblocks, segs), dim3(WG), 0, s, block_hist, seg_hist, nb, k,
                     per_seg);
  hipLaunchKernelGGL(bucket_block_scan_kernel, dim3(kblocks, segs), dim3(WG), 0, s, block_hist, seg_hist,
                     counts, nb, k, per_seg);
  hipLaunchKernelGGL(bucket_scan_kernel, dim3(1), dim3(WG), 0, s, counts, offsets, total, k);
  hipLaunchKernelGGL(bucket_scatter_kernel, dim3(nb), dim3(bucket_waves(k) * 64), lds2, s, labels,
                     block_hist, offsets, order, order_label, n, k, rpb);
  // rows with a label outside [0, k) are not bucketed, so the ordered rows may be fewer
  // than n: the grid covers n positions and every wavefront bounds itself by the
  // device-side total
  const int wm = bucket_window(n) / 64;
  const int64_t windows = (n + (int64_t)wm * 64 - 1) / ((int64_t)wm * 64);
  const unsigned sblocks = (unsigned)((windows + WG / 64 - 1) / (WG / 64));
  // 16-byte loads for any d that holds a whole vector (rows need element alignment only)
#define KM_SEG(VEC, NVEC)                                                                  \
  hipLaunchKernelGGL((window_sum_kernel<T, VEC, NVEC>), dim3(sblocks), dim3(WG), 0, s, X, \
                     order, order_label, partials, total, d, wm)
  if constexpr (sizeof(T) == 4) {
    if (d >= 4) {
      if (d <= 256) KM_SEG(4, 1);
      else if (d <= 512) KM_SEG(4, 2);
      else KM_SEG(4, 4);
    } else {
      KM_SEG(1, 4);
    }
  } else {
    if (d >= 2) {
      if (d <= 128) KM_SEG(2, 1);
      else if (d <= 256) KM_SEG(2, 2);
      else KM_SEG(2, 4);
    } else {
      KM_SEG(1, 4);
    }
  }
#undef KM_SEG
  hipLaunchKernelGGL(bucket_sum_kernel, dim3((unsigned)k, (unsigned)((d + 63) / 64)), dim3(WG), 0, s,
                     partials, offsets, counts, gsum, d, wm * 64);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

// ---------------------------------------------------------------------------
// pass 2: finalize. One thread per centroid coordinate.
// ---------------------------------------------------------------------------
// A workgroup takes EPW consecutive coordinates; RS = 256 / EPW thread groups
// each sum a contiguous range of the row-block slots for those coordinates (slot
// order), then group 0 adds the RS range sums in range order. EPW is 32, or 4
// for a small model with many slots, where 32 would leave a handful of
// workgroups walking thousands of slots one after the other.
template <typename T, int EPW>
__global__ __launch_bounds__(WG) void finalize_kernel(
    const double *__restrict__ psums, const int *__restrict__ pcounts, int row_blocks,
    const T *__restrict__ c_old, T *__restrict__ c_new, int *__restrict__ counts,
    T *__restrict__ shift_partials, int d, int k, const int *__restrict__ frozen, int kps) {
#pragma clang fp contract(off)
  constexpr int RS = WG / EPW;
  __shared__ double part[RS][EPW];
  __shared__ int cpart[RS][EPW];
  __shared__ T red[EPW];
  const int tid = threadIdx.x;
  const int slice = tid / EPW, el = tid % EPW;
  const int64_t kd = (int64_t)k * d;
  const int64_t e = (int64_t)blockIdx.x * EPW + el;
  const bool valid = e < kd;
  const int c = valid ? (int)(e / d) : 0;
  const int per = (row_blocks + RS - 1) / RS;
  const int lo = slice * per, hi = min(row_blocks, lo + per);
  double s = 0;
  int cnt = 0;
  if (valid) {
    int rb = lo;
    for (; rb + 4 <= hi; rb += 4) {
      const double a0 = psums[(size_t)rb * kd + e], a1 = psums[(size_t)(rb + 1) * kd + e];
      const double a2 = psums[(size_t)(rb + 2) * kd + e], a3 = psums[(size_t)(rb + 3) * kd + e];
      const int b0 = pcounts[(size_t)rb * k + c], b1 = pcounts[(size_t)(rb + 1) * k + c];
      const int b2 = pcounts[(size_t)(rb + 2) * k + c], b3 = pcounts[(size_t)(rb + 3) * k + c];
      s = s + a0;
      s = s + a1;
      s = s + a2;
      s = s + a3;
      cnt += b0 + b1 + b2 + b3;
    }
    for (; rb < hi; rb++) {
      s = s + psums[(size_t)rb * kd + e];
      cnt += pcounts[(size_t)rb * k + c];
    }
  }
  part[slice][el] = s;
  cpart[slice][el] = cnt;
  __syncthreads();
  T diff2 = 0;
  if (slice == 0 && valid) {
    double tot = part[0][el];
    int ctot = cpart[0][el];
#pragma unroll
    for (int q = 1; q < RS; q++) {
      tot = tot + part[q][el];
      ctot += cpart[q][el];
    }
    const T oldv = c_old[e];
    T newv;
    // (frozen: a stacked model's set that has met its convergence test keeps its centroids)
    if (ctot < 1 || (frozen != nullptr && frozen[c / kps] != 0)) {
      newv = oldv;  // revert_zeroed_centroids, kmeans_centroids.h:77-88
    } else {
      const T scale = (T)1.0 / (T)ctot;  // scale_centroids, kmeans_centroids.h:90-105
      newv = (T)tot * scale;
    }
    c_new[e] = newv;
    if (e - (int64_t)c * d == 0) counts[c] = ctot;
    const T df = oldv - newv;
    diff2 = df * df;
  }
  if (slice == 0) red[el] = diff2;
  __syncthreads();
  if (tid == 0) {
    T acc = 0;
    for (int q = 0; q < EPW; q++) acc = acc + red[q];
    shift_partials[blockIdx.x] = acc;
  }
}

template <typename T>
int launch_finalize(hipStream_t s, int slots, const double *psums,
                    const int *pcounts, const T *c_old, T *c_new, int *counts,
                    T *shift_partials, int *n_shift_partials, int d, int k, const int *frozen,
                    int kps) {
  const int64_t kd = (int64_t)k * d;
  // (a stacked model always takes the wide form: its sets' partials must not share a block)
  const bool narrow = kd <= FINALIZE_NARROW_KD && slots >= 256 && frozen == nullptr;
  const int blocks = narrow ? (int)((kd + 3) / 4) : (int)((kd + 31) / 32);
  if (narrow)
    hipLaunchKernelGGL((finalize_kernel<T, 4>), dim3(blocks), dim3(WG), 0, s, psums, pcounts,
                       slots, c_old, c_new, counts, shift_partials, d, k, frozen, kps);
  else
    hipLaunchKernelGGL((finalize_kernel<T, 32>), dim3(blocks), dim3(WG), 0, s, psums, pcounts,
                       slots, c_old, c_new, counts, shift_partials, d, k, frozen, kps);
  KM_HIP_TRY(hipGetLastError());
  *n_shift_partials = blocks;
  return 0;
}

// ---------------------------------------------------------------------------
// pass 3: centroid norms + ordered sum of shift partials.
// Blocks 0 .. ceil(k/WG)-1 compute norms; the last block sums the partials
// with one wavefront in a fixed order.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(WG) void post_update_kernel(
    const T *__restrict__ c_new, T *__restrict__ cnorm,
    const T *__restrict__ shift_partials, int n_partials, T *__restrict__ shift2,
    int d, int k) {
#pragma clang fp contract(off)
  const int tid = threadIdx.x;
  if (blockIdx.x == gridDim.x - 1) {
    __shared__ T red[WG];
    // eight loads in flight per thread, added in index order
    T acc = 0;
    int i = tid;
    for (; i + 7 * WG < n_partials; i += 8 * WG) {
      T v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = shift_partials[i + u * WG];
#pragma unroll
      for (int u = 0; u < 8; u++) acc = acc + v[u];
    }
    for (; i < n_partials; i += WG) acc = acc + shift_partials[i];
    red[tid] = acc;
    __syncthreads();
    for (int off = WG / 2; off > 0; off >>= 1) {
      if (tid < off) red[tid] = red[tid] + red[tid + off];
      __syncthreads();
    }
    if (tid == 0) *shift2 = red[0];
    return;
  }
  const int c = blockIdx.x * WG + tid;
  if (c >= k || cnorm == nullptr) return;
  const T *x = c_new + (size_t)c * d;
  T acc = 0;
  for (int j = 0; j < d; j++) {
    const T v = x[j];
    acc = acc + v * v;
  }
  cnorm[c] = acc;
}

template <typename T>
int launch_post_update(hipStream_t s, const T *c_new, T *cnorm,
                       const T *shift_partials, int n_shift_partials, T *shift2,
                       int d, int k) {
  // large centroid sets: norms by the coalesced row-norm kernel (same summation order),
  // this kernel then only adds up the shift partials
  const bool separate_norms = d >= 8 && ((int64_t)k * d >= 65536 || d >= 64);
  const int blocks = separate_norms ? 1 : (k + WG - 1) / WG + 1;
  hipLaunchKernelGGL((post_update_kernel<T>), dim3(blocks), dim3(WG), 0, s, c_new,
                     separate_norms ? (T *)nullptr : cnorm, shift_partials, n_shift_partials,
                     shift2, d, k);
  KM_HIP_TRY(hipGetLastError());
  if (separate_norms) return launch_row_norms<T>(s, c_new, cnorm, k, d);
  return 0;
}

// ---------------------------------------------------------------------------
// Deterministic sum of n values in double: stage 1 gives every block a fixed
// contiguous range and a fixed tree, stage 2 adds the block results in order.
// ---------------------------------------------------------------------------
static const int SUM_BLOCKS = 1024;
int sum_partials_needed() { return SUM_BLOCKS; }

template <typename T>
__global__ __launch_bounds__(WG) void sum_stage1_kernel(const T *__restrict__ v,
                                                       int64_t n,
                                                       double *__restrict__ partials) {
  __shared__ double red[WG];
  const int tid = threadIdx.x;
  const int64_t per = (n + gridDim.x - 1) / gridDim.x;
  const int64_t lo = (int64_t)blockIdx.x * per;
  const int64_t hi = min(n, lo + per);
  double acc = 0;
  for (int64_t i = lo + tid; i < hi; i += WG) acc += (double)v[i];
  red[tid] = acc;
  __syncthreads();
  for (int off = WG / 2; off > 0; off >>= 1) {
    if (tid < off) red[tid] += red[tid + off];
    __syncthreads();
  }
  if (tid == 0) partials[blockIdx.x] = red[0];
}
__global__ __launch_bounds__(WG) void sum_stage2_kernel(const double *__restrict__ partials,
                                                       int np, double *__restrict__ out) {
  __shared__ double red[WG];
  const int tid = threadIdx.x;
  double acc = 0;
  for (int i = tid; i < np; i += WG) acc += partials[i];
  red[tid] = acc;
  __syncthreads();
  for (int off = WG / 2; off > 0; off >>= 1) {
    if (tid < off) red[tid] += red[tid + off];
    __syncthreads();
  }
  if (tid == 0) *out = red[0];
}

template <typename T>
int launch_sum(hipStream_t s, const T *v, int64_t n, double *partials,
               int n_partials, double *out) {
  int blocks = n_partials < SUM_BLOCKS ? n_partials : SUM_BLOCKS;
  if (blocks < 1) return H2O4GPU_KMEANS_EARG;
  hipLaunchKernelGGL((sum_stage1_kernel<T>), dim3(blocks), dim3(WG), 0, s, v, n, partials);
  hipLaunchKernelGGL(sum_stage2_kernel, dim3(1), dim3(WG), 0, s, partials, blocks, out);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template <typename T>
__global__ void gather_rows_kernel(const T *__restrict__ X, const int *__restrict__ idx,
                                   T *__restrict__ C, int k, int d) {
  const int64_t e = (int64_t)blockIdx.x * WG + threadIdx.x;
  if (e >= (int64_t)k * d) return;
  const int c = (int)(e / d), j = (int)(e - (int64_t)c * d);
  C[e] = X[(int64_t)idx[c] * d + j];
}
template <typename T>
int launch_gather_rows(hipStream_t s, const T *X, const int *idx, T *C, int k, int d) {
  const int64_t kd = (int64_t)k * d;
  hipLaunchKernelGGL((gather_rows_kernel<T>), dim3((unsigned)((kd + WG - 1) / WG)),
                     dim3(WG), 0, s, X, idx, C, k, d);
  KM_HIP_TRY(hipGetLastError());
  return 0;
}

template int launch_bucketed_accumulate<float>(hipStream_t, const float *, const int *, int *, int *,
                                               int *, int *, int *, int *, double *, double *, int *,
                                               int64_t, int, int);
template int launch_bucketed_accumulate<double>(hipStream_t, const double *, const int *, int *, int *,
                                                int *, int *, int *, int *, double *, double *, int *,
                                                int64_t, int, int);

#define KM_INSTANTIATE(T)                                                            \
  template int launch_row_norms<T>(hipStream_t, const T *, T *, int64_t, int);       \
  template UpdatePlan plan_update<T>(int64_t, int, int, int);                        \
  template int launch_finalize<T>(hipStream_t, int, const double *,                  \
                                  const int *, const T *, T *, int *, T *, int *,    \
                                  int, int, const int *, int);                       \
  template int launch_post_update<T>(hipStream_t, const T *, T *, const T *, int,    \
                                     T *, int, int);                                 \
  template int launch_sum<T>(hipStream_t, const T *, int64_t, double *, int,         \
                             double *);                                              \
  template int launch_gather_rows<T>(hipStream_t, const T *, const int *, T *, int,  \
                                     int);
KM_INSTANTIATE(float)
KM_INSTANTIATE(double)

}  // namespace kmhip
