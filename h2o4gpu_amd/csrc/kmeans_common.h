// Shared declarations of the gfx950 k-means engine: status codes, logging,
// launch-parameter structs and the kernel launchers each .hip file provides.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/h2o4gpu_kmeans.h"

namespace kmhip {

// Logger levels as the reference defines them (src/common/logger.h:10-25):
// a message of level L is printed when 0 < L <= verbose.
enum LogLevel {
  LOG_NOTHING = 0,
  LOG_FATAL = 100,
  LOG_ERROR = 200,
  LOG_INFO = 300,
  LOG_WARN = 400,
  LOG_DEBUG = 500,
  LOG_VERBOSE = 600
};
void log_msg(int verbose, int level, const char *fmt, ...)
    __attribute__((format(printf, 3, 4)));

#define KM_HIP_TRY(expr)                                                     \
  do {                                                                       \
    hipError_t _e = (expr);                                                  \
    if (_e != hipSuccess) {                                                  \
      ::kmhip::log_msg(LOG_ERROR, LOG_ERROR, "%s:%d %s failed: %s", __FILE__, \
                       __LINE__, #expr, hipGetErrorString(_e));              \
      return (_e == hipErrorOutOfMemory) ? H2O4GPU_KMEANS_EALLOC              \
                                         : H2O4GPU_KMEANS_EDEVICE;           \
    }                                                                        \
  } while (0)

#define KM_TRY(expr)            \
  do {                          \
    int _rc = (expr);           \
    if (_rc != 0) return _rc;   \
  } while (0)

// Kernels that use more than 64 KB of dynamic LDS need their limit raised first. That is
// done once per kernel instance, device and size (the largest size granted so far is
// remembered) instead of on every launch; forget_dynamic_lds drops what is remembered for
// a device whose context was reset.
int ensure_dynamic_lds(const void *kernel, size_t bytes);
// How many workgroups of `block` threads with `lds` bytes of dynamic LDS one CU holds at once
// (registers, LDS and wave slots all counted; asked of the runtime once per kernel instance,
// device and size): the grid of a persistent kernel must not exceed this times the CUs, or its
// last workgroups start only when the first ones have finished.
int resident_blocks_per_cu(const void *kernel, int block, size_t lds);
void forget_dynamic_lds(int dev);

// Assign-kernel variants (value of the "assign" option).
enum AssignVariant {
  ASSIGN_AUTO = 0,
  ASSIGN_VALU = 1,     // one thread per row, centroids broadcast from LDS
  ASSIGN_ROWSTAT = 2,  // MFMA, row tile stationary in registers, all centroids in LDS
  ASSIGN_TILED = 3,    // MFMA, both operands staged through LDS over a d-loop
  ASSIGN_LONGROW = 4   // no MFMA: a wavefront along the features of four rows (k <= 16, rows beyond 64 features)
};

// Rows the centroid buffer C (zeros) and entries the norm buffer cnorm (+inf) must
// be padded to: launch_assign / launch_transform may read that far.
static const int CENTROID_PAD = 256;

// Several independent centroid sets (restarts of one fit) laid end to end as one model:
// `sets` sets, each padded to kps rows (a multiple of 32; padding rows are zero) of which
// the first kset are centroids. Labels and minimum distances then hold one [n] block per
// set, the labels counting from the set's own first centroid; partial sums and counts are
// those of the whole stacked model. sets <= 1: an ordinary model. Only the row-stationary
// kernels with the whole model in LDS take a stacked model.
struct StackShape {
  int sets = 1;
  int kps = 0;
  int kset = 0;
};

// Device memory a launch with the bfloat16-parts option may write the centroids' parts to
// (tiled kernel only; tiled_split_scratch_bytes() says how much a shape needs). A launch that
// is given less runs the float32 instructions.
struct SplitScratch {
  void *ptr = nullptr;
  size_t bytes = 0;
  // tiled kernels: stage the operands through registers also where the direct-to-LDS form
  // applies (handle option "tiled_direct" = 0)
  bool through_registers = false;
};

// Fused distance + argmin. labels[i] = argmin_c |(xx_i + cc_c) - 2 x_i.c_c|,
// strict '<', lowest index wins, -1 when no distance is below FLT_MAX.
// mindist (nullable) receives the minimum. Returns the variant actually used
// through *used (nullable).
// exact (float32 MFMA kernels only): compare the float distances themselves instead of
// 16-ulp integer keys; slower, for measuring what the key resolution costs in parity.
template <typename T>
int launch_assign(hipStream_t s, int variant, const T *X, const T *xnorm,
                  const T *C, const T *cnorm, int *labels, T *mindist,
                  int64_t n, int d, int k, int num_cu, int *used, bool exact = false,
                  StackShape st = StackShape(), int split = 0, SplitScratch split_scratch = SplitScratch());
template <typename T>
int pick_assign_variant(int requested, int64_t n, int d, int k);
// The one-pass kernel for long rows and at most 16 centroids (longrow_kernels.hip): whether a
// shape is its (rows of whole 16-byte vectors, centroids and double-precision sums within one
// CU's LDS), the largest number of partial-sum slots its fused form writes, and the launch
// (SUMS false: labels and minimum distances only; cnorm may be null as for the fused kernels).
template <typename T>
bool longrow_applies(int d, int k);
template <typename T>
int longrow_max_slots(int d, int k, int num_cu);
template <typename T, bool SUMS>
int launch_longrow(hipStream_t s, const T *X, const T *xnorm, const T *C, const T *cnorm, int *labels,
                   T *mindist, int64_t n, int d, int k, int num_cu, double *psums, int *pcounts,
                   int *slots);
const char *assign_variant_name(int variant);
// split (float32 matrix-core kernels; 0, 6 or 9): run the dot products on the bfloat16
// matrix pipe as that many products of bfloat16 parts per feature pair (9: every product
// exact, 6: the three below 2^-24 of |x||c| left out). assign_split_products() returns the
// number a launch of this shape uses: 0 where the option does not apply (float64, the
// vector-ALU kernels, rows of fewer than 4 features; row-stationary kernel: rows padded to
// fewer than 16 or more than 64 features, fused step whose staged parts exceed the LDS
// budget; tiled kernel: 64 centroids or fewer), and such launches run the float32 matrix
// instructions.
template <typename T>
int assign_split_products(int variant, int split, int64_t n, int d, int k, bool fused);
// The tiled kernel takes the centroids' parts from device scratch of this many bytes
// (split_scratch of launch_assign / launch_transform), written anew by every launch; without
// the scratch (or with 0 bytes needed) it runs the float32 instructions.
template <typename T>
size_t tiled_split_scratch_bytes(int split, int d, int k);

// Fused assign + accumulate (row-stationary MFMA shapes and the small VALU shapes): labels/mindist as
// launch_assign, plus per-workgroup partial sums psums[slot][k][d] and counts
// pcounts[slot][k]; *slots receives the number of slots written. fused_slots()
// returns the largest slot count the launch can use, or 0 when the shape (or a
// forced assign variant) rules the fused kernel out. cnorm may be null: the kernel then
// computes the centroid norms from C itself (same values, j ascending), so that a Lloyd
// loop that needs no convergence scalar can skip launch_post_update.
template <typename T>
int fused_slots(int requested_variant, int64_t n, int d, int k, int num_cu);
template <typename T>
int launch_assign_accumulate(hipStream_t s, int variant, const T *X, const T *xnorm, const T *C,
                             const T *cnorm, int *labels, T *mindist, int64_t n, int d,
                             int k, int num_cu, double *psums, int *pcounts, int *slots,
                             int *used, StackShape st = StackShape(), int split = 0);

// Full squared-distance matrix, centroid-major: D[c * ldn + i], i < n.
template <typename T>
int launch_transform(hipStream_t s, const T *X, const T *xnorm, const T *C,
                     const T *cnorm, T *D, int64_t n, int64_t ldn, int d, int k,
                     int num_cu, int split = 0, SplitScratch split_scratch = SplitScratch());

// out[i] = sum_j X[i][j]^2, j ascending, no contraction.
template <typename T>
int launch_row_norms(hipStream_t s, const T *X, T *out, int64_t n, int d);

// Centroid update, pass 1: per-row-block partial sums (always double) and counts.
struct UpdatePlan {
  int row_blocks;   // partial slots along rows
  int kc;           // centroids per LDS chunk
  int k_chunks;     // ceil(k / kc)
  int vec;          // elements per load (1, 2 or 4)
  int sd;           // LDS row stride of the sums, in elements
  int threads;      // workgroup size of the accumulate kernel (256, 512 or 1024)
  size_t lds_bytes;
};
template <typename T>
UpdatePlan plan_update(int64_t n, int d, int k, int num_cu);
template <typename T>
int launch_accumulate(hipStream_t s, const UpdatePlan &p, const T *X,
                      const int *labels, double *psums, int *pcounts, int64_t n,
                      int d, int k);
// Pass 1 for shapes whose sums need many LDS chunks: the rows are ordered by label with a
// stable counting sort (order / order_label: [n] int32 each, offsets: [k] int32,
// block_hist: [bucket_blocks(n)][k] int32, seg_hist: [32][k] int32) and summed in fixed
// windows of the ordered rows (partials: [bucket_partial_slots(n, k)][d] double) into
// gsum [k][d] double; counts receives the bucket sizes. Run-to-run reproducible for
// both precisions. The result is consumed by launch_finalize with slots = 1.
bool bucketed_update_applies(int k_chunks, int k, int d);
int bucket_blocks(int64_t n);
size_t bucket_partial_slots(int64_t n, int k);
template <typename T>
int launch_bucketed_accumulate(hipStream_t s, const T *X, const int *labels, int *order,
                               int *order_label, int *offsets, int *block_hist, int *seg_hist,
                               int *total, double *partials, double *gsum, int *counts, int64_t n,
                               int d, int k);

// Pass 2: fixed-order reduction of the partials, empty clusters keep the old
// centroid, mean = sum * (1/count), per-block partial of sum((old-new)^2).
// shift_partials must hold max_shift_partials(d, k) entries. frozen (nullable, device,
// [k / kps] flags): centroids of a set of a stacked model whose flag is set stay as they
// are; each block of 32 coordinates then lies inside one set (kps is a multiple of 32), so
// a set's squared shift is the sum of its own partials.
static const int64_t FINALIZE_NARROW_KD = 4096;
static inline int max_shift_partials(int d, int k) {
  const int64_t kd = (int64_t)k * d;
  return (int)(kd <= FINALIZE_NARROW_KD ? (kd + 3) / 4 : (kd + 31) / 32);
}
template <typename T>
int launch_finalize(hipStream_t s, int slots, const double *psums,
                    const int *pcounts, const T *c_old, T *c_new, int *counts,
                    T *shift_partials, int *n_shift_partials, int d, int k,
                    const int *frozen = nullptr, int kps = 1);
// Pass 3: cnorm of the new centroids and the fixed-order sum of the shift
// partials into *shift2.
template <typename T>
int launch_post_update(hipStream_t s, const T *c_new, T *cnorm,
                       const T *shift_partials, int n_shift_partials, T *shift2,
                       int d, int k);

// Deterministic sum of n values (two fixed-order stages), result in double.
template <typename T>
int launch_sum(hipStream_t s, const T *v, int64_t n, double *partials,
               int n_partials, double *out);
int sum_partials_needed();

// k-means++ seeding, round t (t = 0 first): mind[i] = min(mind[i], |xx_i + cc - 2 x_i.c|)
// against the t-th chosen centre (row `centre_row` of X; t == 0 overwrites), then
// bsums[b] = sum of mind over rows [b*KPP_BLOCK, (b+1)*KPP_BLOCK) in double with a fixed
// tree. nearest [n] keeps the index of the closest chosen centre so far, rows [k] the
// chosen rows and dcc [k] the distances from the newest centre to the earlier ones: rows
// that the triangle inequality rules out are not read.
static const int KPP_BLOCK = 1024;
template <typename T>
int launch_min_dist_update(hipStream_t s, const T *X, const T *xnorm, int64_t centre_row,
                           T *mind, int *nearest, int *rows, T *dcc, int t, double *bsums,
                           int64_t n, int d);

// k-means|| building blocks (kmeans_h2o4gpu.cu:331-563): a padded model of candidate rows
// for the assign kernels; running minimum cost + its fixed-order block sums
// (bsums: [ceil(n / KPP_BLOCK)]); the reference's per-row acceptance test, rows taken
// appended to list (arrival order, *count may exceed cap); rows per nearest candidate;
// one distance step of the host k-means++ over the candidates.
template <typename T>
int launch_gather_model(hipStream_t s, const T *X, const T *xnorm, const int *idx, int m, int mpad,
                        T *Cc, T *ccn, int d);
template <typename T>
int launch_fold_min(hipStream_t s, const T *cur, T *cost, double *bsums, int64_t n, int init,
                    const int *cur_label = nullptr, int *near = nullptr, int label_off = 0);
template <typename T>
int launch_select_rows(hipStream_t s, const T *cost, T total, uint32_t state0, int k, int *list,
                       int *count, int cap, int64_t n);
int launch_label_histogram(hipStream_t s, const int *labels, int *counts, int64_t n);
// CcT: column-major copy of the m candidate rows Cc (launch_transpose_candidates): the dot
// products are then summed over the features in ascending order, as a scalar loop sums them.
// CcT null: several lanes share a candidate (strided partial sums and a tree; much faster,
// another summation order).
template <typename T>
int launch_transpose_candidates(hipStream_t s, const T *Cc, T *CcT, int m, int d);
template <typename T>
int launch_candidate_dists(hipStream_t s, const T *Cc, const T *CcT, const T *ccn, int centre, T *best,
                           T *mirror, int m, int d, int first);

// Copy rows idx[0..k-1] of X into C ([k][d]).
template <typename T>
int launch_gather_rows(hipStream_t s, const T *X, const int *idx, T *C, int k,
                       int d);

}  // namespace kmhip
