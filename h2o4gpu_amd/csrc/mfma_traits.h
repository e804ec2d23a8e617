// gfx950 matrix-core shapes used by the distance kernels.
//
// The distance contraction is D[c][i] = sum_j Cneg2[c][j] * X[i][j] with the
// centroids as the MFMA "A" operand (rows of the result) and the data rows as
// the "B" operand (columns of the result). With that orientation one lane
// holds, for ONE data row, the distances to several centroids, so the running
// argmin over centroids stays inside the lane; lanes only meet once per row
// tile, at the very end.
//
// Operand layout of both instructions (checked on hardware):
//   A: lane l supplies A[i = l % MT][kk = l / MT]
//   B: lane l supplies B[kk = l / MT][j = l % MT]
//   v_mfma_f32_32x32x2_f32 : MT = 32, KL = 2 k-slices, 16 accumulators / lane,
//       accumulator v of lane l is D[i = 8*(v/4) + 4*(l/32) + v%4][j = l%32]
//   v_mfma_f64_16x16x4_f64 : MT = 16, KL = 4 k-slices, 4 accumulators / lane,
//       accumulator v of lane l is D[i = 4*v + l/16][j = l%16]
// The k index a lane group contributes is free as long as A and B agree, so
// the feature axis is cut into 16-byte vectors that are dealt to the KL lane
// groups in turn (vector v: lane group v % KL, step v / KL): a data row is
// fetched with plain 16-byte loads, needs no shuffle on its way into the matrix
// core, and a row (or a last d-step) shorter than the padded width leaves whole
// steps empty, which the kernels skip.
#pragma once
#include <hip/hip_runtime.h>

namespace kmhip {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef double doublex2 __attribute__((ext_vector_type(2)));
// the same 16 bytes at an address that is only aligned to its elements (gfx950 serves such
// loads with one instruction)
typedef float floatx4_u __attribute__((ext_vector_type(4), aligned(4)));
typedef double doublex2_u __attribute__((ext_vector_type(2), aligned(8)));

template <typename T>
struct Mfma;

template <>
struct Mfma<float> {
  static constexpr int MT = 32;
  static constexpr int KL = 2;
  static constexpr int NACC = 16;
  static constexpr int VW = 4;  // elements in a 16-byte vector
  typedef floatx16 acc_t;
  typedef floatx4 vec_t;
  typedef floatx4_u uvec_t;
  static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  // centroid (row of the result tile) held by accumulator v of lane group g
  static __device__ __forceinline__ constexpr int acc_row(int v, int g) {
    return (v >> 2) * 8 + g * 4 + (v & 3);
  }
};

template <>
struct Mfma<double> {
  static constexpr int MT = 16;
  static constexpr int KL = 4;
  static constexpr int NACC = 4;
  static constexpr int VW = 2;
  typedef doublex4 acc_t;
  typedef doublex2 vec_t;
  typedef doublex2_u uvec_t;
  static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ constexpr int acc_row(int v, int g) {
    return 4 * v + g;
  }
};

// Largest finite float: the start value of the running minimum for both
// precisions, as the reference has it (kmeans_labels.h:363).
template <typename T>
__device__ __forceinline__ T argmin_start() {
  return (T)3.402823466e+38F;
}

template <typename T>
__device__ __forceinline__ T pos_inf();
template <>
__device__ __forceinline__ float pos_inf<float>() {
  return __builtin_huge_valf();
}
template <>
__device__ __forceinline__ double pos_inf<double>() {
  return __builtin_huge_val();
}

// Keep (best, idx) or take (ob, oi): lower value wins, equal values keep the
// lower index; idx -1 (nothing found) compares as the largest index.
template <typename T>
__device__ __forceinline__ void argmin_merge(T &best, int &idx, T ob, int oi) {
  if (ob < best || (ob == best && (unsigned)oi < (unsigned)idx)) {
    best = ob;
    idx = oi;
  }
}

}  // namespace kmhip
