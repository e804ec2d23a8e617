/* C++ face of the k-means entry points, for callers written against the reference's
 * src/include/solver/kmeans.h:16-54 (namespace h2o4gpukmeans: makePtr_dense<T>,
 * kmeans_transform<T>, class H2O4GPUKMeans<M>). Header-only: every template forwards to
 * the extern "C" symbols of h2o4gpu_kmeans.h, so a C++ consumer only swaps the include
 * and links libh2o4gpu_kmeans_hip.so. */
#pragma once

#include "h2o4gpu_kmeans.h"

namespace h2o4gpukmeans {

/* The reference declares this class with a constructor only
 * (src/include/solver/kmeans.h:18-29, defined src/gpu/kmeans/kmeans_h2o4gpu.cu:609-615);
 * it records the problem and computes nothing. Kept for source compatibility. */
template <typename M>
class H2O4GPUKMeans {
 private:
  const M *_A;
  int _k;
  int _n;
  int _d;

 public:
  H2O4GPUKMeans(const M *A, int k, int n, int d) : _A(A), _k(k), _n(n), _d(d) {}
  const M *data() const { return _A; }
  int clusters() const { return _k; }
  int rows() const { return _n; }
  int cols() const { return _d; }
};

/* Replaces makePtr_dense<T>, src/gpu/kmeans/kmeans_h2o4gpu.cu:977-991 (float and double
 * are the two instantiations the reference provides, :1050-1058). */
template <typename T>
int makePtr_dense(int dopredict, int verbose, int seed, int gpu_id, int n_gpu, size_t rows,
                  size_t cols, int k, int max_iterations, int init_from_data, T threshold,
                  const T *srcdata, const T *centroids, T **pred_centroids, int **pred_labels);

template <>
inline int makePtr_dense<float>(int dopredict, int verbose, int seed, int gpu_id, int n_gpu,
                                size_t rows, size_t cols, int k, int max_iterations,
                                int init_from_data, float threshold, const float *srcdata,
                                const float *centroids, float **pred_centroids,
                                int **pred_labels) {
  return make_ptr_float_kmeans(dopredict, verbose, seed, gpu_id, n_gpu, rows, cols, k,
                               max_iterations, init_from_data, threshold, srcdata, centroids,
                               pred_centroids, pred_labels);
}

template <>
inline int makePtr_dense<double>(int dopredict, int verbose, int seed, int gpu_id, int n_gpu,
                                 size_t rows, size_t cols, int k, int max_iterations,
                                 int init_from_data, double threshold, const double *srcdata,
                                 const double *centroids, double **pred_centroids,
                                 int **pred_labels) {
  return make_ptr_double_kmeans(dopredict, verbose, seed, gpu_id, n_gpu, rows, cols, k,
                                max_iterations, init_from_data, threshold, srcdata, centroids,
                                pred_centroids, pred_labels);
}

/* Replaces kmeans_transform<T>, src/gpu/kmeans/kmeans_h2o4gpu.cu:891-975. */
template <typename T>
int kmeans_transform(int verbose, int gpu_id, int n_gpu, size_t m, size_t n, int k,
                     const T *srcdata, const T *centroids, T **preds);

template <>
inline int kmeans_transform<float>(int verbose, int gpu_id, int n_gpu, size_t m, size_t n, int k,
                                   const float *srcdata, const float *centroids, float **preds) {
  return kmeans_transform_float(verbose, gpu_id, n_gpu, m, n, k, srcdata, centroids, preds);
}

template <>
inline int kmeans_transform<double>(int verbose, int gpu_id, int n_gpu, size_t m, size_t n, int k,
                                    const double *srcdata, const double *centroids,
                                    double **preds) {
  return kmeans_transform_double(verbose, gpu_id, n_gpu, m, n, k, srcdata, centroids, preds);
}

}  // namespace h2o4gpukmeans
