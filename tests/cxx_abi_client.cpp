// A C++ caller written against the reference's template interface
// (src/include/solver/kmeans.h:16-54; examples/cpp/kmeans_driver.cpp:42-60 calls it this
// way): only the include differs. Built by __graft_entry__.build() with g++; run by
// tests/test_gpu_c_client.py. Prints "ok" when fit, predict and transform agree with a
// brute-force check done here.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../include/h2o4gpu_kmeans.hpp"

template <typename real_t>
static int run(const char *name) {
  const size_t rows = 5000, cols = 10;
  const int k = 6, iters = 4;
  std::vector<real_t> data(rows * cols), start(k * cols);
  for (size_t i = 0; i < rows; i++)
    for (size_t j = 0; j < cols; j++)
      data[i * cols + j] = (real_t)(5.0 * (i % k) + 0.01 * ((i * 11 + j * 7) % 90));
  for (int c = 0; c < k; c++)
    for (size_t j = 0; j < cols; j++) start[c * cols + j] = (real_t)(5.0 * c + 0.3);
  h2o4gpukmeans::H2O4GPUKMeans<real_t> problem(data.data(), k, (int)rows, (int)cols);
  real_t *centroids = nullptr, *dist = nullptr;
  int *labels = nullptr;
  int rc = h2o4gpukmeans::makePtr_dense<real_t>(0, 0, 1, 0, 1, rows, cols, problem.clusters(), iters,
                                                2, (real_t)0, data.data(), start.data(),
                                                &centroids, &labels);
  if (rc != 0) return 1;
  for (size_t i = 0; i < rows; i++)
    if (labels[i] != (int)(i % k)) return 2;
  rc = h2o4gpukmeans::kmeans_transform<real_t>(0, 0, 1, rows, cols, k, data.data(), centroids, &dist);
  if (rc != 0) return 3;
  for (size_t i = 0; i < rows; i += 97)
    for (int c = 0; c < k; c++) {
      double want = 0;
      for (size_t j = 0; j < cols; j++) {
        const double diff = (double)data[i * cols + j] - (double)centroids[c * cols + j];
        want += diff * diff;
      }
      if (std::fabs((double)dist[(size_t)c * rows + i] - want) > 1e-3 * (1.0 + want)) return 4;
    }
  free(dist);
  free(labels);
  free(centroids);
  printf("%s ok\n", name);
  return 0;
}

int main() {
  const int a = run<float>("float");
  const int b = run<double>("double");
  if (a || b) printf("failed %d %d\n", a, b);
  return a || b;
}
