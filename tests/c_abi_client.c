/* A plain C caller of the shared library: includes the public header, links against
 * libh2o4gpu_kmeans_hip.so and calls the four entry points the reference exports
 * (src/include/solver/kmeans.h:56-76) with host pointers, as a compiled consumer would.
 * Prints the results as text; tests/test_gpu_c_client.py checks them against the oracle.
 * Built by __graft_entry__.build() with gcc; not a pytest module. */
#include <stdio.h>
#include <stdlib.h>

#include "../include/h2o4gpu_kmeans.h"

#define ROWS 6000
#define COLS 12
#define K 7
#define ITERS 5

static float value(int i, int j) {
  /* cluster (i mod K) sits at 3*(i mod K) in every coordinate, plus a small pattern */
  return 3.0f * (float)(i % K) + 0.01f * (float)((i * 7 + j * 13) % 100);
}

int main(void) {
  float *X = (float *)malloc(sizeof(float) * ROWS * COLS);
  float *C0 = (float *)malloc(sizeof(float) * K * COLS);
  if (!X || !C0) return 2;
  for (int i = 0; i < ROWS; i++)
    for (int j = 0; j < COLS; j++) X[i * COLS + j] = value(i, j);
  for (int c = 0; c < K; c++)
    for (int j = 0; j < COLS; j++) C0[c * COLS + j] = 3.0f * (float)c + 0.25f;

  float *centroids = NULL;
  int *labels = NULL;
  int rc = make_ptr_float_kmeans(0, 0, 1, 0, 1, ROWS, COLS, K, ITERS, 2, 0.0f, X, C0, &centroids,
                                 &labels);
  printf("fit_rc %d\n", rc);
  if (rc != 0) return 1;
  double inertia = 0.0;
  int iters = 0;
  rc = h2o4gpu_kmeans_last_fit_info(&inertia, &iters);
  printf("info_rc %d iterations %d inertia %.17g\n", rc, iters, inertia);
  for (int c = 0; c < K; c++) {
    printf("centroid %d", c);
    for (int j = 0; j < COLS; j++) printf(" %.9g", centroids[c * COLS + j]);
    printf("\n");
  }
  long long sum = 0;
  for (int i = 0; i < ROWS; i++) sum += (long long)labels[i] * (i % 97 + 1);
  printf("label_checksum %lld\n", sum);

  int *plabels = NULL;
  rc = make_ptr_float_kmeans(1, 0, 1, 0, 1, ROWS, COLS, K, ITERS, 0, 0.0f, X, centroids, NULL, &plabels);
  int same = rc == 0;
  for (int i = 0; same && i < ROWS; i++) same = plabels[i] == labels[i];
  printf("predict_rc %d same_as_fit %d\n", rc, same);

  float *dist = NULL;
  rc = kmeans_transform_float(0, 0, 1, 16, COLS, K, X, centroids, &dist);
  printf("transform_rc %d\n", rc);
  if (rc == 0)
    for (int c = 0; c < K; c++) {
      printf("dist %d", c);
      for (int i = 0; i < 16; i++) printf(" %.9g", dist[c * 16 + i]);
      printf("\n");
    }
  /* the results are malloc()ed by the library and owned by the caller */
  free(dist);
  free(plabels);
  free(labels);
  free(centroids);
  free(C0);
  free(X);
  return 0;
}
