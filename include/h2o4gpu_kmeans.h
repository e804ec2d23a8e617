/*
 * C ABI of the MI355X (gfx950) k-means engine, libh2o4gpu_kmeans_hip.so.
 *
 * Part 1 are the entry points h2o4gpu's language bindings already call for
 * k-means; a binding built against this header works unchanged. Part 2 is the
 * small device-information surface the Python estimator touches before it
 * fits. Part 3 is a handle API that keeps the data set resident in HBM between
 * calls (the reference has no counterpart; it re-uploads on every call).
 *
 * All pointers are plain host pointers unless a parameter is named d_*.
 * Matrices are dense, row-major, contiguous. Every function returns 0 on
 * success and a negative code on failure (no exit(), no exceptions).
 */
#ifndef H2O4GPU_KMEANS_H
#define H2O4GPU_KMEANS_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* error codes */
#define H2O4GPU_KMEANS_OK 0
#define H2O4GPU_KMEANS_EALLOC (-1)   /* allocation failed (the reference's -1) */
#define H2O4GPU_KMEANS_EARG (-2)     /* bad argument */
#define H2O4GPU_KMEANS_EDEVICE (-3)  /* HIP runtime error / no usable device */
#define H2O4GPU_KMEANS_ESTATE (-4)   /* call order (e.g. fit before data) */
#define H2O4GPU_KMEANS_ESCRATCH (-5) /* input beyond the fixed scratch of a no-allocation call */

/* ---------------------------------------------------------------------------
 * Part 1 - drop-in entry points.
 * Replaces: src/include/solver/kmeans.h:56-76 (declarations),
 *           src/gpu/kmeans/kmeans_h2o4gpu.cu:1060-1097 (definitions).
 *
 * dopredict == 0: fit.   srcdata [mTrain][n]; result buffers are allocated
 *   with malloc() and handed to the caller through *pred_centroids ([k][n])
 *   and *pred_labels ([mTrain] int32); the caller owns them.
 *   init_from_data: 0 = seeded random distinct rows (std::shuffle with
 *   std::default_random_engine(seed), as the reference), 1 = k-means|| with
 *   the reference's rounds, acceptance test and host k-means++ over the
 *   candidates (kmeans_h2o4gpu.cu:331-563; the estimator's 'k-means++'),
 *   2 = start from `centroids` ([k][n], extension: the reference ignores
 *   `centroids` when fitting), 3 = k-means++ by D^2 sampling on the device
 *   (extension).
 *   threshold: absolute bound on sum((C_old - C_new)^2); the loop stops when
 *   the sum is below it. Exactly as the reference, a run of N iterations
 *   makes N centroid updates and N+1 assignment passes, the last one with the
 *   final centroids.
 * dopredict != 0: predict. Labels of srcdata against `centroids`; only
 *   *pred_labels is set.
 * gpu_id selects the device as (gpu_id mod visible devices); n_gpu is
 * accepted for compatibility, one device is used.
 * If k > mTrain, k is clamped to mTrain (message on stderr) as in the reference.
 * ------------------------------------------------------------------------- */
int make_ptr_float_kmeans(int dopredict, int verbose, int seed, int gpu_id,
                          int n_gpu, size_t mTrain, size_t n, int k,
                          int max_iterations, int init_from_data,
                          float threshold, const float *srcdata,
                          const float *centroids, float **pred_centroids,
                          int **pred_labels);

int make_ptr_double_kmeans(int dopredict, int verbose, int seed, int gpu_id,
                           int n_gpu, size_t mTrain, size_t n, int k,
                           int max_iterations, int init_from_data,
                           double threshold, const double *srcdata,
                           const double *centroids, double **pred_centroids,
                           int **pred_labels);

/* The rows a fit with init_from_data == 0 starts from: entries 0..k-1 of
 * std::shuffle(iota(rows), std::default_random_engine(seed)) as libstdc++ computes
 * them (the reference's rule, src/gpu/kmeans/kmeans_h2o4gpu.cu:662-669), seed >= 0.
 * Host-only, needs no device. out: [k]. No counterpart in the reference, which does
 * not report the rows it picked. */
int h2o4gpu_kmeans_random_start_rows(int seed, size_t rows, int k, int *out);

/* Inertia (sum over rows of the squared distance to the assigned centroid,
 * accumulated in double in a fixed order) and number of Lloyd iterations of
 * the calling thread's most recent successful fit through make_ptr_*_kmeans.
 * Either pointer may be NULL. Returns H2O4GPU_KMEANS_ESTATE when the thread
 * has no successful fit yet.
 * No counterpart in the reference: its estimator leaves inertia_ at None
 * (src/interface_py/h2o4gpu/solvers/kmeans.py:187) because the entry point
 * has no slot to return it. */
int h2o4gpu_kmeans_last_fit_info(double *inertia, int *iterations);

/* 1 when all `count` values of a host array (elem_size 4: float, 8: double) are
 * finite, 0 when one is an infinity or a NaN, negative on bad arguments. Host
 * threads only, no device is touched.
 * Replaces, for the estimator: _check_data_content,
 * src/interface_py/h2o4gpu/solvers/utils.py:144-158 (two numpy passes and a
 * boolean temporary the size of the data). */
int h2o4gpu_kmeans_host_all_finite(const void *data, size_t count, int elem_size);

/* Squared distances |xx + cc - 2 x.c| of every row to every centroid, no
 * sqrt, centroid-major: (*preds)[c * m + i]. malloc()ed, caller owns.
 * Replaces: kmeans_transform<T>, src/gpu/kmeans/kmeans_h2o4gpu.cu:891-975. */
int kmeans_transform_float(int verbose, int gpu_id, int n_gpu, size_t m,
                           size_t n, int k, const float *srcdata,
                           const float *centroids, float **preds);

int kmeans_transform_double(int verbose, int gpu_id, int n_gpu, size_t m,
                            size_t n, int k, const double *srcdata,
                            const double *centroids, double **preds);

/* ---------------------------------------------------------------------------
 * Part 2 - device information used by the estimator's constructor.
 * Replaces: get_gpu_info_c, src/gpu/utils.cu:57-304 (NVML based; argument
 * list kept, see src/swig/util/gpu.i:64-93), get_compute_capability
 * (src/gpu/utils.cu:40-55), cudaresetdevice / cudaresetdevice_bare.
 * Arrays must hold at least *n_gpus entries; per-process usage arrays are
 * zero-filled (ROCm has no NVML process table here). Returns 0, or 1 when no
 * device is visible (as the reference does when NVML fails).
 * ------------------------------------------------------------------------- */
int get_gpu_info_c(int verbose, int return_memory, int return_name,
                   int return_usage, int return_free_memory,
                   int return_capability, int return_memory_by_pid,
                   int return_usage_by_pid, int return_all,
                   unsigned int *n_gpus, int *gpu_percent_usage,
                   unsigned long long *gpu_total_memory,
                   unsigned long long *gpu_free_memory, char **gpu_name,
                   int *majors, int *minors, unsigned int *num_pids,
                   unsigned int *pids, unsigned long long *usedGpuMemorys,
                   unsigned int *num_pids_usage, unsigned int *pids_usage,
                   unsigned long long *usedGpuUsage);
int get_compute_capability(int d_idx, int *major, int *minor, int *ratioperf);
int cudaresetdevice(int wDev, int nDev);
int cudaresetdevice_bare(void);
/* Number of visible HIP devices (0 if the runtime cannot be initialised). */
int h2o4gpu_kmeans_device_count(void);

/* ---------------------------------------------------------------------------
 * Part 3 - resident-data handle API (no counterpart in the reference).
 * One handle = one data set [rows][cols] of one precision on one device plus
 * the working set of a k-cluster model. Calls on one handle are serialised by
 * the caller; different handles are independent.
 * ------------------------------------------------------------------------- */
typedef struct h2o4gpu_kmeans_handle h2o4gpu_kmeans_handle;

/* elem_size: 4 = float, 8 = double. rows <= INT32_MAX (labels are int32). k may
 * exceed rows; only the row-based starts (init_random_rows, init_plusplus) then
 * return H2O4GPU_KMEANS_EARG. */
int h2o4gpu_kmeans_create(h2o4gpu_kmeans_handle **out, int elem_size,
                          size_t rows, size_t cols, int k, int gpu_id,
                          int verbose);
int h2o4gpu_kmeans_destroy(h2o4gpu_kmeans_handle *h);

/* Stacked restarts (the reference documents n_init > 1 as unsupported,
 * src/interface_py/h2o4gpu/solvers/kmeans.py:722-725): a handle holding `sets` independent
 * centroid sets of k centroids each over the same rows. One kernel labels every row against
 * all sets (the sets lie end to end as one model, the argmin taken per set) and sums the
 * rows per set, so the rows are read once per iteration for all restarts.
 * stack_width: the largest number of sets (<= max_sets) such a handle can hold for this
 * shape, 1 when the shape does not stack (restarts then run one after another on an
 * ordinary handle). create_stacked with sets < 2 is create.
 * On a stacked handle select_set picks the set addressed by set_centroids_host, init_*,
 * get_centroids / labels / counts / min_distances / seed_rows and inertia; fit, iterate and
 * assign work on all sets. With a threshold every set stops at its own iteration (its
 * centroids then stay as they are); set_iterations returns the [sets] update counts of the
 * last fit. update, set_labels_host, predict_host and transform_* are not offered. */
int h2o4gpu_kmeans_stack_width(int elem_size, size_t rows, size_t cols, int k, int max_sets);
int h2o4gpu_kmeans_create_stacked(h2o4gpu_kmeans_handle **out, int elem_size, size_t rows,
                                  size_t cols, int k, int sets, int gpu_id, int verbose);
int h2o4gpu_kmeans_select_set(h2o4gpu_kmeans_handle *h, int set);
int h2o4gpu_kmeans_set_iterations(h2o4gpu_kmeans_handle *h, int *iterations);

/* Upload rows from host memory (copies) / adopt a device pointer (no copy,
 * caller keeps it alive). Row norms are computed on the device either way. */
int h2o4gpu_kmeans_set_data_host(h2o4gpu_kmeans_handle *h, const void *X);
int h2o4gpu_kmeans_set_data_device(h2o4gpu_kmeans_handle *h, const void *d_X);

/* Initial centroids: given ([k][cols] host), seeded random distinct rows
 * (the reference's std::shuffle rule), k-means++ (D^2 sampling) on the device, or
 * k-means|| as the reference runs it for init_from_data == 1 (kmeans_parallel,
 * src/gpu/kmeans/kmeans_h2o4gpu.cu:331-563, with its host k-means++ over the
 * weighted candidates, :154-279). */
int h2o4gpu_kmeans_set_centroids_host(h2o4gpu_kmeans_handle *h, const void *C);
int h2o4gpu_kmeans_init_random_rows(h2o4gpu_kmeans_handle *h, int seed);
int h2o4gpu_kmeans_init_plusplus(h2o4gpu_kmeans_handle *h, int seed);
int h2o4gpu_kmeans_init_parallel(h2o4gpu_kmeans_handle *h, int seed);
/* Data rows the last init_* call chose ([k] int32; -1 where k-means|| found fewer than k
 * candidates and left a zero row, as the reference does). */
int h2o4gpu_kmeans_get_seed_rows(h2o4gpu_kmeans_handle *h, int *rows);
/* What the last init_parallel call found: *n_candidates; round_count[8] and phi[8]
 * (candidates added and sum of the minimum costs per round); with cap >= *n_candidates
 * also cand_rows (data row of every candidate, in the order found) and weights (rows per
 * nearest candidate; zeros when there were at most k candidates); chosen[k] = candidate
 * index of every final centre (-1: zero row). Any pointer may be NULL. */
int h2o4gpu_kmeans_parallel_seed_info(h2o4gpu_kmeans_handle *h, int cap, int *cand_rows,
                                      int *n_candidates, int *round_count, double *phi,
                                      double *weights, int *chosen);

/* The reference's loop (kmeans_impl.h:109-232): up to max_iterations of
 * assign + update, stop when shift^2 < threshold, final assignment with the
 * final centroids. *iterations_run receives the number of centroid updates. */
int h2o4gpu_kmeans_fit(h2o4gpu_kmeans_handle *h, int max_iterations,
                       double threshold, int *iterations_run);

/* Single steps (for lock-step checks and custom loops). assign: labels (and
 * per-row minimum squared distance) against the current centroids. update:
 * centroids <- per-label means of the current labels (empty clusters keep
 * their centroid); *shift2 (may be NULL) = sum((C_old - C_new)^2). */
int h2o4gpu_kmeans_assign(h2o4gpu_kmeans_handle *h);
int h2o4gpu_kmeans_update(h2o4gpu_kmeans_handle *h, double *shift2);
int h2o4gpu_kmeans_set_labels_host(h2o4gpu_kmeans_handle *h, const int *labels);
/* Enqueue `steps` iterations (assign + update each) on the handle's stream
 * without convergence test or host synchronisation (timing loops). */
int h2o4gpu_kmeans_iterate(h2o4gpu_kmeans_handle *h, int steps);

/* Results to host memory. */
int h2o4gpu_kmeans_get_centroids(h2o4gpu_kmeans_handle *h, void *C);
int h2o4gpu_kmeans_get_labels(h2o4gpu_kmeans_handle *h, int *labels);
int h2o4gpu_kmeans_get_counts(h2o4gpu_kmeans_handle *h, int *counts);
int h2o4gpu_kmeans_get_min_distances(h2o4gpu_kmeans_handle *h, void *mind);
/* Sum over rows of the minimum squared distance found by the last assign. */
int h2o4gpu_kmeans_inertia(h2o4gpu_kmeans_handle *h, double *inertia);

/* Labels / squared distances of other rows against the handle's centroids.
 * X: [rows][cols] host memory. dist: [k][rows] host memory. */
int h2o4gpu_kmeans_predict_host(h2o4gpu_kmeans_handle *h, size_t rows,
                                const void *X, int *labels);
int h2o4gpu_kmeans_transform_host(h2o4gpu_kmeans_handle *h, size_t rows,
                                  const void *X, void *dist);
/* Same on the handle's own resident rows, output left on the device:
 * d_dist [k][rows] device memory provided by the caller. */
int h2o4gpu_kmeans_transform_resident(h2o4gpu_kmeans_handle *h, void *d_dist);

/* Kernel selection: "assign" = 0 auto, 1 VALU, 2 MFMA row-stationary,
 * 3 MFMA tiled, 4 the one-pass kernel for rows beyond 64 features and at most 16
 * centroids (a wavefront along the features of four rows; a shape outside its range
 * reports "unsupported"); "fuse" = 1 (default) lets fit/iterate run assignment and the
 * per-centroid accumulation as one kernel where the shape allows, 0 keeps them
 * separate; "buckets" = 1 (default) sums the centroids of shapes whose sums do not
 * fit LDS by bucketing rows by label, 0 uses the chunked LDS kernel for them too;
 * "exact_argmin" = 1 makes the float32 matrix-core kernels compare the float distances
 * themselves instead of 16-ulp integer keys (slower, never fused; 0 is the default).
 * "transform_batch_mb" (default 4096) bounds the device buffer transform_host fills per
 * batch of rows; smaller values force more, shorter batches.
 * "fp32_split" = 9 or 6 (default 0) makes the float32 matrix-core kernels form their dot
 * products on the bfloat16 matrix pipe: every float is the exact sum of three bfloat16
 * parts (rounded to nearest), 9 runs all nine products of the parts (each exact,
 * accumulated in float32), 6
 * leaves out the three smallest (below one ulp of xx + cc per distance). 1.4 to 1.9 times
 * faster on matrix-bound shapes, same parity bars; shapes it does not apply to (float64,
 * k <= 16 && d <= 64, rows of fewer than 4 features, ...) run as without it, and
 * h2o4gpu_kmeans_assign_variant() names what runs ("mfma_tiled_bf16x6", ...). The
 * environment variable H2O4GPU_KMEANS_FP32_SPLIT=6|9 sets it for every handle created
 * afterwards, the reference's four entry points included.
 * "transform_buffers" = 2 (default) gives a transform in several batches two sets of device
 * buffers, so that a batch is computed while the previous one is downloaded (this is also
 * what happens with 1, one batch at a time, when the second set cannot be allocated).
 * "tiled_direct" = 1 (default) lets the tiled matrix-core kernels fetch their operands with
 * direct-to-LDS loads wherever rows and centroids are whole stages and 16-byte aligned; 0
 * stages them through registers everywhere (the form that serves every other shape). Same
 * labels up to near-ties: the two forms add the norms to the dot product at different ends
 * of the sum.
 * "seed_matrix" = 1 (default) lets init_parallel compute the distances between its
 * candidates as one matrix (while it fits 1 GiB) and pick the centres on the host from it:
 * for the duration of the seeding that takes up to 1 GiB of device memory and as much host
 * memory for the downloaded copy (M x M values for M candidates; when either allocation
 * fails the picks fall back to the other form); 0 runs one small kernel per pick, as
 * "assign" = 1 always does.
 * Unknown names return EARG. */
int h2o4gpu_kmeans_set_option(h2o4gpu_kmeans_handle *h, const char *name,
                              int value);

/* Timing on the handle's stream with HIP events. timer_start/timer_stop
 * bracket any sequence of calls; with kernel profiling on, every kernel launch
 * is bracketed by its own event pair and kernel_time() returns the launch count
 * and summed milliseconds since profiling was switched on, by kernel name
 * ("assign", "accumulate", "assign_accumulate", "finalize", "post_update",
 * "row_norms", "transform", "min_dist_update", "inertia_sum", "seed_assign",
 * "seed_fold", "seed_select", "seed_weights", "seed_pick"). */
int h2o4gpu_kmeans_timer_start(h2o4gpu_kmeans_handle *h);
int h2o4gpu_kmeans_timer_stop(h2o4gpu_kmeans_handle *h, float *milliseconds);
int h2o4gpu_kmeans_profile(h2o4gpu_kmeans_handle *h, int on);
int h2o4gpu_kmeans_kernel_time(h2o4gpu_kmeans_handle *h, const char *kernel,
                               int *launches, double *milliseconds);
/* Name of the assign kernel variant the handle's shape dispatches to. */
const char *h2o4gpu_kmeans_assign_variant(h2o4gpu_kmeans_handle *h);

/* Device-to-device copy bandwidth probe: copies `bytes` from one scratch
 * buffer to another `reps` times and returns the average milliseconds of one
 * copy (used to calibrate byte counters and to report achievable HBM rate). */
int h2o4gpu_kmeans_copy_probe(int gpu_id, size_t bytes, int reps,
                              float *milliseconds);

/* The same measurement for the other streaming patterns a Lloyd step is made of,
 * so that a kernel's bytes per second can be put beside what this device
 * delivers for its own mix of reads and writes and not only beside the
 * datasheet figure. kind: COPY = the kernel above (reads `bytes`, writes
 * `bytes`); READ = a kernel that only reads `bytes` (four 16-byte loads in
 * flight per thread, one float per thread written at the end); WRITE = a
 * kernel that only writes `bytes`; MEMCPY = hipMemcpyAsync device to device
 * (reads and writes `bytes`). Returns the average milliseconds of one pass. */
#define H2O4GPU_KMEANS_PROBE_COPY 0
#define H2O4GPU_KMEANS_PROBE_READ 1
#define H2O4GPU_KMEANS_PROBE_WRITE 2
#define H2O4GPU_KMEANS_PROBE_MEMCPY 3
int h2o4gpu_kmeans_bandwidth_probe(int gpu_id, int kind, size_t bytes, int reps,
                                   float *milliseconds);

/* ---------------------------------------------------------------------------
 * Part 4 - assignment without any allocation.
 * No counterpart in the reference. For callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc. Same result as h2o4gpu_kmeans_predict_host on the same rows
 * and centroids: d_labels[i] = index of the nearest of the k centroids
 * (d_centroids [k][cols]) to row i of d_X [rows][cols]; all three live in
 * device memory of the CURRENT device and are only element-aligned at least.
 * The work is queued on `stream` (a hipStream_t, NULL = the default stream) and
 * the call returns without waiting for it. It calls no hipMalloc / hipFree and
 * creates no stream or event: row norms, running minima, the padded copy of the
 * centroids and their norms live in one fixed array of
 * H2O4GPU_KMEANS_NOALLOC_SCRATCH_BYTES inside the library (one copy per device,
 * held until the process ends). Needed:
 *   round256(roundup(k,256)*cols*elem) + round256(roundup(k,256)*elem)
 *   + 2*round256(rows*elem) bytes;
 * more returns H2O4GPU_KMEANS_ESCRATCH and queues nothing. All calls on one
 * device share that array: calls that overlap in time on one device (other
 * threads, other streams) race; serialise them. The first call on a device
 * looks up the array's address and the device's properties, and the first call
 * of a process for a new kind of shape (a kernel instance that needs more than
 * 64 KB of LDS: wide rows, large models) sets that kernel's LDS limit once
 * (hipFuncSetAttribute): make one call per shape that will be used outside
 * graph capture first. The float32 arithmetic is always the float32 matrix
 * instructions': the environment variable H2O4GPU_KMEANS_FP32_SPLIT, which
 * switches handles to bfloat16 parts, is not read here, so with it set the
 * labels can differ from h2o4gpu_kmeans_predict_host's on near-tie rows.
 * ------------------------------------------------------------------------- */
#define H2O4GPU_KMEANS_NOALLOC_SCRATCH_BYTES (16u << 20)
int h2o4gpu_kmeans_predict_device_noalloc(int elem_size, size_t rows, size_t cols,
                                          int k, const void *d_X,
                                          const void *d_centroids, int *d_labels,
                                          void *stream);

#ifdef __cplusplus
}
#endif
#endif /* H2O4GPU_KMEANS_H */
