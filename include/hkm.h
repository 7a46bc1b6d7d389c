/*
 * hkm.h -- C ABI of libhkm: the k-means Lloyd step (distance -> argmin -> per-cluster mean) as
 * hand-written gfx950 kernels.
 *
 * The reference (helmholtz-analytics/heat) has no FFI for this path: it is a chain of PyTorch calls
 * behind plain Python functions.  Each entry point below therefore cites the Python function whose
 * arithmetic it replaces; the Python host package binds them with ctypes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer (except where noted), row-major, fp32 unless the name says
 *     otherwise; `ld*` are leading dimensions in ELEMENTS (ld >= number of columns);
 *   - X, C, Y and out base pointers must be 4-byte aligned; 16-byte alignment together with
 *     ld % 4 == 0 enables the vector-load fast paths;
 *   - return value: HKM_OK or a negative HKM_E* code; a human-readable message for the last error
 *     of the calling thread is available from hkm_last_error();
 *   - argument validation runs on the host before anything is launched, so it is testable without
 *     a GPU;
 *   - every call only ENQUEUES work on `hip_stream` (a hipStream_t, NULL = default stream); nothing
 *     synchronises; the library allocates nothing: the caller passes a workspace of at least
 *     hkm_workspace_bytes(N, D, K, flags) bytes (256-byte aligned) that must stay alive until the
 *     enqueued work has finished.  Concurrent calls must use different workspaces;
 *   - all reductions use a fixed order, or arithmetic that is exact and therefore independent of the order
 *     (integer sums, fp64 sums of pre-rounded addends): the same inputs give bit-identical outputs on every run.
 *
 * Environment (looked up on every call, nothing is cached)
 *   HKM_PRODUCTS=bf16x3   hkm_assign_f32 / hkm_lloyd_step_f32, every shape with D > 16 except those with
 *                         32 < D <= 128 whose centroids fit in LDS: the cross term x.c is evaluated on
 *                         the bf16 matrix cores from operands split three ways (six partial products,
 *                         fp32 accumulation) instead of fp32 matrix instructions.  Same error bound per
 *                         product as fp32, 1.3x to 1.7x the throughput.  Off by default.
 *   HKM_UPDATE_LISTS=1    hkm_update_f32 and the two-pass part of hkm_lloyd_step_f32 use the list-based
 *                         kernels instead of the sort-based ones (a testing aid).
 *   HKM_SMALL_SUMS=ordered|integer   hkm_lloyd_step_f32 on the narrow shapes (D <= 16, K (D + 1) <= 240) with
 *                         more than 48 accumulator slots: form the per-cluster sums in a fixed order, or as
 *                         exact 64-bit integer sums, whatever N is (unset: integer from about a million rows
 *                         on, from 131072 with more than 32 clusters or more than 8 features).  A testing
 *                         aid; both give the same labels and means equal to fp32 rounding.
 *   HKM_NARROW_MFMA_MIN_K=n   hkm_assign_f32 with 4 <= D <= 16: use the matrix-core kernels from n centroids
 *                         on (default 32) and the vector kernel below.  A measuring and testing aid.
 *   HKM_FIT=steps         (read by the Python estimator, not by the library) KMeans.fit runs one hkm_lloyd_step_f32
 *                         per iteration even where hkm_lloyd_fit_f32 applies.  A testing aid.
 *   HKM_SMALL_BLOCKED_MIN_K=n   the narrow kernels with D <= 3 scan the centroids four at a time from n
 *                         centroids on (default 12), one at a time below.  Same results bit for bit; a
 *                         measuring and testing aid.
 */
#ifndef HKM_H
#define HKM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HKM_OK 0
#define HKM_EINVAL (-1)       /* bad argument (null pointer, negative size, ld < D, misalignment) */
#define HKM_EWORKSPACE (-2)   /* workspace missing or too small */
#define HKM_EHIP (-3)         /* a HIP runtime call failed; message holds hipGetErrorString */
#define HKM_EUNSUPPORTED (-4) /* shape outside what the kernels cover */

/* flags for hkm_workspace_bytes */
#define HKM_WS_ASSIGN 1
#define HKM_WS_UPDATE 2
#define HKM_WS_LLOYD 3 /* assign + update */
#define HKM_WS_SSE 4   /* add when hkm_lloyd_step_f32 is called with sse != NULL (N floats of scratch) */
#define HKM_WS_MEDIAN 8 /* on its own: scratch of hkm_update_median_f32 / hkm_closest_rows_l1_f32 */
#define HKM_WS_F64 16   /* add for the *_f64 entry points (partials and scratch are doubles) */
#define HKM_WS_FIT 32   /* on its own: scratch of hkm_lloyd_fit_f32 (0 where that entry point does not apply) */

/* Library version: major*10000 + minor*100 + patch. */
int hkm_version(void);

/* Message of the last error raised on the calling thread ("" if none). Host pointer, static storage. */
const char* hkm_last_error(void);

/* Bytes of device workspace needed by the entry points below for this problem size; 0 for sizes they
 * refuse (N < 0, D < 1, K < 1, and N > 2^40 rows or K * D > 2^40 centroid coordinates, which return
 * HKM_EUNSUPPORTED: no device holds them, and the byte counts derived from them could wrap around). */
size_t hkm_workspace_bytes(int64_t N, int32_t D, int32_t K, int32_t flags);

/*
 * Fused distance + argmin; the N x K matrix is never materialised.
 *   labels[i] = argmin_k max(0, (|x_i|^2 + |c_k|^2) - 2 x_i.c_k), first index on ties
 *   min_d2[i] = that minimum (clamped, NOT square-rooted); may be NULL.
 * Replaces heat/spatial/distance.py:47-64 (_quadratic_expand), :32-44 (_euclidian_fast; the
 * monotone sqrt is dropped under the argmin) and the argmin of heat/cluster/_kcluster.py:352-370
 * (heat/core/statistics.py:129-200).
 */
int hkm_assign_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                   int64_t ldc, int32_t* labels, float* min_d2, void* ws, size_t ws_bytes,
                   void* hip_stream);

/*
 * hkm_assign_f32 with the labels stored as the int64 the reference returns (heat/core/statistics.py:129-200
 * through heat/core/_operations.py:516-522), for the narrow shapes whose kernel is "valu_fused"
 * (hkm_assign_kernel_name): their assignment is bound by memory traffic, and storing int64 at once saves the
 * second pass over the labels that hkm_widen_labels_i64 makes (8 instead of 4 + 4 + 8 bytes per row).  Same
 * labels and min_d2 as hkm_assign_f32, no workspace.  Other shapes return HKM_EUNSUPPORTED: use hkm_assign_f32
 * and hkm_widen_labels_i64.
 */
int hkm_assign_labels64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                            int64_t ldc, int64_t* labels, float* min_d2, void* hip_stream);

/*
 * hkm_assign_f32 for callers that cannot allocate device memory or carry a workspace: code under HIP
 * graph capture, tight serving loops (predict), harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  Same arguments, results and kernels as hkm_assign_f32, but the scratch (reduction slots,
 * squared centroid norms, the merge keys of the streaming kernel) is a device array of
 * HKM_STATIC_SCRATCH_BYTES built into the library, which every GPU the library runs on holds from the
 * first call on it until the process ends.  The call allocates and frees nothing.  Shapes whose
 * hkm_workspace_bytes(N, D, K, HKM_WS_ASSIGN) exceeds HKM_STATIC_SCRATCH_BYTES return HKM_EUNSUPPORTED
 * (centroids resident in LDS or D <= 64: every K up to about four million; the streaming kernel -- D > 128, or
 * D > 64 with more centroids than LDS holds -- up to about two million rows, 8 bytes each).
 * All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race;
 * calls on one stream are ordered and each refills what it reads.
 * The array's device address is looked up once per device (hipGetSymbolAddress), by whichever comes first on
 * that device: hkm_static_scratch_bytes() or hkm_assign_static_f32.  A stream under capture may refuse that
 * lookup, so call hkm_static_scratch_bytes() once with the device current BEFORE capturing; after that the
 * entry point only enqueues kernels and can be captured into a HIP graph and replayed.
 */
#define HKM_STATIC_SCRATCH_BYTES (16u << 20)
size_t hkm_static_scratch_bytes(void);
int hkm_assign_static_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, void* hip_stream);

/*
 * Deterministic per-cluster mean: C_new[k] = (sum over {i: labels[i]==k} of x_i) / count_k, sums
 * in fp64, count rounded through fp32 like the reference does; an empty cluster gives a zero row.
 * counts (int64[K]) may be NULL.  labels outside [0, K) are ignored.
 * Replaces heat/cluster/kmeans.py:76-103 (KMeans._update_centroids).
 */
int hkm_update_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                   int32_t K, float* C_new, int64_t ldcn, int64_t* counts, void* ws,
                   size_t ws_bytes, void* hip_stream);

/*
 * One Lloyd iteration: labels against C, C_new = per-cluster means, *shift = sum((C - C_new)^2)
 * (fp32 value, device scalar), optional *sse = sum_i min_d2[i] (device scalar; NULL to skip).
 * C and C_new are K x D with leading dimension D.  labels may be NULL where
 * hkm_lloyd_step_labels_optional() says so -- the one-sweep steps that memory bounds ("lloyd_small" and
 * "lloyd_few"): the step then stores no labels (4 of its 4D+4 bytes per point; next to a stream of reads even
 * so small a stream of writes costs up to a sixth of the read bandwidth) -- a fit needs only those of its last
 * iteration, which hkm_assign_f32 against the previous centroids reproduces bit for bit.  shift (and sse) may also point to pinned,
 * device-accessible host memory: the finishing kernel then delivers the scalar itself and no copy
 * sits between two steps on the stream.
 * Replaces the loop body of heat/cluster/kmeans.py:131-143 (KMeans.fit).
 */
int hkm_lloyd_step_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                       float* C_new, int32_t K, int32_t* labels, float* shift, float* sse, void* ws,
                       size_t ws_bytes, void* hip_stream);

/* 1 if hkm_lloyd_step_f32 accepts labels == NULL for this shape, else 0. */
int hkm_lloyd_step_labels_optional(int64_t N, int32_t D, int32_t K);

/*
 * hkm_lloyd_step_f32 with the labels stored as the int64 the reference returns (heat/core/_operations.py:516-522),
 * for the shapes whose step is "lloyd_small" (hkm_lloyd_kernel_name): a fit whose last iteration is known in
 * advance (the max_iter-th) runs that one step through this entry point and needs neither a pass over X for its
 * labels nor a pass over the labels to widen them.  labels must not be NULL here and must be 8-byte aligned; same
 * centroids, shift and sse as hkm_lloyd_step_f32, bit for bit.  Other shapes return HKM_EUNSUPPORTED.
 * Replaces the loop body of heat/cluster/kmeans.py:131-143 in the fit's last iteration.
 */
int hkm_lloyd_step_labels64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, float* C_new,
                                int32_t K, int64_t* labels, float* shift, float* sse, void* ws, size_t ws_bytes,
                                void* hip_stream);

/*
 * The WHOLE Lloyd loop in one launch, for data that stays in the registers of a few dozen workgroups:
 *   for it in 1..max_iter: labels against C; C = per-cluster means; shift = sum((C_old - C)^2);
 *                          stop after the first iteration with use_tol != 0 and shift <= tol
 * with labels (N int64: the (N, 1) matrix the reference returns) those of the LAST assignment, C_out (K x D dense)
 * the centroids after the last update and *shift (device scalar) the last shift.  X is read once per fit; the
 * per-cluster sums are exact 64-bit integer sums (a coordinate enters with 44 bits below the largest value of its
 * column), kept up to date from the rows whose label changed, so two iterations with the same
 * labels give the same centroids bit for bit, as in the reference; the workgroups exchange their sums once per
 * iteration and every one of them forms the centroids and takes the stop decision itself.
 * info (two int32; device memory or pinned, device-accessible host memory) receives, when the launch has
 * finished: info[0] = the iterations run (>= 1), or -1 if a wait between the workgroups ran out (no output is
 * valid then: a workgroup that has waited wait_limit_us microseconds gives up and every other one follows, so
 * the kernel always ends), or -2 if X holds a non-finite coordinate (no output valid either); info[1] = the bits
 * of the last shift.  On a negative status run the loop with hkm_lloyd_step_f32.
 * Shapes: hkm_lloyd_fit_supported(N, D, K) != 0, i.e. D <= 16, K (D + 1) <= 240 and N <= 65536 times the rows
 * a thread holds (4 up to 4 features, 2 up to 8, else 1: 262144 / 131072 / 65536 rows); others return
 * HKM_EUNSUPPORTED.
 * ws: hkm_workspace_bytes(N, D, K, HKM_WS_FIT) bytes.  C0 and C_out may be the same matrix.
 * Replaces heat/cluster/kmeans.py:131-146 (the loop of KMeans.fit) with :76-103 and
 * heat/cluster/_kcluster.py:352-370 inside it.
 */
int hkm_lloyd_fit_supported(int64_t N, int32_t D, int32_t K);
int hkm_lloyd_fit_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C0, int32_t K, int32_t max_iter,
                      int32_t use_tol, double tol, float* C_out, int64_t* labels, float* shift, int32_t* info,
                      uint64_t wait_limit_us, void* ws, size_t ws_bytes, void* hip_stream);

/* *shift = sum((C_old - C_new)^2), fixed order.  Replaces heat/cluster/kmeans.py:141. */
int hkm_shift_f32(const float* C_old, const float* C_new, int32_t K, int32_t D, float* shift,
                  void* hip_stream);

/*
 * Clustering functional of predict(): *out = (sqrt(sum_i sqrt(min_d2[i])^2))^2 in fp32, the sum
 * taken in fp64 in a fixed order.  ws needs hkm_workspace_bytes(N, 1, 1, HKM_WS_ASSIGN) bytes.
 * Replaces heat/cluster/_kcluster.py:367-368 (norm(distances.min(axis=1), 2) ** 2).
 */
int hkm_functional_value_f32(const float* min_d2, int64_t N, float* out, void* ws, size_t ws_bytes,
                             void* hip_stream);

/*
 * Full distance matrix for the public cdist API:
 *   out[i, j] = max(0, (|x_i|^2 + |y_j|^2) - 2 x_i.y_j), square-rooted when sqrt_flag != 0.
 * X is M x D, Y is Nn x D, out is M x Nn with leading dimension ldo.
 * Replaces heat/spatial/distance.py:136-156 (cdist, quadratic_expansion=True) on local tensors.
 */
int hkm_cdist_f32(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                  int32_t D, float* out, int64_t ldo, int32_t sqrt_flag, void* hip_stream);

/*
 * The other pairwise functions of heat/spatial/distance.py on local tensors, out is M x Nn:
 *   HKM_METRIC_EUCLID_QE  sqrt(max(0, |x|^2+|y|^2-2x.y))        cdist(quadratic_expansion=True),  :32-64
 *   HKM_METRIC_EUCLID     sqrt(sum((x-y)^2))                     cdist(quadratic_expansion=False), :17-29
 *   HKM_METRIC_GAUSS_QE   exp(-max(0, expansion) / (2 sigma^2))  rbf(quadratic_expansion=True),    :87-103
 *   HKM_METRIC_GAUSS      exp(-sum((x-y)^2) / (2 sigma^2))       rbf(quadratic_expansion=False),   :67-84
 *   HKM_METRIC_MANHATTAN  sum(|x-y|)                             manhattan(expand=True/False),     :106-133
 * sigma is read for the two Gaussian metrics only.
 */
#define HKM_METRIC_EUCLID_QE 0
#define HKM_METRIC_EUCLID 1
#define HKM_METRIC_GAUSS_QE 2
#define HKM_METRIC_GAUSS 3
#define HKM_METRIC_MANHATTAN 4
int hkm_pairwise_f32(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                     int32_t D, float* out, int64_t ldo, int32_t metric, float sigma, void* hip_stream);

/*
 * Pieces of the k-means|| initialisation (heat/cluster/_kcluster.py:146-247, 283-350); the distance
 * work itself is hkm_assign_f32 with its min_d2 output.
 *
 * hkm_min_dist_sum_f32: *out = sum_i sqrt(min_d2[i]) (fp64 accumulation, fixed order): the
 *   clustering cost `distance.min(axis=1).sum()` of _kcluster.py:163-170 and :312-316.
 *   ws as for hkm_functional_value_f32.
 * hkm_min_merge_sum_f32: min_d2[i] = min(min_d2[i], new_d2[i]) in place and *out = sum_i
 *   sqrt(min_d2[i]) of the merged array (the same sum hkm_min_dist_sum_f32 returns for it).  The
 *   reference recomputes the distances to ALL candidates in every round (_kcluster.py:312-313); the
 *   minimum over the grown candidate set is the minimum of the previous one and the distances to the
 *   round's new candidates, which is what this merges.  ws as for hkm_functional_value_f32.
 * hkm_sample_select_f32: row i is a candidate iff u[i] <= (oversampling * sqrt(min_d2[i])) /
 *   max(*cost, 1e-12) in fp32 (_kcluster.py:314-322: `where(sample <= prob)`); the selected row
 *   indices are written to idx in ascending order (at most cap of them) and their number, which may
 *   exceed cap, to *count.  cost and count are device pointers, no host synchronisation.
 *   ws needs hkm_workspace_bytes(N, 1, 1, HKM_WS_ASSIGN) bytes.
 * hkm_label_counts_i64: counts[k] = #{i : labels[i] == k}, the candidate weights of
 *   _kcluster.py:206-208; labels outside [0, K) are ignored.
 */
int hkm_min_dist_sum_f32(const float* min_d2, int64_t N, float* out, void* ws, size_t ws_bytes,
                         void* hip_stream);
int hkm_min_merge_sum_f32(float* min_d2, const float* new_d2, int64_t N, float* out, void* ws, size_t ws_bytes,
                          void* hip_stream);
int hkm_sample_select_f32(const float* min_d2, const float* u, int64_t N, const float* cost,
                          float oversampling, int64_t* idx, int64_t cap, int64_t* count, void* ws,
                          size_t ws_bytes, void* hip_stream);
int hkm_label_counts_i64(const int32_t* labels, int64_t N, int32_t K, int64_t* counts,
                         void* hip_stream);

/*
 * k-means++ seeding of a small row set in one launch: the reclustering of the k-means|| candidates
 * (heat/cluster/_kcluster.py:216-225 -> heat/cluster/batchparallelclustering.py:22-46).
 *   idx[0] = first;  for k = 1 .. K-1:  dist_i = min over the chosen rows of the p-norm distance
 *   (p = 2: sqrt(sum (x_i - c)^2), p = 1: sum |x_i - c|), mass_i = w_i * dist_i in fp32 (w = NULL: 1),
 *   idx[k] = the first row whose inclusive prefix sum of the mass (fp64, row order) exceeds
 *   u[k-1] * total, u[k-1] in [0, 1).
 * The reference draws with torch.multinomial from torch's unseeded global generator, which cannot be
 * reproduced; the inverse-CDF draw from caller-supplied uniform numbers is the same distribution.
 * A row without mass (every chosen row) is never drawn.  If the total mass is not positive the
 * remaining entries of idx are set to -1 (torch.multinomial raises there).
 * 1 <= M <= HKM_SEED_MAX_ROWS, 0 <= first < M, K >= 1, p in {1, 2}; X, w, u, idx are device pointers.
 */
#define HKM_SEED_MAX_ROWS 16384
/* The same draws for up to HKM_SEED_ROWS_MAX rows (BatchParallelKMeans / BatchParallelKMedians seed their
 * local rows this way, heat/cluster/batchparallelclustering.py:22-46,270-276; the reference subsamples
 * larger sets to 2^24 - 1 rows first).  Two launches per centre, all enqueued without a host round
 * trip: one read of X that updates the running distances and sums their mass per block of rows, and
 * one workgroup that finds the block and then the row holding u[k-1] * total.  Prefix sums are taken
 * over blocks in block order and inside the chosen block in row order.
 * ws needs hkm_workspace_bytes(M, 1, 1, HKM_WS_ASSIGN | HKM_WS_SSE) bytes. */
#define HKM_SEED_ROWS_MAX 16777216
int hkm_seed_plus_plus_f32(const float* X, int32_t M, int32_t D, int64_t ldx, const float* w, int32_t first,
                           const float* u, int32_t K, int32_t p, int64_t* idx, void* hip_stream);
int hkm_seed_plus_plus_rows_f32(const float* X, int64_t M, int32_t D, int64_t ldx, const float* w, int64_t first,
                                const float* u, int32_t K, int32_t p, int64_t* idx, void* ws, size_t ws_bytes,
                                void* hip_stream);

/*
 * Manhattan-metric siblings for k-medians / k-medoids (heat/cluster/kmedians.py:60-106,
 * heat/cluster/kmedoids.py:57-115, heat/cluster/batchparallelclustering.py:49-97 with p = 1).
 *
 * hkm_assign_l1_f32: labels[i] = argmin_k sum_d |x_id - c_kd| (first index on ties), min_dist[i] = that
 *   minimum (may be NULL); the N x K matrix of manhattan(x, c) (heat/spatial/distance.py:106-133) is
 *   never written.  Replaces _KCluster._assign_to_cluster with the Manhattan metric.
 * hkm_closest_rows_l1_f32: idx[m] = argmin_i sum_d |x_id - q_md| over ALL rows of X (first index on
 *   ties), dist[m] = that distance (may be NULL): the snap of a median to the closest sample of
 *   kmedoids.py:91-106.  ws needs hkm_workspace_bytes(N, D, M, HKM_WS_MEDIAN) bytes.
 * hkm_update_median_f32: C_new[k][d] = median over {i : labels[i] == k} of x_id.
 *   mode 0: percentile 50 with linear interpolation as heat/core/statistics.py computes it on the
 *           float64 `x * selection`: the middle value, or lo + (hi - lo) * 0.5 in fp64 rounded to fp32;
 *   mode 1: the lower of the two middle values (torch.median, batchparallelclustering.py:77).
 *   skip_zero_rows != 0 leaves out rows that are entirely zero, as kmedians.py:93-96 does.
 *   An empty cluster takes the data row fallback_rows[k] (int64[K] device array) if that pointer is
 *   given, else keeps C_old[k] if given, else becomes a zero row.  counts (int64[K]) may be NULL.
 *   ws needs hkm_workspace_bytes(N, D, K, HKM_WS_MEDIAN) bytes.
 */
int hkm_assign_l1_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                      int64_t ldc, int32_t* labels, float* min_dist, void* hip_stream);
int hkm_closest_rows_l1_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* Q, int32_t M,
                            int64_t ldq, int64_t* idx, float* dist, void* ws, size_t ws_bytes,
                            void* hip_stream);
int hkm_update_median_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                          const int64_t* fallback_rows, const float* C_old, float* C_new, int64_t ldcn,
                          int64_t* counts, int32_t mode, int32_t skip_zero_rows, void* ws, size_t ws_bytes,
                          void* hip_stream);
/*
 * The medoid snap in the reference's precision (heat/cluster/kmedoids.py:91-106 measures float64
 * distances from the float64 rows of `x` to the float64 median):
 * hkm_update_median_q64_f32 is hkm_update_median_f32 that also returns every median BEFORE it is
 *   rounded to float32 (medians_f64, K x D dense; it differs from C_new for even counts in mode 0);
 * hkm_closest_rows_l1_q64_f32 is hkm_closest_rows_l1_f32 for float64 queries Q (M x D dense) with every
 *   distance summed in float64 from the float32 rows widened on the way; the row splits are merged in
 *   row order, so of two rows at EXACTLY the same distance -- the two members of a cluster on either
 *   side of their midpoint, the two middle values of a one-dimensional cluster -- the first wins, as
 *   with the reference's argmin.  In float32 against a rounded median such rows come out one rounding
 *   error apart in either direction.  dist (M doubles) may be NULL.  Same workspace as the f32 forms.
 */
int hkm_update_median_q64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                              const int64_t* fallback_rows, const float* C_old, float* C_new, int64_t ldcn,
                              int64_t* counts, int32_t mode, int32_t skip_zero_rows, double* medians_f64, void* ws,
                              size_t ws_bytes, void* hip_stream);
int hkm_closest_rows_l1_q64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const double* Q, int32_t M,
                                int64_t* idx, double* dist, void* ws, size_t ws_bytes, void* hip_stream);

/*
 * k nearest rows and their label vote: the predict chain of the k-nearest-neighbours classifier,
 *   distances = cdist(x, self.x); _, indices = topk(distances, k, largest=False);
 *   classes = argmax(sum(self.y[indices], axis=1), axis=1)
 * heat/classification/kneighborsclassifier.py:114-132 (heat/spatial/distance.py:17-29 for the metric,
 * heat/core/manipulations.py `topk` for the selection), without the M x N distance matrix.
 *
 * hkm_knn_f32: for every row of Q (M x D) the k closest rows of X (N x D) in the Euclidean metric:
 *   idx (M x k int64, leading dimension ldi) in ascending order of (distance, row index) -- of rows at
 *   exactly the same squared distance the smaller index comes first -- and, if dist is not NULL, the
 *   distances themselves (M x k float32, leading dimension ldd).  For D < 16 and D > 128 the squared
 *   distance is summed directly as sum (q - x)^2 in fp32; for 16 <= D <= 128 it is the clamped expansion
 *   max(0, (|x|^2 - 2 q.x) + |q|^2) with the products on the matrix cores, accumulated onto |x|^2 (the form
 *   torch.cdist itself takes above 25 rows, in another order of additions): it carries an absolute error of up
 *   to about 4e-7 (|q|^2 + |x|^2), so a row identical to
 *   the query may come back at a small non-zero distance and rows whose squared distances are closer than
 *   that may swap places.  The square root is correctly rounded.  A slot for which no finite distance
 *   is left (NaN or overflowing rows) holds index -1 and distance inf.  1 <= k <= min(N, HKM_KNN_MAX_K).
 *   ws needs hkm_knn_workspace_bytes(M, N) bytes.
 * hkm_knn_vote_f32: classes[m] = the first index of the largest entry of sum_j Y[idx[m][j]] (Y: N x C
 *   float32 label rows, one-hot or weights; the neighbours are added in their order; index -1 is skipped).
 */
#define HKM_KNN_MAX_K 1024
size_t hkm_knn_workspace_bytes(int64_t M, int64_t N);
int hkm_knn_f32(const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx, int32_t D, int32_t k,
                int64_t* idx, int64_t ldi, float* dist, int64_t ldd, void* ws, size_t ws_bytes, void* hip_stream);
int hkm_knn_vote_f32(const int64_t* idx, int64_t M, int32_t k, int64_t ldi, const float* Y, int64_t N, int32_t C,
                     int64_t ldy, int64_t* classes, void* hip_stream);

/*
 * hkm_cluster_distance_sums_f32: S[i][c] = sum over the rows j of cluster c of the Euclidean distance
 * |x_i - x_j| (direct form, correctly rounded square root, float64 accumulation rounded to float32 at the
 * end) -- `clust_dists = matmul(cdist(X, X), labels == unique_labels)` of silhouette_samples,
 * heat/cluster/metrics.py:135-151, without the N x N matrix.  The caller groups the rows by cluster:
 * perm (int64[N]) lists the row indices cluster by cluster, offsets (int64[K + 1]) the start of every
 * cluster in perm (offsets[0] = 0, offsets[K] = N; device arrays, whose contents are not checked: an
 * index outside [0, N) reads outside X).  S is N x K float32 with leading dimension lds.
 */
int hkm_cluster_distance_sums_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int64_t* perm,
                                  const int64_t* offsets, int32_t K, float* S, int64_t lds, void* hip_stream);
/*
 * hkm_silhouette_finish_f32: the silhouette coefficient of every sample from those sums
 * (heat/cluster/metrics.py:153-176): a = S[i][own] / max(n_own - 1, 1), b = min over the other clusters
 * of S[i][c] / n_c, out[i] = (b - a) / max(a, b); 0 for a sample alone in its cluster and where the
 * quotient is not a number (one cluster only).  labels (int64[N]) are the cluster numbers 0 .. K-1 of the
 * samples, counts (int64[K]) the cluster sizes (labels outside [0, K) read outside S: not checked here).
 * Also serves metric="precomputed" with S = matmul(D, labels == unique_labels).
 */
int hkm_silhouette_finish_f32(const float* S, int64_t N, int32_t K, int64_t lds, const int64_t* labels,
                              const int64_t* counts, float* out, void* hip_stream);

/*
 * hkm_laplacian_f32: graph Laplacian L (N x N, leading dimension ldl; may be S itself) from a similarity
 * matrix S (N x N, leading dimension lds) -- Laplacian.construct after the similarity call,
 * heat/graph/laplacian.py:63-98,119-142: the diagonal of S is zeroed, then
 *   mode 0 (fully_connected) A = S; mode 1 (eNeighbour, upper) keeps entries < eps; mode 2 (lower) keeps
 *   entries > eps; weighted != 0 keeps their values, else a kept entry counts 1 (the zeroed diagonal goes
 *   through the same test, so an unweighted upper graph has ones on its diagonal, as in the reference);
 *   degree[i] (N floats, output) = sum_j A[i][j];
 *   definition HKM_LAPLACIAN_SIMPLE: L = diag(degree) - A;
 *   definition HKM_LAPLACIAN_NORM_SYM: L = -(A / sqrt(d_i)) / sqrt(d_j) with zero degrees taken as 1, and
 *   ones on the diagonal.
 * N <= 65535 * 256 = 16 776 960.  hkm_laplacian_f64 is the same on float64 matrices (the reference keeps float64 similarities in
 * float64).  The reference's unweighted simple Laplacian is an integer matrix: its entries are small whole
 * numbers here, which the caller may cast.
 */
#define HKM_LAPLACIAN_SIMPLE 0
#define HKM_LAPLACIAN_NORM_SYM 1
int hkm_laplacian_f32(const float* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                      float eps, float* L, int64_t ldl, float* degree, void* hip_stream);
int hkm_laplacian_f64(const double* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                      double eps, double* L, int64_t ldl, double* degree, void* hip_stream);

/*
 * float64 data.  The reference keeps float64 inputs in float64 through the same op sequence
 * (promote(X, Y, float32), heat/spatial/distance.py:392-403; heat/cluster/kmeans.py:76-148), so these
 * mirror the *_f32 entry points of the same name with double operands: quadratic-expansion distance +
 * argmin, deterministic per-cluster mean (sums in fp64, count through fp32 as in the reference), one
 * Lloyd iteration, centroid shift, clustering functional, full pairwise matrices.  Pointers must be
 * 8-byte aligned; workspaces are sized with HKM_WS_F64 added to the flags (hkm_update_f64:
 * HKM_WS_UPDATE | HKM_WS_F64, hkm_lloyd_step_f64: HKM_WS_LLOYD | HKM_WS_F64 [| HKM_WS_SSE],
 * hkm_functional_value_f64: as the f32 one).  Labels stay int32.  These run on the fp64 vector ALU
 * and read X twice per iteration; they are not the tuned path.
 */
int hkm_assign_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const double* C, int32_t K,
                   int64_t ldc, int32_t* labels, double* min_d2, void* hip_stream);
int hkm_update_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                   double* C_new, int64_t ldcn, int64_t* counts, void* ws, size_t ws_bytes,
                   void* hip_stream);
int hkm_lloyd_step_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const double* C, double* C_new,
                       int32_t K, int32_t* labels, double* shift, double* sse, void* ws, size_t ws_bytes,
                       void* hip_stream);
int hkm_shift_f64(const double* C_old, const double* C_new, int32_t K, int32_t D, double* shift,
                  void* hip_stream);
int hkm_functional_value_f64(const double* min_d2, int64_t N, double* out, void* ws, size_t ws_bytes,
                             void* hip_stream);
int hkm_pairwise_f64(const double* X, int64_t M, int64_t ldx, const double* Y, int64_t Nn, int64_t ldy,
                     int32_t D, double* out, int64_t ldo, int32_t metric, double sigma, void* hip_stream);

/* out[i] = (int64) in[i]: the (N, 1) int64 labels the reference returns (_operations.py:516-522). */
int hkm_widen_labels_i64(const int32_t* in, int64_t N, int64_t* out, void* hip_stream);

/* Name of the kernel family hkm_assign_f32 would launch for this shape ("valu", "valu_fused", "valu_wide" = few
 * clusters of 17 to 64 features, "mfma_resident", "mfma_tiled", "mfma_stream"); host pointer, static storage.  For
 * benchmarks and profiles. */
const char* hkm_assign_kernel_name(int64_t N, int32_t D, int32_t K);

/* Same for hkm_lloyd_step_f32: "lloyd_small", "lloyd_few" and "lloyd_mfma_resident" read X once per step (labels
 * and per-cluster sums in one kernel); every other shape runs "<assign kernel>+update" (two reads of X). */
const char* hkm_lloyd_kernel_name(int64_t N, int32_t D, int32_t K);

#ifdef __cplusplus
}
#endif
#endif /* HKM_H */
