// Internal declarations shared by the translation units of libhkm (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <algorithm>
#include <stdint.h>

#include "hkm.h"

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define HKM_WAVE 64
#define HKM_INF __builtin_inff()

namespace hkm {

#ifdef __HIPCC__
// Orders a wave's LDS accesses across its lanes for the COMPILER: seen from one lane, a store and a
// later load of another lane's address have no dependence, so without this a load may be merged with
// an earlier one or moved across the store.  The hardware runs one wave's LDS operations in order,
// so nothing is emitted.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Correctly rounded square root of t = 0, +inf, NaN or any finite t >= 2^-96: the hardware square root
// (1 ulp) followed by a two-sided test of its neighbours against the exact residual.  Equal to sqrtf
// on every such input (checked exhaustively on the device; the first disagreement lies below 2^-104,
// where the residual underflows) at half of its instruction count: no range scaling, no class test.
// Zero, infinity and NaN fall through because every comparison against a NaN residual is false.
__device__ __forceinline__ float sqrt_rn_short(float t) {
    const float s = __builtin_amdgcn_sqrtf(t);
    const float sd = __uint_as_float(__float_as_uint(s) - 1u), su = __uint_as_float(__float_as_uint(s) + 1u);
    const float ed = fmaf(-sd, s, t), eu = fmaf(-su, s, t);
    float r = ed <= 0.f ? sd : s;
    r = eu > 0.f ? su : r;
    return r;
}
// Sum of one value per thread over the workgroup (power-of-two size, sh holds blockDim.x doubles) as a
// fixed binary tree: the result depends on the values only, never on scheduling.
__device__ __forceinline__ double block_sum_fixed(double v, double* sh) {
    const int tid = threadIdx.x;
    sh[tid] = v;
    __syncthreads();
    for (int w = blockDim.x / 2; w > 0; w >>= 1) {
        if (tid < w) sh[tid] += sh[tid + w];
        __syncthreads();
    }
    const double r = sh[0];
    __syncthreads();
    return r;
}

// Key that orders non-negative floats with zero moved to the top: a minimum over keys below
// SQRT_SHORT_KEY_LIMIT means some value is positive and below 2^-96, outside sqrt_rn_short's range.
__device__ __forceinline__ unsigned sqrt_short_key(float t) { return __float_as_uint(t) - 1u; }
static constexpr unsigned SQRT_SHORT_KEY_LIMIT = 0x0f800000u - 1u;
#endif


// ---- error plumbing (hkm_api.hip) -----------------------------------------------------------
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- kernel family selection ------------------------------------------------------------------
enum AssignKind { ASSIGN_VALU = 0, ASSIGN_MFMA_RESIDENT = 1, ASSIGN_MFMA_STREAM = 2, ASSIGN_MFMA_TILED = 3 };
AssignKind assign_kind(int32_t D, int32_t K);

// padded feature count used by the resident MFMA kernels (8, 16, 24, 32, 48, 64, 96 or 128)
static const int RESIDENT_MAX_D = 128;
static inline int resident_dp(int32_t D) {
    return D <= 8 ? 8 : D <= 16 ? 16 : D <= 24 ? 24 : D <= 32 ? 32 : D <= 48 ? 48 : D <= 64 ? 64 : D <= 96 ? 96 : 128;
}
static inline size_t resident_lds_bytes(int32_t D, int32_t K) {
    size_t kp = (size_t(K) + 31) / 32 * 32;
    return kp * (resident_dp(D) + 5) * sizeof(float);  // rows of DP + 4 floats, plus the squared norms
}

// ---- geometry of the deterministic update ----------------------------------------------------
struct UpdateGeom {
    int64_t rows_per_chunk;  // rows summed in fp32 inside one workgroup before the fp64 reduction
    int32_t S;               // number of row chunks
    int32_t J;               // number of 32-column slices of D
    int32_t Z;               // number of cluster ranges
    int32_t KR;              // clusters per range (LDS accumulator rows)
};
UpdateGeom update_geom(int64_t N, int32_t D, int32_t K, int32_t elem = 4);

// scratch of the sorted update (hkm_update_sorted.hip)
struct SortedWorkspace {
    int32_t* blk_cnt;      // [blocks][K] label counts of every block, then positions inside the cluster's segment
    int64_t* counts;       // [K]
    int64_t* offsets;      // [K + 1]
    int32_t* chunk_start;  // [K + 1]
    int32_t* perm;         // [N] row indices grouped by cluster, ascending inside a cluster
    void* part;            // [chunks][D padded to 32] partial sums (float or double)
    double* shift_part;
    size_t total;
};
SortedWorkspace carve_sorted(void* base, int64_t N, int32_t D, int32_t K, int32_t elem);
bool sorted_update_eligible(int32_t K);

// ---- workspace layout --------------------------------------------------------------------------
struct Workspace {
    float* cn;          // squared centroid norms, padded to a multiple of 128 with +inf
    unsigned long long* keys;  // [N] packed (d2 bits, index) merge keys of the streaming kernel
    float* part_sum;    // [S][K][J*32] fp32 partial sums
    int32_t* part_cnt;  // [S][K]
    int64_t* counts;    // [K]
    double* red;        // [RED_SLOTS] scratch for scalar reductions
    float* min_d2;      // [N] (only with the SSE flag)
    double* shift_part; // [ceil(K*D/64)] per-block shares of the squared centroid shift
    double* small_part; // [SMALL_MAX_GRID][K*(D+1)+1] partial rows of the one-sweep small-D step
    int32_t* small_flags;  // [SMALL_MAX_GRID] 1 = this workgroup's integer sums cannot be trusted
    double* fsum;       // [FUSED_MAX_GRID][K][D] fp64 partial sums of the one-sweep MFMA step
    int32_t* fcnt;      // [FUSED_MAX_GRID][K]
    int32_t* fflags;    // [FUSED_MAX_GRID] 1 = this workgroup's sums may depend on the addition order
    int32_t* lazy_lab;  // [N] labels of a step that ran without storing any, computed only when a flag is up
    SortedWorkspace srt; // scratch of the sorted update (with the UPDATE flag, K <= 4096)
    size_t total;
};
static const int RED_SLOTS = 2048;
static const int SMALL_MAX_GRID = 2048;
static const int FUSED_MAX_GRID = 512;
Workspace carve(void* base, int64_t N, int32_t D, int32_t K, int32_t flags);

// scratch of the per-cluster median (hkm_l1.hip)
struct MedianWorkspace {
    int32_t* eff;          // [N] label, or -1 for a row left out
    int32_t* perm;         // [N] row indices grouped by cluster
    int64_t* counts;       // [K]
    int64_t* offsets;      // [K + 1]
    int32_t* chunk_start;  // [K + 1]
    int32_t* cursor;       // [K]
    unsigned* prefix;      // [K * D]
    int64_t* rank;         // [K * D]
    unsigned* eqcnt;       // [K * D]
    unsigned* next;        // [K * D]
    unsigned* hist;        // [K * D * 256]
    unsigned long long* keys;  // [K] merge keys of the closest-row search
    double* snap_d;        // [closest64_slots(K)] best distance of every (split, query) of the float64 snap
    unsigned* snap_i;      // [closest64_slots(K)] and its row
    size_t total;
};
MedianWorkspace carve_median(void* base, int64_t N, int32_t D, int32_t K);
int64_t closest64_slots(int32_t M);
int launch_closest_rows_l1_q64(const float* X, int64_t N, int32_t D, int64_t ldx, const double* Qm, int32_t M,
                               int64_t* idx, double* dist, double* part_d, unsigned* part_i, hipStream_t st);

// ---- launchers (one per .hip file) ------------------------------------------------------------
int launch_norms(const float* C, int32_t K, int32_t D, int64_t ldc, float* cn, int32_t kpad,
                 hipStream_t st);
int launch_assign_valu(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                       int64_t ldc, int32_t* labels, float* min_d2, hipStream_t st);
int launch_assign_mfma_resident(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                                int32_t K, int64_t ldc, int32_t* labels, float* min_d2,
                                hipStream_t st);
int launch_assign_mfma_tiled(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                             int32_t K, int64_t ldc, const float* cn, int32_t* labels,
                             float* min_d2, bool split, hipStream_t st);
int launch_assign_mfma_stream(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                              int32_t K, int64_t ldc, const float* cn, unsigned long long* keys,
                              int32_t* labels, float* min_d2, bool split, hipStream_t st);
bool fused_eligible(int32_t D, int32_t K);
size_t fused_lds_bytes(int32_t D, int32_t K);
int fused_grid(int64_t N, int32_t D);
// point blocks per wave of the resident matrix-core kernels (hkm_assign_mfma.hip): the choice for a padded
// width and its sources (environment, what the trial on the caller's own steps found on the current device:
// 0 while it has no verdict; trial_report also hands out the per-step times of its last two windows)
int resident_point_blocks(int dp);
int env_point_blocks();
int tuned_point_blocks();
int trial_report(float* ms_two, float* ms_one);
int launch_lloyd_mfma_resident(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                               int32_t K, int64_t ldc, int32_t* labels, float* min_d2, double* fsum,
                               int32_t* fcnt, int32_t* flags, hipStream_t st);
int launch_update_fused(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                        int32_t K, float* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                        int fgrid, const float* C_old, float* shift, hipStream_t st);
// few clusters of wide rows on the vector ALU (hkm_lloyd_few.hip); fsum == nullptr: the assignment alone
bool few_eligible(int32_t D, int32_t K);
int few_grid(int64_t N, int32_t D, int32_t K);
int launch_few(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K, int64_t ldc,
               int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt, int32_t* flags, hipStream_t st,
               const int32_t* gate = nullptr, int ngate = 0);
// the whole Lloyd loop in one launch (hkm_lloyd_fit.hip)
static const int FIT_MAX_GRID = 64;
static const int64_t FIT_MAX_ROWS = int64_t(1) << 18;
bool fit_eligible(int64_t N, int32_t D, int32_t K);
int fit_grid(int64_t N, int32_t D);
size_t fit_workspace_bytes(int32_t D, int32_t K);
int launch_lloyd_fit(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C0, int32_t K, int32_t max_iter,
                     int32_t use_tol, double tol, float* C_out, int64_t* labels, float* shift_out, int32_t* info,
                     void* ws, uint64_t wait_limit_ticks, hipStream_t st);
bool small_eligible(int32_t D, int32_t K);
int small_grid(int64_t N, int32_t D, int32_t K);
// labels64: `labels` points to N 64-bit integers instead of 32-bit ones
int launch_small(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                 int64_t ldc, int32_t* labels, float* min_d2, double* part, int mode, int32_t* flags,
                 hipStream_t st, bool labels64 = false);
int launch_small_finalize(const double* part, int grid, int32_t K, int32_t D, const float* C_old,
                          float* C_new, int64_t ldcn, int64_t* counts, float* shift, float* sse,
                          hipStream_t st);
int launch_update(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                  int32_t K, float* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                  const float* C_old, float* shift, hipStream_t st);
int launch_update_sorted(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                         float* C_new, int64_t ldcn, int64_t* counts, const SortedWorkspace& w,
                         const float* C_old, float* shift, hipStream_t st);
int launch_update_sorted_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                             int32_t K, double* C_new, int64_t ldcn, int64_t* counts,
                             const SortedWorkspace& w, const double* C_old, double* shift, hipStream_t st);
int launch_update_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                      int32_t K, double* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                      const double* C_old, double* shift, hipStream_t st);
int launch_shift_f64(const double* C_old, const double* C_new, int32_t K, int32_t D, double* shift,
                     hipStream_t st);
int launch_sum_min_d2_f64(const double* v, int64_t N, double* out, double* red, int mode,
                          hipStream_t st);
int launch_assign_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const double* C, int32_t K,
                      int64_t ldc, int32_t* labels, double* min_d2, hipStream_t st);
int launch_cdist_f64(const double* X, int64_t M, int64_t ldx, const double* Y, int64_t Nn, int64_t ldy,
                     int32_t D, double* out, int64_t ldo, int32_t metric, int32_t sqrt_flag, double gauss,
                     hipStream_t st);
int launch_shift(const float* C_old, const float* C_new, int32_t K, int32_t D, float* shift,
                 hipStream_t st);
int launch_sum_min_d2(const float* min_d2, int64_t N, float* out, double* red, int mode,
                      hipStream_t st);
int launch_min_merge_sum(float* dmin, const float* dnew, int64_t N, float* out, double* red, hipStream_t st);
bool split_eligible(int32_t D, int32_t K, bool fused);
int split_fused_grid(int64_t N);
int launch_split_resident(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt,
                          int32_t* flags, hipStream_t st);
bool cdist_mfma_eligible(int64_t M, int64_t Nn, int32_t D, int64_t ldx, int64_t ldy, int64_t ldo);
int launch_cdist_mfma(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                      int32_t D, float* out, int64_t ldo, int32_t sqrt_flag, float gauss, hipStream_t st);
int launch_cdist(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                 int32_t D, float* out, int64_t ldo, int32_t metric, int32_t sqrt_flag, float gauss,
                 hipStream_t st);
int launch_select(const float* d2, const float* u, int64_t N, const float* cost, float os,
                  int64_t* idx, int64_t cap, int64_t* count, double* red, hipStream_t st);
int launch_label_counts(const int32_t* labels, int64_t N, int32_t K, int64_t* counts,
                        hipStream_t st);
int launch_seed_plus_plus(const float* X, int32_t M, int32_t D, int64_t ldx, const float* w, int32_t first,
                          const float* u, int32_t K, int32_t p, int64_t* idx, hipStream_t st);
int launch_seed_plus_plus_rows(const float* X, int64_t M, int32_t D, int64_t ldx, const float* w, int64_t first,
                               const float* u, int32_t K, int32_t p, int64_t* idx, float* dist, double* red,
                               hipStream_t st);
int launch_assign_l1(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                     int64_t ldc, int32_t* labels, float* min_dist, hipStream_t st);
int launch_closest_rows_l1(const float* X, int64_t N, int32_t D, int64_t ldx, const float* Qm,
                           int32_t M, int64_t ldq, int64_t* idx, float* dist,
                           unsigned long long* keys, hipStream_t st);
int launch_update_median(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                         int32_t K, const int64_t* fallback_rows, const float* C_old, float* C_new,
                         int64_t ldcn, int64_t* counts_out, int32_t mode, int32_t skip_zero_rows,
                         const MedianWorkspace& w, hipStream_t st, double* med64 = nullptr);
int launch_widen(const int32_t* in, int64_t N, int64_t* out, hipStream_t st);

int num_cus();
// benchmark timing of the dominant kernel: no-ops unless hkm_profile_enable(1) was called on this thread
void prof_begin(hipStream_t st);
void prof_end(hipStream_t st);

// k nearest rows (hkm_knn.hip).  The split of the reference rows over workgroups and the scratch it needs
// follow from the two row counts alone, so that the workspace can be sized before the call.
struct KnnPlan {
    int nsplit;
    int64_t rows_per_split;
    size_t part_slots;  // (distance, row) pairs of the per-split lists; 0 when one split covers all rows
};
KnnPlan knn_plan(int64_t M, int64_t N, int target);
int knn_max_target_workgroups();
int launch_knn(const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx, int32_t D, int32_t k,
               int64_t* idx, int64_t ldi, float* dist, int64_t ldd, float* xn, float* last_d2, unsigned* last_i,
               float* part_d, unsigned* part_i, hipStream_t st);
bool knn_uses_mfma(int32_t D);
int launch_knn_vote(const int64_t* idx, int64_t M, int32_t k, int64_t ldi, const float* Y, int64_t N, int32_t C,
                    int64_t ldy, int64_t* classes, hipStream_t st);

// per-sample, per-cluster sums of Euclidean distances (hkm_silhouette.hip)
int launch_silhouette_finish(const float* S, int64_t N, int32_t K, int64_t lds, const int64_t* enc,
                             const int64_t* counts, float* out, hipStream_t st);
int launch_silhouette_sums(const float* X, int64_t N, int32_t D, int64_t ldx, const int64_t* perm,
                           const int64_t* offsets, int32_t K, float* S, int64_t lds, hipStream_t st);

// graph Laplacian from a similarity matrix (hkm_laplacian.hip)
int launch_laplacian(const float* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                     float eps, float* L, int64_t ldl, float* degree, hipStream_t st);
int launch_laplacian_f64(const double* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                         double eps, double* L, int64_t ldl, double* degree, hipStream_t st);

}  // namespace hkm
