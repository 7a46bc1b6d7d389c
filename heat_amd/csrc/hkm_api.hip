// C ABI of libhkm: host-side validation, workspace carving and kernel dispatch.
// Nothing here allocates device memory or synchronises; every entry point only enqueues kernels.
#include <pthread.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "hkm_bench.h"
#include "hkm_common.h"

namespace hkm {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HKM_EHIP, "%s: %s", what, hipGetErrorString(e));
    return HKM_OK;
}

// ---- timing of the dominant kernel (benchmarks only; off unless hkm_profile_enable(1) was called) ----
// Per calling thread: a ring of event pairs recorded on the launch stream right before and right after
// the launch of the distance kernel of hkm_assign_f32 / hkm_lloyd_step_f32, read back (and waited for) by
// hkm_profile_collect.  Nothing is recorded, created or kept while profiling is off.
static const int PROF_RING = 512;
struct ProfState {
    int on = 0;
    int count = 0;  // pairs recorded since the last collect
    hipEvent_t ev[PROF_RING][2] = {};
    bool made[PROF_RING] = {};
};
static thread_local ProfState g_prof;

void prof_begin(hipStream_t st) {
    ProfState& p = g_prof;
    if (!p.on || p.count >= PROF_RING) return;
    const int i = p.count;
    if (!p.made[i]) {
        if (hipEventCreate(&p.ev[i][0]) != hipSuccess || hipEventCreate(&p.ev[i][1]) != hipSuccess) return;
        p.made[i] = true;
    }
    (void)hipEventRecord(p.ev[i][0], st);
}

void prof_end(hipStream_t st) {
    ProfState& p = g_prof;
    if (!p.on || p.count >= PROF_RING || !p.made[p.count]) return;
    (void)hipEventRecord(p.ev[p.count][1], st);
    p.count++;
}

int num_cus() {
    static thread_local int cached_dev = -1;
    static thread_local int cached_cus = 256;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cached_cus = n;
        cached_dev = dev;
    }
    return cached_cus;
}

// Up to 16 features the vector kernel (one point per lane, K * (D + 3) instructions per point) competes with
// the matrix cores, whose work comes in blocks of 32 centroids and 8 features with a fixed epilogue per
// block.  Measured on 10M rows: for the assignment alone the matrix cores win from about 32 centroids on
// (16 features: equal at 16, 1.4x at 24; 9 features and 16 centroids: the vector kernel is 2x faster), and
// below 4 features three quarters of their work would be padding (HKM_NARROW_MFMA_MIN_K in the environment
// moves the threshold).  The one-sweep step is another matter: see fused_eligible.
static const int NARROW_MFMA_MIN_K = 32;
static int narrow_mfma_min_k() {
    const char* e = getenv("HKM_NARROW_MFMA_MIN_K");
    if (e && e[0]) {
        const int v = atoi(e);
        if (v > 0) return v;
    }
    return NARROW_MFMA_MIN_K;
}

AssignKind assign_kind(int32_t D, int32_t K) {
    if (D <= 16 && (D < 4 || K < narrow_mfma_min_k())) return ASSIGN_VALU;
    if (D <= RESIDENT_MAX_D && resident_lds_bytes(D, K) <= 64 * 1024) return ASSIGN_MFMA_RESIDENT;
    if (D <= 64) return ASSIGN_MFMA_TILED;
    return ASSIGN_MFMA_STREAM;
}

// The one-sweep MFMA step needs the centroids, fp64 accumulators and counts of a workgroup in LDS.  From 2
// features on it is taken whatever K is: what it replaces for narrow rows is the vector assignment PLUS the
// two-pass update, and reading X once beats that 2-3x even with a single centroid or with three quarters of
// the matrix work spent on padding (10M x 16: 0.22 against 1.84 ms at K = 1, 0.24 against 0.79 ms at K = 16;
// 10M x 2, K = 90: 0.28 against 0.55 ms; 10M x 3, K = 256: 0.52 against 0.91 ms).  One feature stays on the
// two passes (0.57 ms at K = 130; with 130 centroids on a line the two arithmetics part on a thousand ties).
bool fused_eligible(int32_t D, int32_t K) {
    return D >= 2 && D <= RESIDENT_MAX_D && resident_lds_bytes(D, K) <= 64 * 1024 && fused_lds_bytes(D, K) <= 160 * 1024;
}

// labels == NULL is accepted by hkm_lloyd_step_f32: the one-sweep steps of the two vector kernels, which memory
// bounds.  (The matrix-core step with few centroids was tried too: 10M x 128, K = 8: 1.203 -> 1.186 ms, 10M x 96,
// K = 32: 0.984 -> 0.972 ms -- its fp64 sums bound it, not the labels; it keeps storing them.)
static bool step_labels_optional(int32_t D, int32_t K) { return small_eligible(D, K) || few_eligible(D, K); }

static size_t cn_pad(int32_t K) { return (size_t(K) + 127) / 128 * 128; }

Workspace carve(void* base, int64_t N, int32_t D, int32_t K, int32_t flags) {
    Workspace w;
    memset(&w, 0, sizeof(w));
    char* p = static_cast<char*>(base);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* r = p ? p + off : nullptr;
        off += align_up(bytes, 256);
        return r;
    };
    w.red = reinterpret_cast<double*>(take(size_t(RED_SLOTS) * sizeof(double)));
    if (flags & HKM_WS_ASSIGN) {
        w.cn = reinterpret_cast<float*>(take(cn_pad(K) * sizeof(float)));
        if (assign_kind(D, K) == ASSIGN_MFMA_STREAM)
            w.keys = reinterpret_cast<unsigned long long*>(take(size_t(N < 1 ? 1 : N) * sizeof(unsigned long long)));
    }
    if ((flags & HKM_WS_UPDATE) && !(flags & HKM_WS_F64) && small_eligible(D, K)) {
        w.small_part = reinterpret_cast<double*>(take(size_t(SMALL_MAX_GRID) * (size_t(K) * (D + 1) + 1) * sizeof(double)));
        w.small_flags = reinterpret_cast<int32_t*>(take(size_t(SMALL_MAX_GRID) * sizeof(int32_t)));
    }
    if (flags & HKM_WS_UPDATE) {
        const size_t elem = (flags & HKM_WS_F64) ? sizeof(double) : sizeof(float);
        const UpdateGeom g = update_geom(N, D, K, int32_t(elem));
        w.part_sum = reinterpret_cast<float*>(take(size_t(g.S) * K * g.J * 32 * elem));
        w.part_cnt = reinterpret_cast<int32_t*>(take(size_t(g.S) * K * sizeof(int32_t)));
        w.counts = reinterpret_cast<int64_t*>(take(size_t(K) * sizeof(int64_t)));
        w.shift_part = reinterpret_cast<double*>(take((size_t(K) * D / 64 + 1) * sizeof(double)));
    }
    if ((flags & HKM_WS_UPDATE) && sorted_update_eligible(K)) {
        const int32_t elem = (flags & HKM_WS_F64) ? 8 : 4;
        w.srt = carve_sorted(p ? p + off : nullptr, N, D, K, elem);
        off += align_up(w.srt.total, 256);
    }
    if ((flags & HKM_WS_LLOYD) == HKM_WS_LLOYD && !(flags & HKM_WS_F64) && fused_eligible(D, K)) {
        w.fsum = reinterpret_cast<double*>(take(size_t(FUSED_MAX_GRID) * K * D * sizeof(double)));
        w.fcnt = reinterpret_cast<int32_t*>(take(size_t(FUSED_MAX_GRID) * K * sizeof(int32_t)));
        w.fflags = reinterpret_cast<int32_t*>(take(size_t(FUSED_MAX_GRID) * sizeof(int32_t)));
        if (few_eligible(D, K)) w.lazy_lab = reinterpret_cast<int32_t*>(take(size_t(N < 1 ? 1 : N) * sizeof(int32_t)));
    }
    if (flags & HKM_WS_SSE)
        w.min_d2 = reinterpret_cast<float*>(
            take(size_t(N < 1 ? 1 : N) * ((flags & HKM_WS_F64) ? sizeof(double) : sizeof(float))));
    w.total = off;
    return w;
}

MedianWorkspace carve_median(void* base, int64_t N, int32_t D, int32_t K) {
    MedianWorkspace w;
    memset(&w, 0, sizeof(w));
    char* p = static_cast<char*>(base);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* r = p ? p + off : nullptr;
        off += align_up(bytes, 256);
        return r;
    };
    const size_t n = size_t(N < 1 ? 1 : N), kd = size_t(K) * D;
    w.eff = reinterpret_cast<int32_t*>(take(n * sizeof(int32_t)));
    w.perm = reinterpret_cast<int32_t*>(take(n * sizeof(int32_t)));
    w.counts = reinterpret_cast<int64_t*>(take(size_t(K) * sizeof(int64_t)));
    w.offsets = reinterpret_cast<int64_t*>(take((size_t(K) + 1) * sizeof(int64_t)));
    w.chunk_start = reinterpret_cast<int32_t*>(take((size_t(K) + 1) * sizeof(int32_t)));
    w.cursor = reinterpret_cast<int32_t*>(take(size_t(K) * sizeof(int32_t)));
    w.prefix = reinterpret_cast<unsigned*>(take(kd * sizeof(unsigned)));
    w.rank = reinterpret_cast<int64_t*>(take(kd * sizeof(int64_t)));
    w.eqcnt = reinterpret_cast<unsigned*>(take(kd * sizeof(unsigned)));
    w.next = reinterpret_cast<unsigned*>(take(kd * sizeof(unsigned)));
    w.hist = reinterpret_cast<unsigned*>(take(kd * 256 * sizeof(unsigned)));
    w.keys = reinterpret_cast<unsigned long long*>(take(size_t(K) * sizeof(unsigned long long)));
    w.snap_d = reinterpret_cast<double*>(take(size_t(closest64_slots(K)) * sizeof(double)));
    w.snap_i = reinterpret_cast<unsigned*>(take(size_t(closest64_slots(K)) * sizeof(unsigned)));
    w.total = off;
    return w;
}

// the two-pass update: stable sort + segmented sums where its per-wave cursors fit in LDS, the
// list-based kernels otherwise.  HKM_UPDATE_LISTS=1 in the environment (looked up per call) forces
// the latter: the one-sweep MFMA step falls back to exactly those kernels, and tests compare the two.
static bool use_sorted_update(int32_t K) {
    const char* e = getenv("HKM_UPDATE_LISTS");
    const bool forced_lists = e && e[0] == '1';
    return sorted_update_eligible(K) && !forced_lists;
}

static int do_update(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                     float* C_new, int64_t ldcn, int64_t* counts, const Workspace& w, const float* C_old,
                     float* shift, hipStream_t st) {
    if (use_sorted_update(K))
        return launch_update_sorted(X, N, D, ldx, labels, K, C_new, ldcn, counts, w.srt, C_old, shift, st);
    return launch_update(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, C_old, shift, st);
}

static int do_update_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                         double* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                         const double* C_old, double* shift, hipStream_t st) {
    if (use_sorted_update(K))
        return launch_update_sorted_f64(X, N, D, ldx, labels, K, C_new, ldcn, counts, w.srt, C_old, shift, st);
    return launch_update_f64(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, C_old, shift, st);
}

static int check_matrix(const char* name, const void* p, int64_t rows, int32_t cols, int64_t ld) {
    if (!p && rows > 0) return fail(HKM_EINVAL, "%s is NULL", name);
    if (reinterpret_cast<uintptr_t>(p) & 3u) return fail(HKM_EINVAL, "%s is not 4-byte aligned", name);
    if (ld < cols) return fail(HKM_EINVAL, "leading dimension of %s (%lld) < columns (%d)", name, (long long)ld, cols);
    return HKM_OK;
}

static int check_matrix64(const char* name, const void* p, int64_t rows, int32_t cols, int64_t ld) {
    if (!p && rows > 0) return fail(HKM_EINVAL, "%s is NULL", name);
    if (reinterpret_cast<uintptr_t>(p) & 7u) return fail(HKM_EINVAL, "%s is not 8-byte aligned", name);
    if (ld < cols) return fail(HKM_EINVAL, "leading dimension of %s (%lld) < columns (%d)", name, (long long)ld, cols);
    return HKM_OK;
}

static int check_shape(int64_t N, int32_t D, int32_t K) {
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    if (K < 1) return fail(HKM_EINVAL, "K = %d must be >= 1", K);
    // sizes no device holds: refused here so that the byte counts computed from them cannot wrap around
    if (N > (int64_t(1) << 40)) return fail(HKM_EUNSUPPORTED, "N = %lld exceeds 2^40 rows", (long long)N);
    if (int64_t(K) * D > (int64_t(1) << 40))
        return fail(HKM_EUNSUPPORTED, "K x D = %lld exceeds 2^40 centroid coordinates", (long long)(int64_t(K) * D));
    return HKM_OK;
}

static int check_ws(void* ws, size_t ws_bytes, size_t need) {
    if (!ws) return fail(HKM_EWORKSPACE, "workspace is NULL (%zu bytes needed)", need);
    if (reinterpret_cast<uintptr_t>(ws) & 255u) return fail(HKM_EWORKSPACE, "workspace is not 256-byte aligned");
    if (ws_bytes < need) return fail(HKM_EWORKSPACE, "workspace too small: %zu bytes given, %zu needed", ws_bytes, need);
    return HKM_OK;
}

// HKM_PRODUCTS=bf16x3 in the environment (looked up per call) evaluates the cross term of the
// resident matrix-core kernels with three-way split bf16 operands instead of fp32 MFMAs
// (hkm_assign_split.hip).  Off by default: the default path computes every product in fp32.
static bool use_split_products() {
    const char* e = getenv("HKM_PRODUCTS");
    return e && strcmp(e, "bf16x3") == 0;
}

static int do_assign(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                     int64_t ldc, int32_t* labels, float* min_d2, const Workspace& w,
                     hipStream_t st) {
    if (N == 0) return HKM_OK;
    switch (assign_kind(D, K)) {
        case ASSIGN_VALU:
            if (small_eligible(D, K))
                return launch_small(X, N, D, ldx, C, K, ldc, labels, min_d2, nullptr, 0, nullptr, st);
            return launch_assign_valu(X, N, D, ldx, C, K, ldc, labels, min_d2, st);
        case ASSIGN_MFMA_RESIDENT:
            // few clusters of wide rows: the vector ALU needs less time than X takes to arrive
            if (few_eligible(D, K)) return launch_few(X, N, D, ldx, C, K, ldc, labels, min_d2, nullptr, nullptr, nullptr, st);
            if (use_split_products() && split_eligible(D, K, false))
                return launch_split_resident(X, N, D, ldx, C, K, ldc, labels, min_d2, nullptr, nullptr, nullptr, st);
            return launch_assign_mfma_resident(X, N, D, ldx, C, K, ldc, labels, min_d2, st);
        case ASSIGN_MFMA_TILED: {
            int rc = launch_norms(C, K, D, ldc, w.cn, int32_t(cn_pad(K)), st);
            if (rc) return rc;
            return launch_assign_mfma_tiled(X, N, D, ldx, C, K, ldc, w.cn, labels, min_d2, use_split_products(), st);
        }
        default: {
            int rc = launch_norms(C, K, D, ldc, w.cn, int32_t(cn_pad(K)), st);
            if (rc) return rc;
            return launch_assign_mfma_stream(X, N, D, ldx, C, K, ldc, w.cn, w.keys, labels, min_d2, use_split_products(), st);
        }
    }
}

}  // namespace hkm

using namespace hkm;

extern "C" {

int hkm_version(void) { return 308; }

const char* hkm_last_error(void) { return g_err; }

int hkm_profile_enable(int32_t on) {
    g_err[0] = 0;
    g_prof.on = on ? 1 : 0;
    g_prof.count = 0;
    return HKM_OK;
}

int hkm_profile_collect(float* ms, int32_t cap, int32_t* count) {
    g_err[0] = 0;
    if (!count || (cap > 0 && !ms) || cap < 0) return fail(HKM_EINVAL, "NULL pointer argument or negative capacity");
    ProfState& p = g_prof;
    int n = 0;
    for (int i = 0; i < p.count; ++i) {
        hipError_t e = hipEventSynchronize(p.ev[i][1]);
        float t = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&t, p.ev[i][0], p.ev[i][1]);
        if (e != hipSuccess) {
            p.count = 0;
            return fail(HKM_EHIP, "hkm_profile_collect: %s", hipGetErrorString(e));
        }
        if (n < cap) ms[n++] = t;
    }
    *count = p.count;
    p.count = 0;
    return HKM_OK;
}

size_t hkm_workspace_bytes(int64_t N, int32_t D, int32_t K, int32_t flags) {
    if (N < 0 || D < 1 || K < 1) return 0;
    if (N > (int64_t(1) << 40) || int64_t(K) * D > (int64_t(1) << 40)) return 0;  // refused by every entry point
    if (flags == HKM_WS_MEDIAN) return carve_median(nullptr, N, D, K).total;
    if (flags == HKM_WS_FIT) return fit_eligible(N, D, K) ? fit_workspace_bytes(D, K) : 0;
    return carve(nullptr, N, D, K, flags).total;
}

const char* hkm_assign_kernel_name(int64_t N, int32_t D, int32_t K) {
    (void)N;
    if (D < 1 || K < 1) return "invalid";
    switch (assign_kind(D, K)) {
        case ASSIGN_VALU: return small_eligible(D, K) ? "valu_fused" : "valu";
        case ASSIGN_MFMA_RESIDENT: return few_eligible(D, K) ? "valu_wide" : "mfma_resident";
        case ASSIGN_MFMA_TILED: return "mfma_tiled";
        default: return "mfma_stream";
    }
}

const char* hkm_lloyd_kernel_name(int64_t N, int32_t D, int32_t K) {
    (void)N;
    if (D < 1 || K < 1) return "invalid";
    if (small_eligible(D, K)) return "lloyd_small";
    if (fused_eligible(D, K)) return few_eligible(D, K) ? "lloyd_few" : "lloyd_mfma_resident";
    switch (assign_kind(D, K)) {
        case ASSIGN_VALU: return "valu+update";
        case ASSIGN_MFMA_RESIDENT: return "mfma_resident+update";
        case ASSIGN_MFMA_TILED: return "mfma_tiled+update";
        default: return "mfma_stream+update";
    }
}

int hkm_assign_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                   int64_t ldc, int32_t* labels, float* min_d2, void* ws, size_t ws_bytes,
                   void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C", C, K, D, ldc))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    const size_t need = carve(nullptr, N, D, K, HKM_WS_ASSIGN).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const Workspace w = carve(ws, N, D, K, HKM_WS_ASSIGN);
    return do_assign(X, N, D, ldx, C, K, ldc, labels, min_d2, w, static_cast<hipStream_t>(hip_stream));
}

int hkm_assign_labels64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                            int64_t ldc, int64_t* labels, float* min_d2, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C", C, K, D, ldc))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    if (reinterpret_cast<uintptr_t>(labels) & 7u) return fail(HKM_EINVAL, "labels is not 8-byte aligned");
    if (!(assign_kind(D, K) == ASSIGN_VALU && small_eligible(D, K)))
        return fail(HKM_EUNSUPPORTED,
                    "D = %d, K = %d: only the narrow kernel (hkm_assign_kernel_name() == \"valu_fused\") stores 64-bit "
                    "labels itself; use hkm_assign_f32 and hkm_widen_labels_i64", D, K);
    if (N == 0) return HKM_OK;
    return launch_small(X, N, D, ldx, C, K, ldc, reinterpret_cast<int32_t*>(labels), min_d2, nullptr, 0, nullptr,
                        static_cast<hipStream_t>(hip_stream), true);
}

// ---- hkm_assign_static_f32: the assignment without a caller-supplied workspace -----------------
// The scratch of the assignment kernels (reduction slots, squared centroid norms, merge keys of the
// streaming kernel) lives in this file-scope device array.  Its name is a host-side handle only: the
// device address is looked up once per device with hipGetSymbolAddress and that pointer is what the
// launchers receive.
static __device__ __align__(256) unsigned char scratch[HKM_STATIC_SCRATCH_BYTES];

static const int STATIC_MAX_DEVICES = 64;
static void* g_scratch_ptr[STATIC_MAX_DEVICES];  // device address of `scratch` on every device, once known
static pthread_mutex_t g_scratch_lock = PTHREAD_MUTEX_INITIALIZER;

// Address of the current device's copy of `scratch` (every device holds its own).
static int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HKM_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES)
        return fail(HKM_EUNSUPPORTED, "device ordinal %d outside 0..%d", dev, STATIC_MAX_DEVICES - 1);
    pthread_mutex_lock(&g_scratch_lock);
    void* p = g_scratch_ptr[dev];
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e == hipSuccess && !p) e = hipErrorInvalidSymbol;
        if (e == hipSuccess) g_scratch_ptr[dev] = p;
    }
    pthread_mutex_unlock(&g_scratch_lock);
    if (e != hipSuccess) return fail(HKM_EHIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    *out = p;
    return HKM_OK;
}

// Also resolves the array's address on the current device, so that a caller who asks for the size first -- the
// documented warm-up -- never meets the symbol lookup inside hkm_assign_static_f32 (a capturing stream may refuse it).
size_t hkm_static_scratch_bytes(void) {
    void* p = nullptr;
    (void)static_scratch(&p);  // a failure (no device) is reported by the entry point that needs the address
    g_err[0] = 0;
    return HKM_STATIC_SCRATCH_BYTES;
}

int hkm_assign_static_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C", C, K, D, ldc))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    const size_t need = carve(nullptr, N, D, K, HKM_WS_ASSIGN).total;
    if (need > HKM_STATIC_SCRATCH_BYTES)
        return fail(HKM_EUNSUPPORTED,
                    "N = %lld, D = %d, K = %d needs %zu bytes of scratch, the built-in array holds %zu: "
                    "use hkm_assign_f32 with a workspace",
                    (long long)N, D, K, need, size_t(HKM_STATIC_SCRATCH_BYTES));
    if (N == 0) return HKM_OK;
    void* base = nullptr;
    if ((rc = static_scratch(&base))) return rc;
    // every kernel that reads the scratch is preceded on the stream by the one that fills it (norms,
    // key fill), so nothing of an earlier call's contents is read
    const Workspace w = carve(base, N, D, K, HKM_WS_ASSIGN);
    return do_assign(X, N, D, ldx, C, K, ldc, labels, min_d2, w, static_cast<hipStream_t>(hip_stream));
}

int hkm_update_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                   int32_t K, float* C_new, int64_t ldcn, int64_t* counts, void* ws,
                   size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C_new", C_new, K, D, ldcn))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    const size_t need = carve(nullptr, N, D, K, HKM_WS_UPDATE).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const Workspace w = carve(ws, N, D, K, HKM_WS_UPDATE);
    return do_update(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, nullptr, nullptr,
                     static_cast<hipStream_t>(hip_stream));
}

// labels64: `labels` points to 64-bit integers (the narrow one-sweep step only)
static int lloyd_step_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, float* C_new, int32_t K,
                          int32_t* labels, bool labels64, float* shift, float* sse, void* ws, size_t ws_bytes,
                          void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C", C, K, D, D))) return rc;
    if ((rc = check_matrix("C_new", C_new, K, D, D))) return rc;
    if (C == C_new) return fail(HKM_EINVAL, "C and C_new must not alias");
    if (!labels && N > 0 && !step_labels_optional(D, K))
        return fail(HKM_EINVAL, "labels is NULL (hkm_lloyd_step_labels_optional() says which steps can run without "
                                "storing labels)");
    if (!shift) return fail(HKM_EINVAL, "shift is NULL");
    const int32_t flags = HKM_WS_LLOYD | (sse ? HKM_WS_SSE : 0);
    const size_t need = carve(nullptr, N, D, K, flags).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const Workspace w = carve(ws, N, D, K, flags);
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    if (small_eligible(D, K) && N > 0) {
        // one sweep over X: labels + private per-lane sums, then a single-workgroup finish
        if ((rc = launch_small(X, N, D, ldx, C, K, D, labels, nullptr, w.small_part, sse ? 3 : 1, w.small_flags, st,
                               labels64)))
            return rc;
        return launch_small_finalize(w.small_part, small_grid(N, D, K), K, D, C, C_new, D, nullptr, shift, sse, st);
    }
    if (fused_eligible(D, K) && N > 0) {
        // one sweep over X on the matrix cores: labels + fp64 per-cluster sums in LDS
        const bool few = few_eligible(D, K);
        const bool split = !few && use_split_products() && split_eligible(D, K, true);
        if (split)
            rc = launch_split_resident(X, N, D, ldx, C, K, D, labels, sse ? w.min_d2 : nullptr, w.fsum, w.fcnt,
                                       w.fflags, st);
        else if (few)
            rc = launch_few(X, N, D, ldx, C, K, D, labels, sse ? w.min_d2 : nullptr, w.fsum, w.fcnt, w.fflags, st);
        else
            rc = launch_lloyd_mfma_resident(X, N, D, ldx, C, K, D, labels, sse ? w.min_d2 : nullptr, w.fsum,
                                            w.fcnt, w.fflags, st);
        if (rc) return rc;
        if (few && !labels) {
            // the step stored no labels; the two-pass update that redoes the sums of a flagged step needs them:
            // one more launch, which returns at once unless a flag is up
            if ((rc = launch_few(X, N, D, ldx, C, K, D, w.lazy_lab, nullptr, nullptr, nullptr, nullptr, st, w.fflags,
                                 few_grid(N, D, K))))
                return rc;
            labels = w.lazy_lab;
        }
        if ((rc = launch_update_fused(X, N, D, ldx, labels, K, C_new, D, nullptr, w,
                                      split ? split_fused_grid(N) : few ? few_grid(N, D, K) : fused_grid(N, D), C,
                                      shift, st)))
            return rc;
    } else {
        if ((rc = do_assign(X, N, D, ldx, C, K, D, labels, sse ? w.min_d2 : nullptr, w, st))) return rc;
        if ((rc = do_update(X, N, D, ldx, labels, K, C_new, D, nullptr, w, C, shift, st))) return rc;
    }
    if (sse) rc = launch_sum_min_d2(w.min_d2, N, sse, w.red, 1, st);
    return rc;
}

int hkm_lloyd_step_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                       float* C_new, int32_t K, int32_t* labels, float* shift, float* sse, void* ws,
                       size_t ws_bytes, void* hip_stream) {
    return lloyd_step_f32(X, N, D, ldx, C, C_new, K, labels, false, shift, sse, ws, ws_bytes, hip_stream);
}

int hkm_lloyd_step_labels64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, float* C_new,
                                int32_t K, int64_t* labels, float* shift, float* sse, void* ws, size_t ws_bytes,
                                void* hip_stream) {
    g_err[0] = 0;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    if (reinterpret_cast<uintptr_t>(labels) & 7u) return fail(HKM_EINVAL, "labels is not 8-byte aligned");
    if (D >= 1 && K >= 1 && !small_eligible(D, K))
        return fail(HKM_EUNSUPPORTED,
                    "D = %d, K = %d: only the narrow one-sweep step (hkm_lloyd_kernel_name() == \"lloyd_small\") stores "
                    "64-bit labels itself; use hkm_lloyd_step_f32 and hkm_widen_labels_i64", D, K);
    return lloyd_step_f32(X, N, D, ldx, C, C_new, K, reinterpret_cast<int32_t*>(labels), true, shift, sse, ws, ws_bytes,
                          hip_stream);
}

int hkm_lloyd_step_labels_optional(int64_t N, int32_t D, int32_t K) {
    if (N < 0 || D < 1 || K < 1) return 0;
    return step_labels_optional(D, K) ? 1 : 0;
}

int hkm_lloyd_fit_supported(int64_t N, int32_t D, int32_t K) {
    if (N < 1 || D < 1 || K < 1) return 0;
    return fit_eligible(N, D, K) ? 1 : 0;
}

int hkm_lloyd_fit_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C0, int32_t K, int32_t max_iter,
                      int32_t use_tol, double tol, float* C_out, int64_t* labels, float* shift, int32_t* info,
                      uint64_t wait_limit_us, void* ws, size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C0", C0, K, D, D))) return rc;
    if ((rc = check_matrix("C_out", C_out, K, D, D))) return rc;
    if (max_iter < 1) return fail(HKM_EINVAL, "max_iter = %d must be >= 1", max_iter);
    if (!labels || !shift || !info) return fail(HKM_EINVAL, "NULL pointer argument");
    if (reinterpret_cast<uintptr_t>(labels) & 7u) return fail(HKM_EINVAL, "labels is not 8-byte aligned");
    if (!fit_eligible(N, D, K))
        return fail(HKM_EUNSUPPORTED,
                    "N = %lld, D = %d, K = %d is outside what one launch holds (hkm_lloyd_fit_supported): run "
                    "hkm_lloyd_step_f32 per iteration", (long long)N, D, K);
    if ((rc = check_ws(ws, ws_bytes, fit_workspace_bytes(D, K)))) return rc;
    // the device clock of the waits ticks at 100 MHz
    const uint64_t ticks = wait_limit_us > (uint64_t(1) << 40) ? (uint64_t(1) << 47) : wait_limit_us * 100u;
    return launch_lloyd_fit(X, N, D, ldx, C0, K, max_iter, use_tol, tol, C_out, labels, shift, info, ws, ticks,
                            static_cast<hipStream_t>(hip_stream));
}

int hkm_point_blocks(int32_t D, int32_t* tuned) {
    if (tuned) *tuned = (env_point_blocks() == 0 && tuned_point_blocks() != 0) ? 1 : 0;
    if (D < 1 || D > RESIDENT_MAX_D) return 0;
    return resident_point_blocks(resident_dp(D));
}

int hkm_point_blocks_trial(float* ms_two, float* ms_one) { return trial_report(ms_two, ms_one); }

int hkm_shift_f32(const float* C_old, const float* C_new, int32_t K, int32_t D, float* shift,
                  void* hip_stream) {
    g_err[0] = 0;
    if (K < 1 || D < 1) return fail(HKM_EINVAL, "K = %d and D = %d must be >= 1", K, D);
    if (!C_old || !C_new || !shift) return fail(HKM_EINVAL, "NULL pointer argument");
    return launch_shift(C_old, C_new, K, D, shift, static_cast<hipStream_t>(hip_stream));
}

int hkm_functional_value_f32(const float* min_d2, int64_t N, float* out, void* ws, size_t ws_bytes,
                             void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if ((!min_d2 && N > 0) || !out) return fail(HKM_EINVAL, "NULL pointer argument");
    const size_t need = carve(nullptr, N, 1, 1, HKM_WS_ASSIGN).total;
    int rc = check_ws(ws, ws_bytes, need);
    if (rc) return rc;
    const Workspace w = carve(ws, N, 1, 1, HKM_WS_ASSIGN);
    return launch_sum_min_d2(min_d2, N, out, w.red, 2, static_cast<hipStream_t>(hip_stream));
}

int hkm_min_dist_sum_f32(const float* min_d2, int64_t N, float* out, void* ws, size_t ws_bytes,
                         void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if ((!min_d2 && N > 0) || !out) return fail(HKM_EINVAL, "NULL pointer argument");
    const size_t need = carve(nullptr, N, 1, 1, HKM_WS_ASSIGN).total;
    int rc = check_ws(ws, ws_bytes, need);
    if (rc) return rc;
    const Workspace w = carve(ws, N, 1, 1, HKM_WS_ASSIGN);
    return launch_sum_min_d2(min_d2, N, out, w.red, 3, static_cast<hipStream_t>(hip_stream));
}

int hkm_min_merge_sum_f32(float* min_d2, const float* new_d2, int64_t N, float* out, void* ws, size_t ws_bytes,
                          void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if (((!min_d2 || !new_d2) && N > 0) || !out) return fail(HKM_EINVAL, "NULL pointer argument");
    const size_t need = carve(nullptr, N, 1, 1, HKM_WS_ASSIGN).total;
    int rc = check_ws(ws, ws_bytes, need);
    if (rc) return rc;
    const Workspace w = carve(ws, N, 1, 1, HKM_WS_ASSIGN);
    return launch_min_merge_sum(min_d2, new_d2, N, out, w.red, static_cast<hipStream_t>(hip_stream));
}

int hkm_sample_select_f32(const float* min_d2, const float* u, int64_t N, const float* cost,
                          float oversampling, int64_t* idx, int64_t cap, int64_t* count, void* ws,
                          size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if (cap < 0) return fail(HKM_EINVAL, "cap = %lld is negative", (long long)cap);
    if (!(oversampling > 0.f)) return fail(HKM_EINVAL, "oversampling = %g must be > 0", double(oversampling));
    if (N > 0 && (!min_d2 || !u)) return fail(HKM_EINVAL, "NULL pointer argument");
    if (!cost || !count || (cap > 0 && !idx)) return fail(HKM_EINVAL, "NULL pointer argument");
    const size_t need = carve(nullptr, N, 1, 1, HKM_WS_ASSIGN).total;
    int rc = check_ws(ws, ws_bytes, need);
    if (rc) return rc;
    const Workspace w = carve(ws, N, 1, 1, HKM_WS_ASSIGN);
    return launch_select(min_d2, u, N, cost, oversampling, idx, cap, count, w.red,
                         static_cast<hipStream_t>(hip_stream));
}

int hkm_label_counts_i64(const int32_t* labels, int64_t N, int32_t K, int64_t* counts,
                         void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if (K < 1) return fail(HKM_EINVAL, "K = %d must be >= 1", K);
    if ((N > 0 && !labels) || !counts) return fail(HKM_EINVAL, "NULL pointer argument");
    return launch_label_counts(labels, N, K, counts, static_cast<hipStream_t>(hip_stream));
}

int hkm_seed_plus_plus_f32(const float* X, int32_t M, int32_t D, int64_t ldx, const float* w, int32_t first,
                           const float* u, int32_t K, int32_t p, int64_t* idx, void* hip_stream) {
    g_err[0] = 0;
    if (M < 1 || M > HKM_SEED_MAX_ROWS)
        return fail(HKM_EINVAL, "M = %d outside 1..%d", M, HKM_SEED_MAX_ROWS);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    if (K < 1) return fail(HKM_EINVAL, "K = %d must be >= 1", K);
    if (ldx < D) return fail(HKM_EINVAL, "leading dimension of X (%lld) < columns (%d)", (long long)ldx, D);
    if (first < 0 || first >= M) return fail(HKM_EINVAL, "first = %d outside 0..%d", first, M - 1);
    if (p != 1 && p != 2) return fail(HKM_EINVAL, "p = %d must be 1 or 2", p);
    if (!X || !idx || (K > 1 && !u)) return fail(HKM_EINVAL, "NULL pointer argument");
    return launch_seed_plus_plus(X, M, D, ldx, w, first, u, K, p, idx, static_cast<hipStream_t>(hip_stream));
}

int hkm_seed_plus_plus_rows_f32(const float* X, int64_t M, int32_t D, int64_t ldx, const float* w, int64_t first,
                                const float* u, int32_t K, int32_t p, int64_t* idx, void* ws, size_t ws_bytes,
                                void* hip_stream) {
    g_err[0] = 0;
    if (M < 1 || M > HKM_SEED_ROWS_MAX)
        return fail(HKM_EINVAL, "M = %lld outside 1..%lld", (long long)M, (long long)HKM_SEED_ROWS_MAX);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    if (K < 1) return fail(HKM_EINVAL, "K = %d must be >= 1", K);
    if (ldx < D) return fail(HKM_EINVAL, "leading dimension of X (%lld) < columns (%d)", (long long)ldx, D);
    if (first < 0 || first >= M) return fail(HKM_EINVAL, "first = %lld outside 0..%lld", (long long)first, (long long)(M - 1));
    if (p != 1 && p != 2) return fail(HKM_EINVAL, "p = %d must be 1 or 2", p);
    if (!X || !idx || (K > 1 && !u)) return fail(HKM_EINVAL, "NULL pointer argument");
    const int32_t flags = HKM_WS_ASSIGN | HKM_WS_SSE;
    const size_t need = carve(nullptr, M, 1, 1, flags).total;
    int rc = check_ws(ws, ws_bytes, need);
    if (rc) return rc;
    const Workspace wk = carve(ws, M, 1, 1, flags);
    return launch_seed_plus_plus_rows(X, M, D, ldx, w, first, u, K, p, idx, wk.min_d2, wk.red,
                                      static_cast<hipStream_t>(hip_stream));
}

// ---- float64 data -----------------------------------------------------------------------------
int hkm_assign_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const double* C, int32_t K,
                   int64_t ldc, int32_t* labels, double* min_d2, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix64("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix64("C", C, K, D, ldc))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    if (N == 0) return HKM_OK;
    return launch_assign_f64(X, N, D, ldx, C, K, ldc, labels, min_d2, static_cast<hipStream_t>(hip_stream));
}

int hkm_update_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                   double* C_new, int64_t ldcn, int64_t* counts, void* ws, size_t ws_bytes,
                   void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix64("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix64("C_new", C_new, K, D, ldcn))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    const int32_t flags = HKM_WS_UPDATE | HKM_WS_F64;
    const size_t need = carve(nullptr, N, D, K, flags).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const Workspace w = carve(ws, N, D, K, flags);
    return do_update_f64(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, nullptr, nullptr,
                         static_cast<hipStream_t>(hip_stream));
}

int hkm_lloyd_step_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const double* C, double* C_new,
                       int32_t K, int32_t* labels, double* shift, double* sse, void* ws, size_t ws_bytes,
                       void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix64("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix64("C", C, K, D, D))) return rc;
    if ((rc = check_matrix64("C_new", C_new, K, D, D))) return rc;
    if (C == C_new) return fail(HKM_EINVAL, "C and C_new must not alias");
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    if (!shift) return fail(HKM_EINVAL, "shift is NULL");
    const int32_t flags = HKM_WS_LLOYD | HKM_WS_F64 | (sse ? HKM_WS_SSE : 0);
    const size_t need = carve(nullptr, N, D, K, flags).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const Workspace w = carve(ws, N, D, K, flags);
    hipStream_t st = static_cast<hipStream_t>(hip_stream);
    double* md = sse ? reinterpret_cast<double*>(w.min_d2) : nullptr;
    if (N > 0 && (rc = launch_assign_f64(X, N, D, ldx, C, K, D, labels, md, st))) return rc;
    if ((rc = do_update_f64(X, N, D, ldx, labels, K, C_new, D, nullptr, w, C, shift, st))) return rc;
    if (sse) rc = launch_sum_min_d2_f64(md, N, sse, w.red, 1, st);
    return rc;
}

int hkm_shift_f64(const double* C_old, const double* C_new, int32_t K, int32_t D, double* shift,
                  void* hip_stream) {
    g_err[0] = 0;
    if (K < 1 || D < 1) return fail(HKM_EINVAL, "K = %d and D = %d must be >= 1", K, D);
    if (!C_old || !C_new || !shift) return fail(HKM_EINVAL, "NULL pointer argument");
    return launch_shift_f64(C_old, C_new, K, D, shift, static_cast<hipStream_t>(hip_stream));
}

int hkm_functional_value_f64(const double* min_d2, int64_t N, double* out, void* ws, size_t ws_bytes,
                             void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if (!min_d2 || !out) return fail(HKM_EINVAL, "NULL pointer argument");
    const size_t need = carve(nullptr, N, 1, 1, HKM_WS_ASSIGN).total;
    int rc = check_ws(ws, ws_bytes, need);
    if (rc) return rc;
    const Workspace w = carve(ws, N, 1, 1, HKM_WS_ASSIGN);
    return launch_sum_min_d2_f64(min_d2, N, out, w.red, 2, static_cast<hipStream_t>(hip_stream));
}

int hkm_pairwise_f64(const double* X, int64_t M, int64_t ldx, const double* Y, int64_t Nn, int64_t ldy,
                     int32_t D, double* out, int64_t ldo, int32_t metric, double sigma, void* hip_stream) {
    g_err[0] = 0;
    if (M < 0 || Nn < 0) return fail(HKM_EINVAL, "negative row count (M = %lld, Nn = %lld)", (long long)M, (long long)Nn);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    if (metric < HKM_METRIC_EUCLID_QE || metric > HKM_METRIC_MANHATTAN) return fail(HKM_EINVAL, "unknown metric %d", metric);
    const bool gaussian = metric == HKM_METRIC_GAUSS_QE || metric == HKM_METRIC_GAUSS;
    if (gaussian && !(sigma > 0.0)) return fail(HKM_EINVAL, "sigma = %g must be > 0", sigma);
    int rc;
    if ((rc = check_matrix64("X", X, M, D, ldx))) return rc;
    if ((rc = check_matrix64("Y", Y, Nn, D, ldy))) return rc;
    if (!out) return fail(HKM_EINVAL, "out is NULL");
    if (ldo < Nn) return fail(HKM_EINVAL, "leading dimension of out (%lld) < columns (%lld)", (long long)ldo, (long long)Nn);
    if (M == 0 || Nn == 0) return HKM_OK;
    const int form = (metric == HKM_METRIC_EUCLID_QE || metric == HKM_METRIC_GAUSS_QE) ? 0
                     : (metric == HKM_METRIC_MANHATTAN ? 2 : 1);
    return launch_cdist_f64(X, M, ldx, Y, Nn, ldy, D, out, ldo, form, gaussian ? 0 : 1,
                            gaussian ? 1.0 / (2.0 * sigma * sigma) : 0.0, static_cast<hipStream_t>(hip_stream));
}

int hkm_assign_l1_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                      int64_t ldc, int32_t* labels, float* min_dist, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C", C, K, D, ldc))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    if (N == 0) return HKM_OK;
    return launch_assign_l1(X, N, D, ldx, C, K, ldc, labels, min_dist, static_cast<hipStream_t>(hip_stream));
}

int hkm_closest_rows_l1_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const float* Q, int32_t M,
                            int64_t ldq, int64_t* idx, float* dist, void* ws, size_t ws_bytes,
                            void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, M);
    if (rc) return rc;
    if (N < 1) return fail(HKM_EINVAL, "N = %lld: there is no closest row in an empty matrix", (long long)N);
    if (N > 0xfffffffeLL) return fail(HKM_EUNSUPPORTED, "N = %lld exceeds 32-bit row indices", (long long)N);
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("Q", Q, M, D, ldq))) return rc;
    if (!idx) return fail(HKM_EINVAL, "idx is NULL");
    const size_t need = carve_median(nullptr, N, D, M).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const MedianWorkspace w = carve_median(ws, N, D, M);
    return launch_closest_rows_l1(X, N, D, ldx, Q, M, ldq, idx, dist, w.keys, static_cast<hipStream_t>(hip_stream));
}

int hkm_closest_rows_l1_q64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const double* Q, int32_t M,
                                int64_t* idx, double* dist, void* ws, size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, M);
    if (rc) return rc;
    if (N < 1) return fail(HKM_EINVAL, "N = %lld: there is no closest row in an empty matrix", (long long)N);
    if (N > 0xfffffffeLL) return fail(HKM_EUNSUPPORTED, "N = %lld exceeds 32-bit row indices", (long long)N);
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix64("Q", Q, M, D, D))) return rc;
    if (!idx) return fail(HKM_EINVAL, "idx is NULL");
    const size_t need = carve_median(nullptr, N, D, M).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const MedianWorkspace w = carve_median(ws, N, D, M);
    return launch_closest_rows_l1_q64(X, N, D, ldx, Q, M, idx, dist, w.snap_d, w.snap_i,
                                      static_cast<hipStream_t>(hip_stream));
}

struct KnnWorkspace {
    float* xn;  // squared norms of the reference rows, padded to a whole tile
    float* last_d2;
    unsigned* last_i;
    float* part_d;
    unsigned* part_i;
    size_t total;
};

static KnnWorkspace carve_knn(void* base, int64_t M, int64_t N) {
    KnnWorkspace w;
    char* p = static_cast<char*>(base);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* r = p ? p + off : nullptr;
        off += align_up(bytes, 256);
        return r;
    };
    const size_t m = size_t(M < 1 ? 1 : M);
    // sized for the largest number of splits any feature count asks for
    const size_t slots = knn_plan(M, N, knn_max_target_workgroups()).part_slots;
    w.xn = reinterpret_cast<float*>(take((size_t(N < 1 ? 1 : N) + 64) * sizeof(float)));
    w.last_d2 = reinterpret_cast<float*>(take(m * sizeof(float)));
    w.last_i = reinterpret_cast<unsigned*>(take(m * sizeof(unsigned)));
    w.part_d = reinterpret_cast<float*>(take((slots ? slots : 1) * sizeof(float)));
    w.part_i = reinterpret_cast<unsigned*>(take((slots ? slots : 1) * sizeof(unsigned)));
    w.total = off;
    return w;
}

size_t hkm_knn_workspace_bytes(int64_t M, int64_t N) {
    if (M < 0 || N < 1) return 0;
    return carve_knn(nullptr, M, N).total;
}

int hkm_knn_f32(const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx, int32_t D, int32_t k,
                int64_t* idx, int64_t ldi, float* dist, int64_t ldd, void* ws, size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    if (M < 0) return fail(HKM_EINVAL, "M = %lld is negative", (long long)M);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    if (N < 1) return fail(HKM_EINVAL, "N = %lld: there are no neighbours in an empty matrix", (long long)N);
    if (N > 0xfffffffeLL) return fail(HKM_EUNSUPPORTED, "N = %lld exceeds 32-bit row indices", (long long)N);
    if (k < 1 || k > N) return fail(HKM_EINVAL, "k = %d must be in [1, N = %lld]", k, (long long)N);
    if (k > HKM_KNN_MAX_K) return fail(HKM_EUNSUPPORTED, "k = %d exceeds HKM_KNN_MAX_K = %d", k, HKM_KNN_MAX_K);
    int rc;
    if ((rc = check_matrix("Q", Q, M, D, ldq))) return rc;
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if (!idx && M > 0) return fail(HKM_EINVAL, "idx is NULL");
    if (ldi < k) return fail(HKM_EINVAL, "leading dimension of idx (%lld) < k (%d)", (long long)ldi, k);
    if (dist && ldd < k) return fail(HKM_EINVAL, "leading dimension of dist (%lld) < k (%d)", (long long)ldd, k);
    if (reinterpret_cast<uintptr_t>(idx) & 7u) return fail(HKM_EINVAL, "idx is not 8-byte aligned");
    if (reinterpret_cast<uintptr_t>(dist) & 3u) return fail(HKM_EINVAL, "dist is not 4-byte aligned");
    const size_t need = carve_knn(nullptr, M, N).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const KnnWorkspace w = carve_knn(ws, M, N);
    return launch_knn(Q, M, ldq, X, N, ldx, D, k, idx, ldi, dist, ldd, w.xn, w.last_d2, w.last_i, w.part_d, w.part_i,
                      static_cast<hipStream_t>(hip_stream));
}

int hkm_cluster_distance_sums_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int64_t* perm,
                                  const int64_t* offsets, int32_t K, float* S, int64_t lds, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if (K > 65535) return fail(HKM_EUNSUPPORTED, "K = %d exceeds 65535 clusters", K);
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("S", S, N, K, lds))) return rc;
    if (!offsets || (N > 0 && !perm)) return fail(HKM_EINVAL, "perm or offsets is NULL");
    if ((reinterpret_cast<uintptr_t>(perm) | reinterpret_cast<uintptr_t>(offsets)) & 7u)
        return fail(HKM_EINVAL, "perm or offsets is not 8-byte aligned");
    return launch_silhouette_sums(X, N, D, ldx, perm, offsets, K, S, lds, static_cast<hipStream_t>(hip_stream));
}

int hkm_silhouette_finish_f32(const float* S, int64_t N, int32_t K, int64_t lds, const int64_t* labels,
                              const int64_t* counts, float* out, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, 1, K);
    if (rc) return rc;
    if ((rc = check_matrix("S", S, N, K, lds))) return rc;
    if (!counts || (N > 0 && (!labels || !out))) return fail(HKM_EINVAL, "labels, counts or out is NULL");
    if ((reinterpret_cast<uintptr_t>(labels) | reinterpret_cast<uintptr_t>(counts)) & 7u)
        return fail(HKM_EINVAL, "labels or counts is not 8-byte aligned");
    if (reinterpret_cast<uintptr_t>(out) & 3u) return fail(HKM_EINVAL, "out is not 4-byte aligned");
    return launch_silhouette_finish(S, N, K, lds, labels, counts, out, static_cast<hipStream_t>(hip_stream));
}

// rows run along grid.x, 256-column slices along grid.y (at most 65535 of them); a matrix of that many rows
// would be a petabyte
static const int64_t LAPLACIAN_MAX_N = int64_t(65535) * 256;

// 0: nothing to do, 1: arguments fine, launch; negative: error
static int laplacian_check(size_t elem, const void* S, int64_t N, int64_t lds, int32_t definition, int32_t mode,
                           const void* L, int64_t ldl, const void* degree) {
    g_err[0] = 0;
    if (N < 0 || N > LAPLACIAN_MAX_N)
        return fail(HKM_EUNSUPPORTED, "N = %lld must be in [0, %lld]", (long long)N, (long long)LAPLACIAN_MAX_N);
    if (definition != HKM_LAPLACIAN_SIMPLE && definition != HKM_LAPLACIAN_NORM_SYM)
        return fail(HKM_EINVAL, "definition = %d is neither simple (0) nor norm_sym (1)", definition);
    if (mode < 0 || mode > 2) return fail(HKM_EINVAL, "mode = %d must be 0 (fully connected), 1 (upper) or 2 (lower)", mode);
    if (N == 0) return 0;
    int rc;
    if (elem == 8) {
        if ((rc = check_matrix64("S", S, N, (int32_t)N, lds))) return rc;
        if ((rc = check_matrix64("L", L, N, (int32_t)N, ldl))) return rc;
    } else {
        if ((rc = check_matrix("S", S, N, (int32_t)N, lds))) return rc;
        if ((rc = check_matrix("L", L, N, (int32_t)N, ldl))) return rc;
    }
    if (!degree) return fail(HKM_EINVAL, "degree is NULL");
    if (reinterpret_cast<uintptr_t>(degree) & (elem - 1)) return fail(HKM_EINVAL, "degree is misaligned");
    return 1;
}

int hkm_laplacian_f32(const float* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                      float eps, float* L, int64_t ldl, float* degree, void* hip_stream) {
    const int rc = laplacian_check(4, S, N, lds, definition, mode, L, ldl, degree);
    if (rc != 1) return rc;
    return launch_laplacian(S, N, lds, definition, mode, weighted ? 1 : 0, eps, L, ldl, degree,
                            static_cast<hipStream_t>(hip_stream));
}

int hkm_laplacian_f64(const double* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                      double eps, double* L, int64_t ldl, double* degree, void* hip_stream) {
    const int rc = laplacian_check(8, S, N, lds, definition, mode, L, ldl, degree);
    if (rc != 1) return rc;
    return launch_laplacian_f64(S, N, lds, definition, mode, weighted ? 1 : 0, eps, L, ldl, degree,
                                static_cast<hipStream_t>(hip_stream));
}

int hkm_knn_vote_f32(const int64_t* idx, int64_t M, int32_t k, int64_t ldi, const float* Y, int64_t N, int32_t C,
                     int64_t ldy, int64_t* classes, void* hip_stream) {
    g_err[0] = 0;
    if (M < 0) return fail(HKM_EINVAL, "M = %lld is negative", (long long)M);
    if (k < 1) return fail(HKM_EINVAL, "k = %d must be >= 1", k);
    if (C < 1) return fail(HKM_EINVAL, "C = %d must be >= 1", C);
    if (N < 1) return fail(HKM_EINVAL, "N = %lld must be >= 1", (long long)N);
    if (ldi < k) return fail(HKM_EINVAL, "leading dimension of idx (%lld) < k (%d)", (long long)ldi, k);
    int rc;
    if ((rc = check_matrix("Y", Y, N, C, ldy))) return rc;
    if (M > 0 && (!idx || !classes)) return fail(HKM_EINVAL, "idx or classes is NULL");
    if ((reinterpret_cast<uintptr_t>(idx) | reinterpret_cast<uintptr_t>(classes)) & 7u)
        return fail(HKM_EINVAL, "idx or classes is not 8-byte aligned");
    return launch_knn_vote(idx, M, k, ldi, Y, N, C, ldy, classes, static_cast<hipStream_t>(hip_stream));
}

static int update_median_common(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                                const int64_t* fallback_rows, const float* C_old, float* C_new, int64_t ldcn,
                                int64_t* counts, int32_t mode, int32_t skip_zero_rows, double* medians_f64, void* ws,
                                size_t ws_bytes, void* hip_stream);

int hkm_update_median_q64_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                              const int64_t* fallback_rows, const float* C_old, float* C_new, int64_t ldcn,
                              int64_t* counts, int32_t mode, int32_t skip_zero_rows, double* medians_f64, void* ws,
                              size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    if (!medians_f64) return fail(HKM_EINVAL, "medians_f64 is NULL");
    if (reinterpret_cast<uintptr_t>(medians_f64) & 7u) return fail(HKM_EINVAL, "medians_f64 is not 8-byte aligned");
    return update_median_common(X, N, D, ldx, labels, K, fallback_rows, C_old, C_new, ldcn, counts, mode,
                                skip_zero_rows, medians_f64, ws, ws_bytes, hip_stream);
}

int hkm_update_median_f32(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                          const int64_t* fallback_rows, const float* C_old, float* C_new, int64_t ldcn,
                          int64_t* counts, int32_t mode, int32_t skip_zero_rows, void* ws, size_t ws_bytes,
                          void* hip_stream) {
    g_err[0] = 0;
    return update_median_common(X, N, D, ldx, labels, K, fallback_rows, C_old, C_new, ldcn, counts, mode,
                                skip_zero_rows, nullptr, ws, ws_bytes, hip_stream);
}

static int update_median_common(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                                const int64_t* fallback_rows, const float* C_old, float* C_new, int64_t ldcn,
                                int64_t* counts, int32_t mode, int32_t skip_zero_rows, double* medians_f64, void* ws,
                                size_t ws_bytes, void* hip_stream) {
    g_err[0] = 0;
    int rc = check_shape(N, D, K);
    if (rc) return rc;
    if (N > 0x7ffffffeLL) return fail(HKM_EUNSUPPORTED, "N = %lld exceeds 31-bit row indices", (long long)N);
    if (mode != 0 && mode != 1) return fail(HKM_EINVAL, "mode = %d must be 0 (mean of the middles) or 1 (lower middle)", mode);
    if ((rc = check_matrix("X", X, N, D, ldx))) return rc;
    if ((rc = check_matrix("C_new", C_new, K, D, ldcn))) return rc;
    if (C_old && (rc = check_matrix("C_old", C_old, K, D, D))) return rc;
    if (!labels && N > 0) return fail(HKM_EINVAL, "labels is NULL");
    const size_t need = carve_median(nullptr, N, D, K).total;
    if ((rc = check_ws(ws, ws_bytes, need))) return rc;
    const MedianWorkspace w = carve_median(ws, N, D, K);
    return launch_update_median(X, N, D, ldx, labels, K, fallback_rows, C_old, C_new, ldcn, counts, mode,
                                skip_zero_rows, w, static_cast<hipStream_t>(hip_stream), medians_f64);
}

int hkm_cdist_f32(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                  int32_t D, float* out, int64_t ldo, int32_t sqrt_flag, void* hip_stream) {
    g_err[0] = 0;
    if (M < 0 || Nn < 0) return fail(HKM_EINVAL, "negative row count (M = %lld, Nn = %lld)", (long long)M, (long long)Nn);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    int rc;
    if ((rc = check_matrix("X", X, M, D, ldx))) return rc;
    if ((rc = check_matrix("Y", Y, Nn, D, ldy))) return rc;
    if (!out) return fail(HKM_EINVAL, "out is NULL");
    if (ldo < Nn) return fail(HKM_EINVAL, "leading dimension of out (%lld) < columns (%lld)", (long long)ldo, (long long)Nn);
    if (M == 0 || Nn == 0) return HKM_OK;
    return launch_cdist(X, M, ldx, Y, Nn, ldy, D, out, ldo, 0, sqrt_flag, 0.f, static_cast<hipStream_t>(hip_stream));
}

int hkm_pairwise_f32(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                     int32_t D, float* out, int64_t ldo, int32_t metric, float sigma, void* hip_stream) {
    g_err[0] = 0;
    if (M < 0 || Nn < 0) return fail(HKM_EINVAL, "negative row count (M = %lld, Nn = %lld)", (long long)M, (long long)Nn);
    if (D < 1) return fail(HKM_EINVAL, "D = %d must be >= 1", D);
    if (metric < HKM_METRIC_EUCLID_QE || metric > HKM_METRIC_MANHATTAN) return fail(HKM_EINVAL, "unknown metric %d", metric);
    const bool gaussian = metric == HKM_METRIC_GAUSS_QE || metric == HKM_METRIC_GAUSS;
    if (gaussian && !(sigma > 0.f)) return fail(HKM_EINVAL, "sigma = %g must be > 0", double(sigma));
    int rc;
    if ((rc = check_matrix("X", X, M, D, ldx))) return rc;
    if ((rc = check_matrix("Y", Y, Nn, D, ldy))) return rc;
    if (!out) return fail(HKM_EINVAL, "out is NULL");
    if (ldo < Nn) return fail(HKM_EINVAL, "leading dimension of out (%lld) < columns (%lld)", (long long)ldo, (long long)Nn);
    if (M == 0 || Nn == 0) return HKM_OK;
    const int form = (metric == HKM_METRIC_EUCLID_QE || metric == HKM_METRIC_GAUSS_QE) ? 0
                     : metric == HKM_METRIC_MANHATTAN                                   ? 2
                                                                                        : 1;
    const float gauss = gaussian ? 1.0f / (2.0f * sigma * sigma) : 0.f;
    return launch_cdist(X, M, ldx, Y, Nn, ldy, D, out, ldo, form, 1, gauss, static_cast<hipStream_t>(hip_stream));
}

int hkm_widen_labels_i64(const int32_t* in, int64_t N, int64_t* out, void* hip_stream) {
    g_err[0] = 0;
    if (N < 0) return fail(HKM_EINVAL, "N = %lld is negative", (long long)N);
    if (!in || !out) return fail(HKM_EINVAL, "NULL pointer argument");
    if (N == 0) return HKM_OK;
    return launch_widen(in, N, out, static_cast<hipStream_t>(hip_stream));
}

}  // extern "C"
