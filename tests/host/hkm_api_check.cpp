// Host-side driver for the argument-validation layer of libhkm (include/hkm.h), meant to run under the host
// compiler's AddressSanitizer (heat_amd/csrc/Makefile, target asan-host): every call below is refused -- or
// returns at once for an empty problem -- before anything reaches the device, so it runs without a GPU.  What
// the sanitizer watches is the host code on those paths: the checks themselves, the formatting of the
// thread-local message, the workspace carving arithmetic.  Pointers handed in are made-up non-null addresses
// that are never dereferenced.
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "hkm.h"
#include "hkm_bench.h"

static int failures = 0;

#define EXPECT(call, want)                                                                     \
    do {                                                                                       \
        const int rc_ = (call);                                                                \
        if (rc_ != (want)) {                                                                   \
            std::printf("FAIL %s:%d  %s  returned %d, expected %d (%s)\n", __FILE__, __LINE__, \
                        #call, rc_, (want), hkm_last_error());                                 \
            ++failures;                                                                        \
        }                                                                                      \
    } while (0)

#define EXPECT_MSG(sub)                                                                                   \
    do {                                                                                                  \
        if (!std::strstr(hkm_last_error(), (sub))) {                                                      \
            std::printf("FAIL %s:%d  message '%s' lacks '%s'\n", __FILE__, __LINE__, hkm_last_error(), (sub)); \
            ++failures;                                                                                   \
        }                                                                                                 \
    } while (0)

int main() {
    float* const f = reinterpret_cast<float*>(uintptr_t(4096));
    double* const d = reinterpret_cast<double*>(uintptr_t(4096));
    int32_t* const i32 = reinterpret_cast<int32_t*>(uintptr_t(4096));
    int64_t* const i64 = reinterpret_cast<int64_t*>(uintptr_t(4096));
    void* const ws = reinterpret_cast<void*>(uintptr_t(1) << 20);
    const size_t big = size_t(1) << 30;

    if (hkm_version() < 302) {
        std::printf("FAIL version %d\n", hkm_version());
        ++failures;
    }

    // ---- hkm_assign_f32
    EXPECT(hkm_assign_f32(nullptr, 10, 3, 3, f, 8, 3, i32, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT_MSG("X is NULL");
    EXPECT(hkm_assign_f32(f, -1, 3, 3, f, 8, 3, i32, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_f32(f, 10, 0, 3, f, 8, 3, i32, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_f32(f, 10, 3, 3, f, 0, 3, i32, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_f32(f, 10, 3, 2, f, 8, 3, i32, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_f32(reinterpret_cast<float*>(uintptr_t(4098)), 10, 3, 3, f, 8, 3, i32, nullptr, ws, big, nullptr),
           HKM_EINVAL);
    EXPECT(hkm_assign_f32(f, 10, 3, 3, f, 8, 3, nullptr, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_f32(f, 10, 3, 3, f, 8, 3, i32, nullptr, nullptr, 0, nullptr), HKM_EWORKSPACE);
    EXPECT(hkm_assign_f32(f, 10, 3, 3, f, 8, 3, i32, nullptr, ws, 16, nullptr), HKM_EWORKSPACE);
    EXPECT(hkm_assign_f32(f, 10, 3, 3, f, 8, 3, i32, nullptr, reinterpret_cast<void*>((uintptr_t(1) << 20) + 8), big, nullptr),
           HKM_EWORKSPACE);
    // every kernel family's shape goes through the same checks and its own workspace arithmetic
    const int32_t shapes[][2] = {{3, 8}, {8, 16}, {32, 256}, {64, 1024}, {512, 1024}, {100, 5000}, {17, 3}};
    for (const auto& s : shapes) {
        EXPECT(hkm_assign_f32(f, 1000, s[0], s[0], f, s[1], s[0], i32, nullptr, ws, 16, nullptr), HKM_EWORKSPACE);
        EXPECT(hkm_lloyd_step_f32(f, 1000, s[0], s[0], f, f + 1024, s[1], i32, f, nullptr, ws, 16, nullptr), HKM_EWORKSPACE);
        if (hkm_workspace_bytes(1000, s[0], s[1], HKM_WS_ASSIGN) > hkm_workspace_bytes(1000, s[0], s[1], HKM_WS_LLOYD)) {
            std::printf("FAIL workspace sizes D=%d K=%d\n", s[0], s[1]);
            ++failures;
        }
    }
    // a message longer than most: formatted into the thread-local buffer
    EXPECT(hkm_assign_f32(f, INT64_MAX / 2, INT32_MAX, INT64_MAX / 4, f, INT32_MAX, INT64_MAX / 8, i32, nullptr, ws, big, nullptr),
           HKM_EUNSUPPORTED);

    // ---- update / step / shift
    EXPECT(hkm_update_f32(f, 10, 3, 3, nullptr, 8, f, 3, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_update_f32(f, 10, 3, 3, i32, 8, f, 2, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_update_f32(f, 10, 3, 3, i32, 8, f, 3, nullptr, ws, 8, nullptr), HKM_EWORKSPACE);
    EXPECT(hkm_lloyd_step_f32(f, 10, 3, 3, f, f, 8, i32, f, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_shift_f32(nullptr, f, 8, 3, f, nullptr), HKM_EINVAL);
    EXPECT(hkm_shift_f32(f, f, 0, 3, f, nullptr), HKM_EINVAL);
    EXPECT(hkm_functional_value_f32(f, -1, f, ws, big, nullptr), HKM_EINVAL);

    // ---- the whole loop in one launch, and the assignment that stores 64-bit labels: shapes and arguments
    int32_t info[2] = {0, 0};
    if (hkm_lloyd_fit_supported(100000, 8, 16) != 1 || hkm_lloyd_fit_supported(131073, 8, 16) != 0 ||
        hkm_lloyd_fit_supported(262144, 4, 5) != 1 || hkm_lloyd_fit_supported(1000, 17, 5) != 0 ||
        hkm_lloyd_fit_supported(1000, 8, 27) != 0 || hkm_lloyd_fit_supported(0, 8, 4) != 0 ||
        hkm_workspace_bytes(1000, 17, 5, HKM_WS_FIT) != 0 || hkm_workspace_bytes(1000, 8, 16, HKM_WS_FIT) == 0) {
        std::printf("FAIL hkm_lloyd_fit_supported / HKM_WS_FIT\n");
        ++failures;
    }
    EXPECT(hkm_lloyd_fit_f32(nullptr, 1000, 8, 8, f, 16, 5, 1, 0.0, f + 4096, i64, f, info, 1000, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_lloyd_fit_f32(f, 1000, 8, 8, f, 16, 0, 1, 0.0, f + 4096, i64, f, info, 1000, ws, big, nullptr), HKM_EINVAL);
    EXPECT_MSG("max_iter");
    EXPECT(hkm_lloyd_fit_f32(f, 1000, 8, 8, f, 16, 5, 1, 0.0, f + 4096, nullptr, f, info, 1000, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_lloyd_fit_f32(f, 1000, 8, 8, f, 16, 5, 1, 0.0, f + 4096, i64, f, nullptr, 1000, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_lloyd_fit_f32(f, 1000, 8, 8, f, 16, 5, 1, 0.0, f + 4096, i64, f, info, 1000, ws, 16, nullptr), HKM_EWORKSPACE);
    EXPECT(hkm_lloyd_fit_f32(f, 1000, 32, 32, f, 16, 5, 1, 0.0, f + 4096, i64, f, info, 1000, ws, big, nullptr), HKM_EUNSUPPORTED);
    EXPECT(hkm_lloyd_fit_f32(f, 300000, 8, 8, f, 16, 5, 1, 0.0, f + 4096, i64, f, info, 1000, ws, big, nullptr), HKM_EUNSUPPORTED);
    EXPECT(hkm_assign_labels64_f32(f, 10, 3, 3, f, 8, 3, nullptr, nullptr, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_labels64_f32(f, 10, 3, 2, f, 8, 3, i64, nullptr, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_labels64_f32(f, 10, 32, 32, f, 8, 32, i64, nullptr, nullptr), HKM_EUNSUPPORTED);
    EXPECT(hkm_assign_labels64_f32(f, 0, 3, 3, f, 8, 3, i64, nullptr, nullptr), HKM_OK);
    if (hkm_lloyd_step_labels_optional(1000, 32, 8) != 1 || hkm_lloyd_step_labels_optional(1000, 32, 256) != 0 ||
        hkm_lloyd_step_labels_optional(1000, 0, 8) != 0 || hkm_lloyd_step_labels_optional(-1, 3, 8) != 0) {
        std::printf("FAIL hkm_lloyd_step_labels_optional\n");
        ++failures;
    }
    EXPECT(hkm_lloyd_step_f32(f, 10, 32, 32, f, f + 4096, 256, nullptr, f, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT_MSG("labels is NULL");
    // the step that stores 64-bit labels: labels required and aligned, narrow shapes only, the usual checks behind
    EXPECT(hkm_lloyd_step_labels64_f32(f, 10, 3, 3, f, f + 4096, 8, nullptr, f, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_lloyd_step_labels64_f32(f, 10, 3, 3, f, f + 4096, 8,
                                       reinterpret_cast<int64_t*>(reinterpret_cast<char*>(i64) + 4), f, nullptr, ws, big,
                                       nullptr), HKM_EINVAL);
    EXPECT(hkm_lloyd_step_labels64_f32(f, 10, 32, 32, f, f + 4096, 8, i64, f, nullptr, ws, big, nullptr), HKM_EUNSUPPORTED);
    EXPECT(hkm_lloyd_step_labels64_f32(f, 10, 3, 3, f, f, 8, i64, f, nullptr, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_lloyd_step_labels64_f32(f, 10, 3, 3, f, f + 4096, 8, i64, f, nullptr, ws, 16, nullptr), HKM_EWORKSPACE);

    // ---- the allocation-free assignment: its built-in scratch has a stated size
    EXPECT(hkm_assign_static_f32(nullptr, 10, 3, 3, f, 8, 3, i32, nullptr, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_static_f32(f, int64_t(1) << 26, 512, 512, f, 1024, 512, i32, nullptr, nullptr), HKM_EUNSUPPORTED);
    if (hkm_static_scratch_bytes() != size_t(HKM_STATIC_SCRATCH_BYTES)) {
        std::printf("FAIL static scratch size\n");
        ++failures;
    }

    // ---- distances
    EXPECT(hkm_cdist_f32(f, 4, 3, f, 4, 3, 3, f, 3, 1, nullptr), HKM_EINVAL);
    EXPECT(hkm_cdist_f32(f, -4, 3, f, 4, 3, 3, f, 4, 1, nullptr), HKM_EINVAL);
    EXPECT(hkm_pairwise_f32(f, 4, 3, f, 4, 3, 3, f, 4, 9, 1.0f, nullptr), HKM_EINVAL);
    EXPECT(hkm_pairwise_f32(f, 4, 3, f, 4, 3, 3, f, 4, HKM_METRIC_GAUSS, 0.0f, nullptr), HKM_EINVAL);
    EXPECT(hkm_pairwise_f64(d, 4, 3, d, 4, 3, 3, d, 4, 9, 1.0, nullptr), HKM_EINVAL);
    EXPECT(hkm_widen_labels_i64(nullptr, 4, i64, nullptr), HKM_EINVAL);

    // ---- float64 entry points
    EXPECT(hkm_assign_f64(reinterpret_cast<double*>(uintptr_t(4100)), 10, 3, 3, d, 8, 3, i32, nullptr, nullptr), HKM_EINVAL);
    EXPECT(hkm_assign_f64(d, 10, 3, 2, d, 8, 3, i32, nullptr, nullptr), HKM_EINVAL);
    EXPECT(hkm_update_f64(d, 10, 3, 3, i32, 8, d, 3, nullptr, ws, 8, nullptr), HKM_EWORKSPACE);
    EXPECT(hkm_shift_f64(nullptr, d, 8, 3, d, nullptr), HKM_EINVAL);

    // ---- k nearest neighbours
    EXPECT(hkm_knn_f32(f, 4, 3, f, 0, 3, 3, 1, i64, 1, nullptr, 0, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_knn_f32(f, 4, 3, f, 10, 3, 3, 11, i64, 11, nullptr, 0, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_knn_f32(f, 4, 3, f, 10, 3, 3, 2, i64, 1, nullptr, 0, ws, big, nullptr), HKM_EINVAL);
    EXPECT(hkm_knn_f32(f, 4, 3, f, 10, 3, 3, 2, i64, 2, nullptr, 0, ws, 8, nullptr), HKM_EWORKSPACE);
    if (hkm_knn_workspace_bytes(1000, 100000) == 0 || hkm_knn_workspace_bytes(-1, 10) != 0) {
        std::printf("FAIL knn workspace size\n");
        ++failures;
    }

    // ---- Laplacian (S, N, lds, definition, mode, weighted, eps, L, ldl, degree)
    EXPECT(hkm_laplacian_f32(nullptr, 4, 4, 0, 0, 0, 0.0f, f, 4, f, nullptr), HKM_EINVAL);
    EXPECT(hkm_laplacian_f32(f, 4, 3, 0, 0, 0, 0.0f, f, 4, f, nullptr), HKM_EINVAL);
    EXPECT(hkm_laplacian_f32(f, (int64_t(1) << 24) + 1, int64_t(1) << 25, 0, 0, 0, 0.0f, f, int64_t(1) << 25, f, nullptr),
           HKM_EUNSUPPORTED);
    EXPECT(hkm_laplacian_f64(d, 4, 3, 0, 0, 0, 0.0, d, 4, d, nullptr), HKM_EINVAL);

    // ---- empty problems succeed without touching the device, and clear the message
    EXPECT(hkm_widen_labels_i64(i32, 0, i64, nullptr), HKM_OK);
    EXPECT(hkm_cdist_f32(nullptr, 0, 3, f, 4, 3, 3, f, 4, 1, nullptr), HKM_OK);
    if (hkm_last_error()[0] != 0) {
        std::printf("FAIL message not cleared: %s\n", hkm_last_error());
        ++failures;
    }

    // ---- the launch-geometry choice of the resident kernels: queries and refusals only
    int32_t tuned = -1;
    if (hkm_point_blocks(0, &tuned) != 0 || hkm_point_blocks(130, nullptr) != 0 || hkm_point_blocks(48, &tuned) != 1 ||
        tuned != 0) {
        std::printf("FAIL hkm_point_blocks\n");
        ++failures;
    }
    float ms_two = -1.f, ms_one = -1.f;
    if (hkm_point_blocks_trial(&ms_two, &ms_one) != 0 || hkm_point_blocks_trial(nullptr, nullptr) != 0) {
        std::printf("FAIL hkm_point_blocks_trial\n");
        ++failures;
    }

    // ---- the measurement hooks with nothing recorded
    float ms[4];
    int32_t count = -1;
    EXPECT(hkm_profile_enable(1), HKM_OK);
    EXPECT(hkm_profile_collect(ms, 4, &count), HKM_OK);
    EXPECT(hkm_profile_enable(0), HKM_OK);
    if (count != 0) {
        std::printf("FAIL profile count %d\n", count);
        ++failures;
    }

    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
