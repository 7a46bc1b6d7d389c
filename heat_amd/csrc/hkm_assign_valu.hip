// Fused distance + argmin for small feature counts (D <= 16): one point per lane in registers,
// centroids and their squared norms in LDS, read as wave-wide broadcasts.  The step is bound by
// streaming X from HBM; there is no contraction worth an MFMA at these D.
//
// Arithmetic mirrors heat/spatial/distance.py:59-64: d2 = (|x|^2 + |c|^2) - 2*(x.c), clamped at 0,
// scanned over k ascending with a strict '<' so the first index wins ties
// (torch.min semantics, heat/core/statistics.py:177).  The squared norms are sums of ROUNDED squares
// in feature order and the dot product is an FMA chain in feature order: for D <= 8 that is the
// order torch's CPU reduction and sgemm use, so the fp32 distances agree bit for bit with the
// reference's there.
#include "hkm_common.h"

namespace hkm {

// also computes squared centroid norms for the kernels that take them from global memory
__global__ void norms_kernel(const float* __restrict__ C, int K, int D, int64_t ldc,
                             float* __restrict__ cn, int kpad) {
    int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= kpad) return;
    float s = HKM_INF;
    if (k < K) {
        s = 0.f;
        const float* c = C + int64_t(k) * ldc;
        for (int d = 0; d < D; ++d) s = __fadd_rn(s, __fmul_rn(c[d], c[d]));
    }
    cn[k] = s;
}

int launch_norms(const float* C, int32_t K, int32_t D, int64_t ldc, float* cn, int32_t kpad,
                 hipStream_t st) {
    hipLaunchKernelGGL(norms_kernel, dim3((kpad + 255) / 256), dim3(256), 0, st, C, K, D, ldc, cn,
                       kpad);
    return check_launch("norms_kernel");
}

static constexpr int VALU_THREADS = 256;
static constexpr int VALU_LDS_FLOATS = 8192;  // 32 KB centroid tile

template <int D>
__global__ __launch_bounds__(VALU_THREADS) void assign_valu_kernel(
    const float* __restrict__ X, int64_t N, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, int32_t* __restrict__ labels, float* __restrict__ min_d2, int ktile,
    int64_t nbatches) {
    constexpr int S = D + 1;  // LDS row: D coordinates then the squared norm
    __shared__ float sC[VALU_LDS_FLOATS];
    const int tid = threadIdx.x;
    const int nkt = (K + ktile - 1) / ktile;

    auto stage = [&](int kt) {
        const int k0 = kt * ktile;
        const int kn = min(ktile, K - k0);
        for (int i = tid; i < kn * D; i += VALU_THREADS) {
            int r = i / D, c = i - r * D;
            sC[r * S + c] = C[int64_t(k0 + r) * ldc + c];
        }
        __syncthreads();
        for (int r = tid; r < kn; r += VALU_THREADS) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) s = __fadd_rn(s, __fmul_rn(sC[r * S + d], sC[r * S + d]));
            sC[r * S + D] = s;
        }
        __syncthreads();
        return kn;
    };

    int kn = 0;
    if (nkt == 1) kn = stage(0);

    for (int64_t b = blockIdx.x; b < nbatches; b += gridDim.x) {
        const int64_t i = b * VALU_THREADS + tid;
        const int64_t ir = i < N ? i : N - 1;
        float x[D];
        const float* xp = X + ir * ldx;
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = xp[d];
        float xn = 0.f;
#pragma unroll
        for (int d = 0; d < D; ++d) xn = __fadd_rn(xn, __fmul_rn(x[d], x[d]));

        float m = HKM_INF;
        int mi = 0;
        for (int kt = 0; kt < nkt; ++kt) {
            if (nkt > 1) {
                __syncthreads();
                kn = stage(kt);
            }
            const int k0 = kt * ktile;
#pragma unroll 4
            for (int k = 0; k < kn; ++k) {
                const float* c = sC + k * S;
                float dot = x[0] * c[0];
#pragma unroll
                for (int d = 1; d < D; ++d) dot = fmaf(x[d], c[d], dot);
                float dist = fmaf(-2.0f, dot, xn + c[D]);
                dist = fmaxf(dist, 0.0f);
                if (dist < m) {
                    m = dist;
                    mi = k0 + k;
                }
            }
        }
        if (i < N) {
            labels[i] = mi;
            if (min_d2) min_d2[i] = m;
        }
    }
}

template <int D>
static int launch_valu_t(const float* X, int64_t N, int64_t ldx, const float* C, int32_t K,
                         int64_t ldc, int32_t* labels, float* min_d2, hipStream_t st) {
    const int ktile = VALU_LDS_FLOATS / (D + 1);
    const int64_t nbatches = (N + VALU_THREADS - 1) / VALU_THREADS;
    int64_t grid = int64_t(num_cus()) * 8;
    if (grid > nbatches) grid = nbatches;
    prof_begin(st);
    hipLaunchKernelGGL(assign_valu_kernel<D>, dim3((unsigned)grid), dim3(VALU_THREADS), 0, st, X, N,
                       ldx, C, K, ldc, labels, min_d2, ktile, nbatches);
    prof_end(st);
    return check_launch("assign_valu_kernel");
}

int launch_assign_valu(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                       int64_t ldc, int32_t* labels, float* min_d2, hipStream_t st) {
#define HKM_CASE(d) \
    case d:         \
        return launch_valu_t<d>(X, N, ldx, C, K, ldc, labels, min_d2, st);
    switch (D) {
        HKM_CASE(1) HKM_CASE(2) HKM_CASE(3) HKM_CASE(4) HKM_CASE(5) HKM_CASE(6) HKM_CASE(7)
        HKM_CASE(8) HKM_CASE(9) HKM_CASE(10) HKM_CASE(11) HKM_CASE(12) HKM_CASE(13) HKM_CASE(14)
        HKM_CASE(15) HKM_CASE(16)
        default:
            return fail(HKM_EUNSUPPORTED, "assign_valu: D=%d outside 1..16", D);
    }
#undef HKM_CASE
}

}  // namespace hkm
