// float64 data: fused quadratic-expansion distance + argmin on the fp64 vector ALU.  The reference
// runs float64 inputs through the same op sequence in float64 (promote(X, Y, float32) keeps float64,
// heat/spatial/distance.py:392-403), so d2 = max(0, (|x|^2 + |c|^2) - 2 x.c) is evaluated in fp64
// here as well; the N x K matrix is never written.  Same tiling as the Manhattan kernel: a workgroup
// owns 64 points and walks the centroids in tiles of 64 (4 x 4 register block per lane, 16-feature
// chunks through LDS); squared norms are accumulated from the staged tiles on the way.
#include "hkm_common.h"

namespace hkm {

static constexpr int F64_T = 64;
static constexpr int F64_KC = 16;

__global__ __launch_bounds__(256) void assign_f64_kernel(const double* __restrict__ X, int64_t N,
                                                         int64_t ldx, const double* __restrict__ C,
                                                         int K, int64_t ldc, int D,
                                                         int32_t* __restrict__ labels,
                                                         double* __restrict__ min_d2) {
    __shared__ double sX[F64_KC][F64_T + 2];
    __shared__ double sC[F64_KC][F64_T + 2];
    __shared__ double sXn[F64_T], sCn[F64_T];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int lk = tid & 15, lr = tid >> 4;
    const int64_t i0 = int64_t(blockIdx.x) * F64_T;

    // squared norms of the tile's points, summed in feature order
    if (tid < F64_T) {
        const int64_t g = i0 + tid;
        double s = 0.0;
        if (g < N) {
            const double* row = X + g * ldx;
            for (int d = 0; d < D; ++d) s = fma(row[d], row[d], s);
        }
        sXn[tid] = s;
    }

    double bd[4];
    int bi[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        bd[a] = __builtin_inf();
        bi[a] = 0x7fffffff;
    }

    for (int j0 = 0; j0 < K; j0 += F64_T) {
        __syncthreads();  // previous tile's sCn is no longer read
        if (tid < F64_T) {
            const int g = j0 + tid;
            double s = 0.0;
            if (g < K) {
                const double* row = C + int64_t(g) * ldc;
                for (int d = 0; d < D; ++d) s = fma(row[d], row[d], s);
            }
            sCn[tid] = s;
        }
        double acc[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[a][b] = 0.0;
        for (int d0 = 0; d0 < D; d0 += F64_KC) {
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int r = lr + 16 * q;
                const int d = d0 + lk;
                const int64_t gi = i0 + r;
                const int gj = j0 + r;
                sX[lk][r] = (gi < N && d < D) ? X[gi * ldx + d] : 0.0;
                sC[lk][r] = (gj < K && d < D) ? C[int64_t(gj) * ldc + d] : 0.0;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < F64_KC; ++k) {
                double xa[4], cb[4];
#pragma unroll
                for (int a = 0; a < 4; ++a) xa[a] = sX[k][ty * 4 + a];
#pragma unroll
                for (int b = 0; b < 4; ++b) cb[b] = sC[k][tx * 4 + b];
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int b = 0; b < 4; ++b) acc[a][b] = fma(xa[a], cb[b], acc[a][b]);
            }
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const double xn = sXn[ty * 4 + a];
            double d = __builtin_inf();
            int i = 0x7fffffff;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int gj = j0 + tx * 4 + b;
                if (gj >= K) continue;
                double v = fma(-2.0, acc[a][b], xn + sCn[tx * 4 + b]);
                v = v > 0.0 ? v : (v != v ? v : 0.0);
                if (v < d) {  // ascending index, strict '<': first index wins ties
                    d = v;
                    i = gj;
                }
            }
#pragma unroll
            for (int w = 1; w < 16; w <<= 1) {
                const double od = __shfl_xor(d, w);
                const int oi = __shfl_xor(i, w);
                if (od < d || (od == d && oi < i)) {
                    d = od;
                    i = oi;
                }
            }
            if (d < bd[a] || (d == bd[a] && i < bi[a])) {
                bd[a] = d;
                bi[a] = i;
            }
        }
    }

    if (tx == 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t gi = i0 + ty * 4 + a;
            if (gi >= N) continue;
            labels[gi] = bi[a] == 0x7fffffff ? 0 : bi[a];
            if (min_d2) min_d2[gi] = bd[a];
        }
    }
}

// Narrow rows and few centroids (D <= 8, K (D + 1) <= F64S_LDS): the 64 x 64 tile would be mostly
// padding.  One point per lane, the centroids and their squared norms broadcast from LDS; every sum
// in feature order with fma, so the values equal those of the tiled kernel bit for bit.
static constexpr int F64S_THREADS = 256;
static constexpr int F64S_LDS = 2048;  // doubles: K rows of D coordinates + the squared norm

template <int D>
__global__ __launch_bounds__(F64S_THREADS) void assign_f64_small_kernel(
    const double* __restrict__ X, int64_t N, int64_t ldx, const double* __restrict__ C, int K, int64_t ldc,
    int32_t* __restrict__ labels, double* __restrict__ min_d2, int64_t nbatches) {
    __shared__ double sC[F64S_LDS];
    const int tid = threadIdx.x;
    for (int k = tid; k < K; k += F64S_THREADS) {
        const double* row = C + int64_t(k) * ldc;
        double s = 0.0;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            sC[k * (D + 1) + d] = row[d];
            s = fma(row[d], row[d], s);
        }
        sC[k * (D + 1) + D] = s;
    }
    __syncthreads();
    for (int64_t b = blockIdx.x; b < nbatches; b += gridDim.x) {
        const int64_t i = b * F64S_THREADS + tid;
        const double* xp = X + (i < N ? i : N - 1) * ldx;
        double x[D], xn = 0.0;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            x[d] = xp[d];
            xn = fma(x[d], x[d], xn);
        }
        double m = __builtin_inf();
        int mi = 0x7fffffff;
#pragma unroll 4
        for (int k = 0; k < K; ++k) {
            const double* c = sC + k * (D + 1);
            double dot = 0.0;
#pragma unroll
            for (int d = 0; d < D; ++d) dot = fma(x[d], c[d], dot);
            double v = fma(-2.0, dot, xn + c[D]);
            v = v > 0.0 ? v : (v != v ? v : 0.0);
            if (v < m) {  // ascending index, strict '<': first index wins ties
                m = v;
                mi = k;
            }
        }
        if (i < N) {
            labels[i] = mi == 0x7fffffff ? 0 : mi;
            if (min_d2) min_d2[i] = m;
        }
    }
}

template <int D>
static int launch_assign_f64_small_t(const double* X, int64_t N, int64_t ldx, const double* C, int32_t K,
                                     int64_t ldc, int32_t* labels, double* min_d2, hipStream_t st) {
    const int64_t nbatches = (N + F64S_THREADS - 1) / F64S_THREADS;
    int64_t grid = int64_t(num_cus()) * 8;
    if (grid > nbatches) grid = nbatches;
    hipLaunchKernelGGL(assign_f64_small_kernel<D>, dim3((unsigned)grid), dim3(F64S_THREADS), 0, st, X, N, ldx, C, K,
                       ldc, labels, min_d2, nbatches);
    return check_launch("assign_f64_small_kernel");
}

int launch_assign_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const double* C, int32_t K,
                      int64_t ldc, int32_t* labels, double* min_d2, hipStream_t st) {
    if (D <= 8 && int64_t(K) * (D + 1) <= F64S_LDS) {
#define HKM_CASE(d) \
    case d:         \
        return launch_assign_f64_small_t<d>(X, N, ldx, C, K, ldc, labels, min_d2, st);
        switch (D) {
            HKM_CASE(1) HKM_CASE(2) HKM_CASE(3) HKM_CASE(4) HKM_CASE(5) HKM_CASE(6) HKM_CASE(7) HKM_CASE(8)
        }
#undef HKM_CASE
    }
    const int64_t tiles = (N + F64_T - 1) / F64_T;
    if (tiles > 0x7fffffffLL) return fail(HKM_EUNSUPPORTED, "assign_f64: too many row tiles");
    hipLaunchKernelGGL(assign_f64_kernel, dim3((unsigned)tiles), dim3(256), 0, st, X, N, ldx, C, K, ldc, D,
                       labels, min_d2);
    return check_launch("assign_f64_kernel");
}

}  // namespace hkm
