// Full pairwise distance matrices for the public cdist / rbf / manhattan API
// (heat/spatial/distance.py:17-133): quadratic expansion max(0, (|x|^2 + |y|^2) - 2 x.y), the direct
// form sum((x-y)^2) and sum|x-y|, followed by sqrt or exp(-d2 / (2 sigma^2)).  The output is M x Nn
// floats, so for the feature counts these functions are used with the kernel is bound by writing the
// matrix; a 64 x 64 output tile per workgroup with a 4 x 4 register block per lane keeps the X / Y
// re-reads in L2 and the stores 16 bytes wide.
#include "hkm_common.h"

namespace hkm {

static constexpr int CD_T = 64;   // tile edge
static constexpr int CD_KC = 16;  // feature chunk

// METRIC: 0 = quadratic expansion (squared, optional sqrt), 1 = direct sum((x-y)^2) (optional sqrt),
//         2 = sum |x-y|;  gauss != 0 applies exp(-d2 * gauss) to the squared distance instead of sqrt
// square roots of a lane's block: float takes the short correctly rounded form unless some lane of
// the wave holds a positive value below its range (one integer minimum tree decides)
__device__ __forceinline__ void cd_sqrt_block(float (&v)[4][4]) {
    unsigned m = 0xffffffffu;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; b += 2) m = min(m, min(sqrt_short_key(v[a][b]), sqrt_short_key(v[a][b + 1])));
    if (__builtin_amdgcn_ballot_w64(m < SQRT_SHORT_KEY_LIMIT) != 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) v[a][b] = sqrtf(v[a][b]);
    } else {
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) v[a][b] = sqrt_rn_short(v[a][b]);
    }
}
__device__ __forceinline__ void cd_sqrt_block(double (&v)[4][4]) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) v[a][b] = sqrt(v[a][b]);
}
__device__ __forceinline__ void store_row4(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store_row4(double* p, const double (&v)[4]) {
#pragma unroll
    for (int b = 0; b < 4; ++b) p[b] = v[b];
}
__device__ __forceinline__ float cd_exp(float v) { return expf(v); }
__device__ __forceinline__ double cd_exp(double v) { return exp(v); }
__device__ __forceinline__ float cd_abs(float v) { return fabsf(v); }
__device__ __forceinline__ double cd_abs(double v) { return fabs(v); }
__device__ __forceinline__ float cd_fma(float a, float b, float c) { return fmaf(a, b, c); }
__device__ __forceinline__ double cd_fma(double a, double b, double c) { return fma(a, b, c); }

// KU: features of a staged chunk that take part in the arithmetic (rows of at most 4 / 8 features
// would otherwise spend three quarters / half of their instructions on the zero padding)
template <typename T, int METRIC, int KU>
__global__ __launch_bounds__(256) void cdist_kernel(const T* __restrict__ X, int64_t M,
                                                    int64_t ldx, const T* __restrict__ Y,
                                                    int64_t Nn, int64_t ldy, int D,
                                                    T* __restrict__ out, int64_t ldo,
                                                    int sqrt_flag, T gauss, int64_t tiles_n, bool vec_out) {
    __shared__ T sX[CD_KC][CD_T + 4];
    __shared__ T sY[CD_KC][CD_T + 4];
    __shared__ T sXn[CD_T], sYn[CD_T];
    const int tid = threadIdx.x;
    const int64_t tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int64_t i0 = tm * CD_T, j0 = tn * CD_T;

    // squared norms of the tile's rows / columns (quadratic expansion only), each summed in feature
    // order from the staged chunks: thread r < 64 owns row r of the X tile, thread 64 + r row r of Y
    T nrm = T(0);

    const int tx = tid & 15, ty = tid >> 4;
    T acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = T(0);

    // staging role: element (row lr, feature lk) of both tiles, 4 passes of 16 rows
    const int lk = tid & 15, lr = tid >> 4;
    for (int d0 = 0; d0 < D; d0 += CD_KC) {
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int r = lr + 16 * q;
            const int d = d0 + lk;
            const int64_t gi = i0 + r, gj = j0 + r;
            sX[lk][r] = (gi < M && d < D) ? X[gi * ldx + d] : T(0);
            sY[lk][r] = (gj < Nn && d < D) ? Y[gj * ldy + d] : T(0);
        }
        __syncthreads();
        if (METRIC == 0 && tid < 2 * CD_T) {
            const T(*tile)[CD_T + 4] = tid < CD_T ? sX : sY;
            const int r = tid & (CD_T - 1);
#pragma unroll
            for (int k = 0; k < KU; ++k) nrm = cd_fma(tile[k][r], tile[k][r], nrm);
        }
#pragma unroll
        for (int k = 0; k < KU; ++k) {
            T xa[4], yb[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) xa[a] = sX[k][ty * 4 + a];
#pragma unroll
            for (int b = 0; b < 4; ++b) yb[b] = sY[k][tx * 4 + b];
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    if (METRIC == 0) {
                        acc[a][b] = cd_fma(xa[a], yb[b], acc[a][b]);
                    } else if (METRIC == 1) {
                        const T df = xa[a] - yb[b];
                        acc[a][b] = cd_fma(df, df, acc[a][b]);
                    } else {
                        acc[a][b] += cd_abs(xa[a] - yb[b]);
                    }
                }
        }
    }
    if (METRIC == 0) {
        if (tid < 2 * CD_T) (tid < CD_T ? sXn : sYn)[tid & (CD_T - 1)] = nrm;
        __syncthreads();
    }

    // epilogue over the lane's 4 x 4 block, in place
    if (METRIC == 0) {
        T yn[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) yn[b] = sYn[tx * 4 + b];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const T xn = sXn[ty * 4 + a];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                // the reference's order; clamp at 0 (a NaN passes: NaN < 0 is false; the value is never
                // -0 because the sum of the norms is never -0)
                const T d = cd_fma(T(-2), acc[a][b], xn + yn[b]);
                acc[a][b] = d < T(0) ? T(0) : d;
            }
        }
    }
    if (METRIC != 2) {
        if (gauss != T(0)) {
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b) acc[a][b] = cd_exp(-acc[a][b] * gauss);
        } else if (sqrt_flag) {
            cd_sqrt_block(acc);
        }
    }
    // 16-byte stores where the row of four lies inside the matrix and is aligned
    const int64_t gj0 = j0 + tx * 4;
    const bool vec4 = sizeof(T) == 4 && vec_out && gj0 + 3 < Nn;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int64_t gi = i0 + ty * 4 + a;
        if (gi >= M) continue;
        T* row = out + gi * ldo + gj0;
        if (vec4) {
            store_row4(row, acc[a]);
        } else {
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (gj0 + b < Nn) row[b] = acc[a][b];
        }
    }
}

template <typename T>
static int launch_cdist_t(const T* X, int64_t M, int64_t ldx, const T* Y, int64_t Nn, int64_t ldy,
                          int32_t D, T* out, int64_t ldo, int32_t metric, int32_t sqrt_flag, T gauss,
                          hipStream_t st) {
    const int64_t tiles_m = (M + CD_T - 1) / CD_T, tiles_n = (Nn + CD_T - 1) / CD_T;
    const int64_t total = tiles_m * tiles_n;
    if (total > 0x7fffffffLL) return fail(HKM_EUNSUPPORTED, "cdist: %lld tiles exceed the grid limit", (long long)total);
#define HKM_GO1(MET, KU)                                                                                      \
    hipLaunchKernelGGL((cdist_kernel<T, MET, KU>), dim3((unsigned)total), dim3(256), 0, st, X, M, ldx, Y, Nn, \
                       ldy, D, out, ldo, sqrt_flag, gauss, tiles_n, vec_out)
#define HKM_GO(MET)                  \
    do {                             \
        if (D <= 4) HKM_GO1(MET, 4); \
        else if (D <= 8) HKM_GO1(MET, 8); \
        else HKM_GO1(MET, CD_KC);    \
    } while (0)
    const bool vec_out = aligned16(out) && ldo % 4 == 0;
    if (metric == 0) HKM_GO(0);
    else if (metric == 1) HKM_GO(1);
    else HKM_GO(2);
#undef HKM_GO
#undef HKM_GO1
    return check_launch("cdist_kernel");
}

int launch_cdist(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                 int32_t D, float* out, int64_t ldo, int32_t metric, int32_t sqrt_flag, float gauss,
                 hipStream_t st) {
    // the quadratic expansion is a matrix product: matrix cores from 16 features on
    if (metric == 0 && cdist_mfma_eligible(M, Nn, D, ldx, ldy, ldo))
        return launch_cdist_mfma(X, M, ldx, Y, Nn, ldy, D, out, ldo, sqrt_flag, gauss, st);
    return launch_cdist_t<float>(X, M, ldx, Y, Nn, ldy, D, out, ldo, metric, sqrt_flag, gauss, st);
}

int launch_cdist_f64(const double* X, int64_t M, int64_t ldx, const double* Y, int64_t Nn, int64_t ldy,
                     int32_t D, double* out, int64_t ldo, int32_t metric, int32_t sqrt_flag, double gauss,
                     hipStream_t st) {
    return launch_cdist_t<double>(X, M, ldx, Y, Nn, ldy, D, out, ldo, metric, sqrt_flag, gauss, st);
}

}  // namespace hkm
