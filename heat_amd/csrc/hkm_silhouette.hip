// Per-sample, per-cluster sums of Euclidean distances without the N x N matrix: the
// `clust_dists = matmul(cdist(X, X), labels == unique_labels)` step of silhouette_samples
// (heat/cluster/metrics.py:135-151).
//
// The caller passes the rows grouped by cluster (a permutation and the cluster offsets).  Workgroup
// (tile of 64 samples, cluster c) walks the rows of cluster c in tiles of 64 (4 x 4 register block per
// lane, both tiles staged through LDS in chunks of 16 features, sum (x - y)^2 in fp32, the direct form
// of torch.cdist), takes the square root of every pair and adds it up in float64 per lane; the 16 lanes
// that share a sample are added in a fixed order.  Bound: the vector ALU, 2 operations per
// (sample, row, feature) plus one square root per pair.
#include "hkm_common.h"

namespace hkm {

static constexpr int SIL_T = 64;
static constexpr int SIL_KC = 16;

__global__ __launch_bounds__(256) void silhouette_sums_kernel(const float* __restrict__ X, int64_t N, int64_t ldx, int D,
                                                              const int64_t* __restrict__ perm,
                                                              const int64_t* __restrict__ offsets, int K,
                                                              float* __restrict__ S, int64_t lds) {
    __shared__ float sQ[SIL_KC][SIL_T + 4];
    __shared__ float sR[SIL_KC][SIL_T + 4];
    __shared__ int64_t sRow[SIL_T];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int lk = tid & 15, lr = tid >> 4;
    const int64_t i0 = int64_t(blockIdx.x) * SIL_T;
    const int c = blockIdx.y;
    const int64_t r_begin = offsets[c], r_end = offsets[c + 1];

    double sum[4] = {0.0, 0.0, 0.0, 0.0};
    for (int64_t j0 = r_begin; j0 < r_end; j0 += SIL_T) {
        __syncthreads();
        if (tid < SIL_T) sRow[tid] = j0 + tid < r_end ? perm[j0 + tid] : int64_t(-1);
        float acc[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[a][b] = 0.0f;
        for (int d0 = 0; d0 < D; d0 += SIL_KC) {
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int r = lr + 16 * q;
                const int d = d0 + lk;
                const int64_t gi = i0 + r, gj = sRow[r];
                sQ[lk][r] = (gi < N && d < D) ? X[gi * ldx + d] : 0.0f;
                sR[lk][r] = (gj >= 0 && d < D) ? X[gj * ldx + d] : 0.0f;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < SIL_KC; ++k) {
                float qa[4], rb[4];
#pragma unroll
                for (int a = 0; a < 4; ++a) qa[a] = sQ[k][ty * 4 + a];
#pragma unroll
                for (int b = 0; b < 4; ++b) rb[b] = sR[k][tx * 4 + b];
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const float df = qa[a] - rb[b];
                        acc[a][b] = fmaf(df, df, acc[a][b]);
                    }
            }
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const bool valid = j0 + tx * 4 + b < r_end;
#pragma unroll
            for (int a = 0; a < 4; ++a) sum[a] += valid ? double(sqrtf(acc[a][b])) : 0.0;
        }
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        double s = sum[a];
#pragma unroll
        for (int w = 1; w < 16; w <<= 1) s += __shfl_xor(s, w);
        const int64_t gi = i0 + ty * 4 + a;
        if (tx == 0 && gi < N) S[gi * lds + c] = float(s);
    }
}

// One thread per sample: a = S[i][own] / max(n_own - 1, 1), b = min over the other clusters of
// S[i][c] / n_c, silhouette = (b - a) / max(a, b), 0 for a sample alone in its cluster and wherever the
// quotient is not a number (heat/cluster/metrics.py:153-176), all in float32.
__global__ void silhouette_finish_kernel(const float* __restrict__ S, int64_t N, int K, int64_t lds,
                                         const int64_t* __restrict__ enc, const int64_t* __restrict__ counts,
                                         float* __restrict__ out) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const int own = int(enc[i]);
    const int64_t n_own = counts[own];
    const float a = S[i * lds + own] / float(n_own - 1 > 0 ? n_own - 1 : 1);
    float b = HKM_INF;
    for (int c = 0; c < K; ++c)
        if (c != own) b = fminf(b, S[i * lds + c] / float(counts[c]));
    float v = (b - a) / fmaxf(a, b);
    if (n_own <= 1 || v != v) v = 0.0f;
    out[i] = fminf(fmaxf(v, -3.402823466e38f), 3.402823466e38f);
}

int launch_silhouette_finish(const float* S, int64_t N, int32_t K, int64_t lds, const int64_t* enc,
                             const int64_t* counts, float* out, hipStream_t st) {
    if (N == 0) return HKM_OK;
    hipLaunchKernelGGL(silhouette_finish_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, st, S, N, K, lds, enc,
                       counts, out);
    return check_launch("silhouette_finish_kernel");
}

int launch_silhouette_sums(const float* X, int64_t N, int32_t D, int64_t ldx, const int64_t* perm,
                           const int64_t* offsets, int32_t K, float* S, int64_t lds, hipStream_t st) {
    if (N == 0) return HKM_OK;
    hipLaunchKernelGGL(silhouette_sums_kernel, dim3((unsigned)((N + SIL_T - 1) / SIL_T), (unsigned)K), dim3(256), 0, st, X,
                       N, ldx, D, perm, offsets, K, S, lds);
    return check_launch("silhouette_sums_kernel");
}

}  // namespace hkm
