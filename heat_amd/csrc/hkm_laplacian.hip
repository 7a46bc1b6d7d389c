// Graph Laplacian from a similarity matrix (heat/graph/laplacian.py:100-142): zero the diagonal, apply the
// epsilon-neighbourhood threshold, row sums (the degrees), then L = D - A or L = I - D^-1/2 A D^-1/2.
// The reference makes about eight passes over the N x N matrix; here the degrees come from one read
// (laplacian_degree_kernel, one workgroup per row, fixed-order float64 tree) and L from a second read and one
// write that recompute the adjacency on the fly (laplacian_finish_kernel).  Bound: HBM, 2 reads + 1 write.
#include "hkm_common.h"

namespace hkm {

// adjacency entry from a similarity entry: mode 0 fully connected, 1 keep below eps, 2 keep above eps; an
// unweighted graph has 1 where the entry is kept.  The diagonal is zeroed BEFORE the threshold, as in the
// reference, so an unweighted "below eps" graph with eps > 0 has ones on its diagonal.
__device__ __forceinline__ float lap_adjacency(float s, bool diag, int mode, int weighted, float eps) {
    if (diag) s = 0.0f;
    if (mode == 0) return s;
    const bool keep = mode == 1 ? s < eps : s > eps;
    return weighted ? (keep ? s : 0.0f) : (keep ? 1.0f : 0.0f);
}

__global__ __launch_bounds__(256) void laplacian_degree_kernel(const float* __restrict__ S, int64_t N, int64_t lds,
                                                               int mode, int weighted, float eps,
                                                               float* __restrict__ degree) {
    __shared__ double sh[256];
    const int64_t i = blockIdx.x;
    const float* row = S + i * lds;
    double acc = 0.0;
    for (int64_t j = threadIdx.x; j < N; j += 256) acc += double(lap_adjacency(row[j], j == i, mode, weighted, eps));
    const double total = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) degree[i] = float(total);
}

// definition 0: L = diag(degree) - A;  1: L = -(A / sqrt(d_i)) / sqrt(d_j) with zero degrees replaced by 1
// and ones on the diagonal.
__global__ __launch_bounds__(256) void laplacian_finish_kernel(const float* __restrict__ S, int64_t N, int64_t lds,
                                                               int definition, int mode, int weighted, float eps,
                                                               const float* __restrict__ degree, float* __restrict__ L,
                                                               int64_t ldl) {
    const int64_t i = blockIdx.y;
    const int64_t j = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (j >= N) return;
    const float a = lap_adjacency(S[i * lds + j], j == i, mode, weighted, eps);
    float v;
    if (definition == 0) {
        v = (j == i ? degree[i] : 0.0f) - a;
    } else {
        const float di = degree[i] == 0.0f ? 1.0f : degree[i];
        const float dj = degree[j] == 0.0f ? 1.0f : degree[j];
        v = j == i ? 1.0f : ((a / sqrtf(di)) / sqrtf(dj)) * -1.0f;
    }
    L[i * ldl + j] = v;
}

int launch_laplacian(const float* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                     float eps, float* L, int64_t ldl, float* degree, hipStream_t st) {
    if (N == 0) return HKM_OK;
    hipLaunchKernelGGL(laplacian_degree_kernel, dim3((unsigned)N), dim3(256), 0, st, S, N, lds, mode, weighted, eps,
                       degree);
    int rc = check_launch("laplacian_degree_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(laplacian_finish_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)N), dim3(256), 0, st, S, N,
                       lds, definition, mode, weighted, eps, degree, L, ldl);
    return check_launch("laplacian_finish_kernel");
}

}  // namespace hkm
