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
template <typename T>
__device__ __forceinline__ T lap_adjacency(T s, bool diag, int mode, int weighted, T eps) {
    if (diag) s = T(0);
    if (mode == 0) return s;
    const bool keep = mode == 1 ? s < eps : s > eps;
    return weighted ? (keep ? s : T(0)) : (keep ? T(1) : T(0));
}

template <typename T>
__global__ __launch_bounds__(256) void laplacian_degree_kernel(const T* __restrict__ S, int64_t N, int64_t lds,
                                                               int mode, int weighted, T eps,
                                                               T* __restrict__ degree) {
    __shared__ double sh[256];
    const int64_t i = blockIdx.x;
    const T* row = S + i * lds;
    double acc = 0.0;
    for (int64_t j = threadIdx.x; j < N; j += 256) acc += double(lap_adjacency<T>(row[j], j == i, mode, weighted, eps));
    const double total = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) degree[i] = T(total);
}

// definition 0: L = diag(degree) - A;  1: L = -(A / sqrt(d_i)) / sqrt(d_j) with zero degrees replaced by 1
// and ones on the diagonal.  S and L may be the same matrix (every entry is read and written by one thread),
// so neither is declared free of aliases.  Rows run along grid.x (up to 2^31 - 1), 256-column slices along
// grid.y.
template <typename T>
__global__ __launch_bounds__(256) void laplacian_finish_kernel(const T* S, int64_t N, int64_t lds, int definition,
                                                               int mode, int weighted, T eps,
                                                               const T* __restrict__ degree, T* L, int64_t ldl) {
    const int64_t i = blockIdx.x;
    const int64_t j = int64_t(blockIdx.y) * 256 + threadIdx.x;
    if (j >= N) return;
    const T a = lap_adjacency<T>(S[i * lds + j], j == i, mode, weighted, eps);
    T v;
    if (definition == 0) {
        v = (j == i ? degree[i] : T(0)) - a;
    } else {
        const T di = degree[i] == T(0) ? T(1) : degree[i];
        const T dj = degree[j] == T(0) ? T(1) : degree[j];
        if (sizeof(T) == 8 && !weighted && mode != 0) {
            // an unweighted graph is an int32 adjacency matrix in the reference, divided by the float32 square
            // roots of its integer degrees (heat/graph/laplacian.py:96-97,129-133): float32 arithmetic whatever
            // the similarities' type was (adjacency and degrees are small integers, exact in either type)
            v = j == i ? T(1) : T(((float(a) / sqrtf(float(di))) / sqrtf(float(dj))) * -1.0f);
        } else {
            v = j == i ? T(1) : ((a / sqrt(di)) / sqrt(dj)) * T(-1);
        }
    }
    L[i * ldl + j] = v;
}

template <typename T>
static int launch_laplacian_t(const T* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                              T eps, T* L, int64_t ldl, T* degree, hipStream_t st) {
    if (N == 0) return HKM_OK;
    hipLaunchKernelGGL(laplacian_degree_kernel<T>, dim3((unsigned)N), dim3(256), 0, st, S, N, lds, mode, weighted, eps,
                       degree);
    int rc = check_launch("laplacian_degree_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(laplacian_finish_kernel<T>, dim3((unsigned)N, (unsigned)((N + 255) / 256)), dim3(256), 0, st, S,
                       N, lds, definition, mode, weighted, eps, static_cast<const T*>(degree), L, ldl);
    return check_launch("laplacian_finish_kernel");
}

int launch_laplacian(const float* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                     float eps, float* L, int64_t ldl, float* degree, hipStream_t st) {
    return launch_laplacian_t<float>(S, N, lds, definition, mode, weighted, eps, L, ldl, degree, st);
}

int launch_laplacian_f64(const double* S, int64_t N, int64_t lds, int32_t definition, int32_t mode, int32_t weighted,
                         double eps, double* L, int64_t ldl, double* degree, hipStream_t st) {
    return launch_laplacian_t<double>(S, N, lds, definition, mode, weighted, eps, L, ldl, degree, st);
}

}  // namespace hkm
