// Device side of the k-means|| centroid initialisation (heat/cluster/_kcluster.py:146-247,283-350):
// the distance work is the assign kernel with its min d^2 output; what is left are an ordered
// Bernoulli selection of candidate rows and a histogram of labels.  Both are integer work and
// reproducible: the selection is a count / scan / write compaction in row order, the histogram
// uses integer atomics only.
#include "hkm_common.h"

namespace hkm {

// row i is selected iff u[i] <= (oversampling * sqrt(min_d2[i])) / max(cost, 1e-12), evaluated in
// fp32 in that order (_kcluster.py:314-322)
__device__ __forceinline__ bool selected(float d2, float u, float os, float denom) {
    const float p = (os * sqrtf(d2)) / denom;
    return u <= p;
}

__global__ __launch_bounds__(256) void select_count_kernel(const float* __restrict__ d2,
                                                           const float* __restrict__ u, int64_t n,
                                                           int64_t per_block,
                                                           const float* __restrict__ cost, float os,
                                                           long long* __restrict__ block_cnt) {
    __shared__ int sh[256];
    const float denom = fmaxf(*cost, 1e-12f);
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    int c = 0;
    for (int64_t i = b0 + threadIdx.x; i < b1; i += 256) c += selected(d2[i], u[i], os, denom) ? 1 : 0;
    sh[threadIdx.x] = c;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if (threadIdx.x < w) sh[threadIdx.x] += sh[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) block_cnt[blockIdx.x] = sh[0];
}

// exclusive scan of the block counts in place (nb <= RED_SLOTS), total to *count
__global__ __launch_bounds__(256) void select_scan_kernel(long long* __restrict__ block_cnt, int nb,
                                                          long long* __restrict__ count) {
    __shared__ long long sh[256];
    const int per = (nb + 255) / 256;
    const int i0 = threadIdx.x * per, i1 = min(nb, i0 + per);
    long long s = 0;
    for (int i = i0; i < i1; ++i) s += block_cnt[i];
    sh[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        long long run = 0;
        for (int t = 0; t < 256; ++t) {
            const long long v = sh[t];
            sh[t] = run;
            run += v;
        }
        *count = run;
    }
    __syncthreads();
    long long run = sh[threadIdx.x];
    for (int i = i0; i < i1; ++i) {
        const long long v = block_cnt[i];
        block_cnt[i] = run;
        run += v;
    }
}

__global__ __launch_bounds__(256) void select_write_kernel(const float* __restrict__ d2,
                                                           const float* __restrict__ u, int64_t n,
                                                           int64_t per_block,
                                                           const float* __restrict__ cost, float os,
                                                           const long long* __restrict__ block_off,
                                                           int64_t* __restrict__ idx, int64_t cap) {
    __shared__ int wave_cnt[4];
    const float denom = fmaxf(*cost, 1e-12f);
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    long long run = block_off[blockIdx.x];
    for (int64_t base = b0; base < b1; base += 256) {
        const int64_t i = base + threadIdx.x;
        const bool f = i < b1 && selected(d2[i], u[i], os, denom);
        const unsigned long long m = __ballot(f);
        const int before = __popcll(m & ((1ull << lane) - 1ull));
        if (lane == 0) wave_cnt[wave] = __popcll(m);
        __syncthreads();
        int off = 0, tot = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int c = wave_cnt[w];
            if (w < wave) off += c;
            tot += c;
        }
        if (f) {
            const long long pos = run + off + before;
            if (pos < cap) idx[pos] = i;
        }
        run += tot;
        __syncthreads();
    }
}

int launch_select(const float* d2, const float* u, int64_t N, const float* cost, float os,
                  int64_t* idx, int64_t cap, int64_t* count, double* red, hipStream_t st) {
    int nb = int((N + 16383) / 16384);
    if (nb < 1) nb = 1;
    if (nb > RED_SLOTS) nb = RED_SLOTS;
    int64_t per_block = (N + nb - 1) / nb;
    per_block = (per_block + 255) / 256 * 256;
    long long* bc = reinterpret_cast<long long*>(red);
    hipLaunchKernelGGL(select_count_kernel, dim3(nb), dim3(256), 0, st, d2, u, N, per_block, cost, os, bc);
    int rc = check_launch("select_count_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(select_scan_kernel, dim3(1), dim3(256), 0, st, bc, nb,
                       reinterpret_cast<long long*>(count));
    if ((rc = check_launch("select_scan_kernel"))) return rc;
    hipLaunchKernelGGL(select_write_kernel, dim3(nb), dim3(256), 0, st, d2, u, N, per_block, cost, os,
                       bc, idx, cap);
    return check_launch("select_write_kernel");
}

// ---- histogram of labels ---------------------------------------------------------------------
static constexpr int HIST_LDS = 4096;

__global__ __launch_bounds__(256) void zero_i64_kernel(long long* __restrict__ p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

__global__ __launch_bounds__(256) void label_hist_kernel(const int32_t* __restrict__ labels,
                                                         int64_t n, int64_t per_block, int K,
                                                         unsigned long long* __restrict__ counts) {
    __shared__ unsigned int sh[HIST_LDS];
    const bool lds = K <= HIST_LDS;
    if (lds) {
        for (int k = threadIdx.x; k < K; k += 256) sh[k] = 0;
        __syncthreads();
    }
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    for (int64_t i = b0 + threadIdx.x; i < b1; i += 256) {
        const int l = labels[i];
        if (l < 0 || l >= K) continue;
        if (lds) atomicAdd(&sh[l], 1u);
        else atomicAdd(&counts[l], 1ull);
    }
    if (lds) {
        __syncthreads();
        for (int k = threadIdx.x; k < K; k += 256) {
            const unsigned int c = sh[k];
            if (c) atomicAdd(&counts[k], (unsigned long long)c);
        }
    }
}

int launch_label_counts(const int32_t* labels, int64_t N, int32_t K, int64_t* counts,
                        hipStream_t st) {
    hipLaunchKernelGGL(zero_i64_kernel, dim3((K + 255) / 256), dim3(256), 0, st,
                       reinterpret_cast<long long*>(counts), K);
    int rc = check_launch("zero_i64_kernel");
    if (rc || N == 0) return rc;
    int64_t nb = (N + 65535) / 65536;
    const int64_t cap = int64_t(num_cus()) * 8;
    if (nb > cap) nb = cap;
    const int64_t per_block = (N + nb - 1) / nb;
    hipLaunchKernelGGL(label_hist_kernel, dim3((unsigned)nb), dim3(256), 0, st, labels, N, per_block, K,
                       reinterpret_cast<unsigned long long*>(counts));
    return check_launch("label_hist_kernel");
}

}  // namespace hkm
