// Per-cluster mean by a stable counting sort of the row indices followed by segmented column sums.
//
//   1. group: the rows are cut into blocks, one wave per block.  A first pass counts the labels of
//      every block (integer LDS atomics), a scan turns the counts into the position of every
//      (block, cluster) run inside the cluster's segment, a second pass walks the block again 64 rows
//      at a time and gives every row its place: lanes with equal labels are found with one ballot per
//      label bit, the rank of a lane among them is a population count, and a running per-cluster
//      cursor in LDS (one writer per cluster and step: the lowest lane of the group) advances.  The
//      result `perm` lists the rows of every cluster in ASCENDING row order -- a stable sort, so it
//      does not depend on scheduling.
//   2. segmented sums: a workgroup takes up to 2048 consecutive entries of one cluster's segment and a
//      32-column slice; its 8 row-lanes add rows r, r+8, ... in order (several independent loads in
//      flight, no LDS traffic, no atomics) and are combined in lane order -- all in fp64, like the
//      reference's float64 x * selection: the sum of a cluster is rounded once, when the mean is
//      stored, so the means equal the reference's bit for bit except where its own fp64 sum rounds.
//   3. finalize: the chunk partials of a cluster are added in chunk order in fp64, divided by the
//      count (rounded through fp32 like the reference, heat/core/rounding.py:156-164), stored as fp32;
//      an empty cluster gives a zero row (heat/cluster/kmeans.py:88-101).
// Every floating-point sum has a fixed order: results are bit-reproducible.
#include <string.h>

#include "hkm_common.h"

namespace hkm {

static constexpr int SRT_R = 2048;      // rows of one cluster per segmented-sum workgroup
static constexpr int SRT_MAXBLK = 4096;  // blocks of the grouping passes (one wave each)
static constexpr int SRT_MAXK = 4096;    // per-wave LDS cursors: 4 waves x K x 4 B <= 64 KB

bool sorted_update_eligible(int32_t K) { return K <= SRT_MAXK; }

int64_t sorted_block_rows(int64_t N) {
    int64_t b = (N + SRT_MAXBLK - 1) / SRT_MAXBLK;
    b = (b + 63) / 64 * 64;
    return b < 1024 ? 1024 : b;
}

__global__ __launch_bounds__(256) void srt_count_kernel(const int32_t* __restrict__ labels, int64_t N,
                                                        int K, int64_t blk_rows, int nblk,
                                                        int32_t* __restrict__ blk_cnt) {
    extern __shared__ int lcnt[];  // [4 waves][K]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.x * 4 + wave;
    int* cnt = lcnt + wave * K;
    for (int k = lane; k < K; k += 64) cnt[k] = 0;
    if (b >= nblk) return;
    wave_lds_sync();
    const int64_t r0 = int64_t(b) * blk_rows, r1 = min(N, r0 + blk_rows);
    for (int64_t r = r0 + lane; r < r1; r += 64) {
        const int l = labels[r];
        if (l >= 0 && l < K) atomicAdd(&cnt[l], 1);
    }
    wave_lds_sync();
    for (int k = lane; k < K; k += 64) blk_cnt[int64_t(b) * K + k] = cnt[k];
}

// one workgroup per cluster: exclusive scan of its counts over the blocks (in place), total to counts
__global__ __launch_bounds__(256) void srt_scan_blocks_kernel(int32_t* __restrict__ blk_cnt, int nblk,
                                                              int K, int64_t* __restrict__ counts) {
    __shared__ int sh[256];
    const int k = blockIdx.x, tid = threadIdx.x;
    const int per = (nblk + 255) / 256;
    const int b0 = tid * per, b1 = min(nblk, b0 + per);
    int s = 0;
    for (int b = b0; b < b1; ++b) s += blk_cnt[int64_t(b) * K + k];
    sh[tid] = s;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int t = 0; t < 256; ++t) {
            const int v = sh[t];
            sh[t] = run;
            run += v;
        }
        counts[k] = run;
    }
    __syncthreads();
    int run = sh[tid];
    for (int b = b0; b < b1; ++b) {
        const int v = blk_cnt[int64_t(b) * K + k];
        blk_cnt[int64_t(b) * K + k] = run;
        run += v;
    }
}

__global__ __launch_bounds__(256) void srt_scatter_kernel(const int32_t* __restrict__ labels, int64_t N,
                                                          int K, int nbits, int64_t blk_rows, int nblk,
                                                          const int32_t* __restrict__ blk_base,
                                                          const int64_t* __restrict__ offsets,
                                                          int32_t* __restrict__ perm) {
    extern __shared__ int lcur[];  // [4 waves][K] next free position of every cluster, relative to its segment
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.x * 4 + wave;
    if (b >= nblk) return;
    int* cur = lcur + wave * K;
    for (int k = lane; k < K; k += 64) cur[k] = blk_base[int64_t(b) * K + k];
    const int64_t r0 = int64_t(b) * blk_rows, r1 = min(N, r0 + blk_rows);
    const unsigned long long lt = (1ull << lane) - 1ull;
    for (int64_t base = r0; base < r1; base += 64) {
        wave_lds_sync();  // the cursors other lanes advanced in the previous batch
        const int64_t r = base + lane;
        int l = r < r1 ? labels[r] : -1;
        const bool ok = l >= 0 && l < K;
        // lanes holding the same label as this one: one ballot per label bit
        unsigned long long same = __ballot(ok);
        for (int bit = 0; bit < nbits; ++bit) {
            const unsigned long long bal = __ballot((l >> bit) & 1);
            same &= ((l >> bit) & 1) ? bal : ~bal;
        }
        if (ok) {
            const int rank = __popcll(same & lt);
            const int start = cur[l];
            perm[offsets[l] + start + rank] = int32_t(r);
            // the lowest lane of the group advances the cursor; every lane of the group has read it
            if (rank == 0) cur[l] = start + __popcll(same);
        }
    }
}

__device__ __forceinline__ int srt_find_cluster(const int32_t* __restrict__ chunk_start, int K, int chunk) {
    int lo = 0, hi = K;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (chunk_start[mid] <= chunk) lo = mid;
        else hi = mid;
    }
    return lo;
}

// offsets / chunk_start from the counts (one workgroup)
__global__ __launch_bounds__(1024) void srt_scan_clusters_kernel(const int64_t* __restrict__ counts, int K,
                                                                 int64_t* __restrict__ offsets,
                                                                 int32_t* __restrict__ chunk_start) {
    __shared__ long long so[1024];
    __shared__ int sc[1024];
    const int tid = threadIdx.x;
    const int per = (K + 1023) / 1024;
    const int k0 = tid * per, k1 = min(K, k0 + per);
    long long o = 0;
    int c = 0;
    for (int k = k0; k < k1; ++k) {
        o += counts[k];
        c += int((counts[k] + SRT_R - 1) / SRT_R);
    }
    so[tid] = o;
    sc[tid] = c;
    __syncthreads();
    if (tid == 0) {
        long long ro = 0;
        int rc = 0;
        for (int t = 0; t < 1024; ++t) {
            const long long vo = so[t];
            const int vc = sc[t];
            so[t] = ro;
            sc[t] = rc;
            ro += vo;
            rc += vc;
        }
        offsets[K] = ro;
        chunk_start[K] = rc;
    }
    __syncthreads();
    o = so[tid];
    c = sc[tid];
    for (int k = k0; k < k1; ++k) {
        offsets[k] = o;
        chunk_start[k] = c;
        o += counts[k];
        c += int((counts[k] + SRT_R - 1) / SRT_R);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void srt_segsum_kernel(const T* __restrict__ X, int64_t ldx, int D,
                                                         const int32_t* __restrict__ perm,
                                                         const int64_t* __restrict__ offsets,
                                                         const int32_t* __restrict__ chunk_start, int K,
                                                         double* __restrict__ part, int DPAD) {
    __shared__ double red[8][33];  // fp64 inside a chunk: the pass is bound by its loads, and 256 fp32
                                    // additions per lane would cost two decimal digits of the mean
    const int chunk = blockIdx.x;
    if (chunk >= chunk_start[K]) return;
    const int k = srt_find_cluster(chunk_start, K, chunk);
    const int64_t r0 = offsets[k] + int64_t(chunk - chunk_start[k]) * SRT_R;
    const int64_t r1 = min(offsets[k + 1], r0 + SRT_R);
    const int col = threadIdx.x & 31, rl = threadIdx.x >> 5;
    const int d = blockIdx.y * 32 + col;
    const bool ok = d < D;
    const T* xc = X + (ok ? d : 0);
    constexpr int U = 8;
    double acc = 0.0;
    int64_t r = r0 + rl;
    for (; r + 8 * (U - 1) < r1; r += 8 * U) {
        T v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = xc[int64_t(perm[r + 8 * u]) * ldx];
#pragma unroll
        for (int u = 0; u < U; ++u) acc += double(v[u]);
    }
    for (; r < r1; r += 8) acc += double(xc[int64_t(perm[r]) * ldx]);
    red[rl][col] = ok ? acc : 0.0;
    __syncthreads();
    if (rl == 0) {
        double s = red[0][col];
#pragma unroll
        for (int q = 1; q < 8; ++q) s += red[q][col];
        part[int64_t(chunk) * DPAD + blockIdx.y * 32 + col] = s;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void srt_finalize_kernel(const double* __restrict__ part, int DPAD,
                                                           const int32_t* __restrict__ chunk_start,
                                                           const int64_t* __restrict__ cnts, int K, int D,
                                                           T* __restrict__ C_new, int64_t ldcn,
                                                           int64_t* __restrict__ counts_out,
                                                           const T* __restrict__ C_old,
                                                           double* __restrict__ shift_part) {
    __shared__ double ssq[256];
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    const bool ok = i < int64_t(K) * D;
    double sq = 0.0;
    if (ok) {
        const int k = int(i / D), d = int(i - int64_t(k) * D);
        double sum = 0.0;
        for (int c = chunk_start[k]; c < chunk_start[k + 1]; ++c) sum += part[int64_t(c) * DPAD + d];
        const int64_t n = cnts[k];
        const double cnt = double(float(n < 1 ? 1 : n));
        const T cnew = T(sum / cnt);
        C_new[int64_t(k) * ldcn + d] = cnew;
        if (d == 0 && counts_out) counts_out[k] = n;
        if (C_old) {
            const T df = C_old[int64_t(k) * D + d] - cnew;
            sq = double(df * df);
        }
    }
    if (C_old) {
        ssq[threadIdx.x] = sq;
        __syncthreads();
        if (threadIdx.x == 0) {
            double t = 0.0;
            for (int q = 0; q < 256; ++q) t += ssq[q];
            shift_part[blockIdx.x] = t;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void srt_shift_final_kernel(const double* __restrict__ part, int nb,
                                                              T* __restrict__ out) {
    __shared__ double sh[256];
    const int per = (nb + 255) / 256;
    double acc = 0.0;
    const int b0 = threadIdx.x * per, b1 = min(nb, b0 + per);
    for (int i = b0; i < b1; ++i) acc += part[i];
    sh[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < 256; ++i) t += sh[i];
        *out = T(t);
    }
}

SortedWorkspace carve_sorted(void* base, int64_t N, int32_t D, int32_t K, int32_t elem) {
    SortedWorkspace w;
    memset(&w, 0, sizeof(w));
    char* p = static_cast<char*>(base);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* r = p ? p + off : nullptr;
        off += align_up(bytes, 256);
        return r;
    };
    const int64_t blk_rows = sorted_block_rows(N);
    const int64_t nblk = N > 0 ? (N + blk_rows - 1) / blk_rows : 1;
    const int64_t max_chunks = N / SRT_R + K;
    const int dpad = (D + 31) / 32 * 32;
    w.blk_cnt = reinterpret_cast<int32_t*>(take(size_t(nblk) * K * sizeof(int32_t)));
    w.counts = reinterpret_cast<int64_t*>(take(size_t(K) * sizeof(int64_t)));
    w.offsets = reinterpret_cast<int64_t*>(take((size_t(K) + 1) * sizeof(int64_t)));
    w.chunk_start = reinterpret_cast<int32_t*>(take((size_t(K) + 1) * sizeof(int32_t)));
    w.perm = reinterpret_cast<int32_t*>(take(size_t(N < 1 ? 1 : N) * sizeof(int32_t)));
    w.part = take(size_t(max_chunks) * dpad * sizeof(double));  // chunk sums stay in fp64 until the division
    w.shift_part = reinterpret_cast<double*>(take((size_t(K) * D / 256 + 1) * sizeof(double)));
    w.total = off;
    return w;
}

template <typename T>
static int launch_update_sorted_t(const T* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                                  int32_t K, T* C_new, int64_t ldcn, int64_t* counts,
                                  const SortedWorkspace& w, const T* C_old, T* shift, hipStream_t st) {
    int rc;
    const int64_t blk_rows = sorted_block_rows(N);
    const int nblk = N > 0 ? int((N + blk_rows - 1) / blk_rows) : 1;
    const unsigned gblocks = unsigned((nblk + 3) / 4);
    const size_t glds = size_t(4) * K * sizeof(int);
    int nbits = 0;
    while ((1 << nbits) < K) ++nbits;
    hipLaunchKernelGGL(srt_count_kernel, dim3(gblocks), dim3(256), glds, st, labels, N, K, blk_rows, nblk,
                       w.blk_cnt);
    if ((rc = check_launch("srt_count_kernel"))) return rc;
    hipLaunchKernelGGL(srt_scan_blocks_kernel, dim3(K), dim3(256), 0, st, w.blk_cnt, nblk, K, w.counts);
    if ((rc = check_launch("srt_scan_blocks_kernel"))) return rc;
    hipLaunchKernelGGL(srt_scan_clusters_kernel, dim3(1), dim3(1024), 0, st, w.counts, K, w.offsets,
                       w.chunk_start);
    if ((rc = check_launch("srt_scan_clusters_kernel"))) return rc;
    const int dpad = (D + 31) / 32 * 32;
    double* part = reinterpret_cast<double*>(w.part);
    if (N > 0) {
        hipLaunchKernelGGL(srt_scatter_kernel, dim3(gblocks), dim3(256), glds, st, labels, N, K, nbits, blk_rows,
                           nblk, w.blk_cnt, w.offsets, w.perm);
        if ((rc = check_launch("srt_scatter_kernel"))) return rc;
        const int64_t max_chunks = N / SRT_R + K;
        hipLaunchKernelGGL(srt_segsum_kernel<T>, dim3((unsigned)max_chunks, (D + 31) / 32), dim3(256), 0, st, X, ldx,
                           D, w.perm, w.offsets, w.chunk_start, K, part, dpad);
        if ((rc = check_launch("srt_segsum_kernel"))) return rc;
    }
    const int nb = int((int64_t(K) * D + 255) / 256);
    hipLaunchKernelGGL(srt_finalize_kernel<T>, dim3(nb), dim3(256), 0, st, static_cast<const double*>(part), dpad,
                       w.chunk_start, w.counts, K, D, C_new, ldcn, counts, C_old, w.shift_part);
    if ((rc = check_launch("srt_finalize_kernel")) || !C_old) return rc;
    hipLaunchKernelGGL(srt_shift_final_kernel<T>, dim3(1), dim3(256), 0, st,
                       static_cast<const double*>(w.shift_part), nb, shift);
    return check_launch("srt_shift_final_kernel");
}

int launch_update_sorted(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels, int32_t K,
                         float* C_new, int64_t ldcn, int64_t* counts, const SortedWorkspace& w,
                         const float* C_old, float* shift, hipStream_t st) {
    return launch_update_sorted_t<float>(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, C_old, shift, st);
}

int launch_update_sorted_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                             int32_t K, double* C_new, int64_t ldcn, int64_t* counts,
                             const SortedWorkspace& w, const double* C_old, double* shift, hipStream_t st) {
    return launch_update_sorted_t<double>(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, C_old, shift, st);
}

}  // namespace hkm
