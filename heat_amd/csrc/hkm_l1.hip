// Manhattan-metric kernels for the k-medians / k-medoids estimators (heat/cluster/kmedians.py,
// heat/cluster/kmedoids.py, heat/cluster/batchparallelclustering.py with p = 1):
//
//   * l1_argmin_kernel: fused sum|q - r| + argmin.  For every row of Q the closest row of R, the
//     M x Nn matrix is never written.  A workgroup owns 64 rows of Q and walks R in tiles of 64 rows
//     (4 x 4 register block per lane, both tiles staged through LDS in chunks of 16 features).  Used
//     as the assignment (Q = points, R = centroids) and, with R split over many workgroups and a
//     64-bit atomic-min merge of (distance bits, index) keys, to snap a median to the closest data
//     row (Q = medians, R = points).  There is no matrix-core form of an L1 distance: the bound is
//     the vector ALU, 2 operations per (row, row, feature).
//   * per-cluster median of every coordinate by radix selection: the rows are grouped by cluster
//     with a counting sort (the order inside a cluster is irrelevant to an order statistic), then
//     four passes build 256-bin histograms of one byte of the order-preserving integer image of the
//     values -- in LDS per chunk of one cluster's rows, merged with integer atomics -- and narrow the
//     candidate range of every (cluster, coordinate) down to the value of rank (n-1)/2.  For an even
//     count one more pass finds the next larger value.  Integer work throughout: bit-reproducible.
#include "hkm_common.h"

namespace hkm {

// ------------------------------------------------------------------------------------------------
// fused L1 distance + argmin
// ------------------------------------------------------------------------------------------------
static constexpr int L1_T = 64;
static constexpr int L1_KC = 16;
static constexpr int CLOSEST64_ITEMS = 4096;  // (query tile, row split) workgroups of the float64 snap

template <typename T>
__device__ __forceinline__ void l1_better(T& bd, unsigned& bi, T d, unsigned i) {
    if (d < bd || (d == bd && i < bi)) {
        bd = d;
        bi = i;
    }
}
__device__ __forceinline__ float l1_abs(float v) { return fabsf(v); }
__device__ __forceinline__ double l1_abs(double v) { return fabs(v); }

// T = float: everything in fp32.  T = double: the rows of Q are float64 and every distance is summed in
// float64 from the float32 rows of R widened on the way into LDS -- the medoid snap of the reference,
// which measures float64 distances to the float64 median (heat/cluster/kmedoids.py:91-106): two rows at
// exactly the same distance (the two members of a cluster on either side of their midpoint, the two
// middle values of a one-dimensional cluster) must come out EQUAL so that the first one wins, and in
// fp32 against a rounded median they come out one rounding error apart in either direction.  The
// float64 variant writes the best (distance, row) of every split to part_d / part_i; the splits are
// merged in row order by l1_merge_splits_kernel.
template <typename T>
__global__ __launch_bounds__(256) void l1_argmin_kernel(
    const T* __restrict__ Q, int64_t M, int64_t ldq, const float* __restrict__ R, int64_t Nn,
    int64_t ldr, int D, int64_t rows_per_split, int32_t* __restrict__ labels,
    float* __restrict__ min_dist, unsigned long long* __restrict__ keys, double* __restrict__ part_d,
    unsigned* __restrict__ part_i) {
    constexpr bool F64 = sizeof(T) == 8;
    __shared__ T sQ[L1_KC][L1_T + 4];
    __shared__ T sR[L1_KC][L1_T + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int lk = tid & 15, lr = tid >> 4;
    const int64_t i0 = int64_t(blockIdx.x) * L1_T;
    const int64_t r_begin = int64_t(blockIdx.y) * rows_per_split;
    const int64_t r_end = min(Nn, r_begin + rows_per_split);

    T bd[4];
    unsigned bi[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        bd[a] = T(HKM_INF);
        bi[a] = 0xffffffffu;
    }

    for (int64_t j0 = r_begin; j0 < r_end; j0 += L1_T) {
        T acc[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[a][b] = T(0);
        for (int d0 = 0; d0 < D; d0 += L1_KC) {
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int r = lr + 16 * q;
                const int d = d0 + lk;
                const int64_t gi = i0 + r, gj = j0 + r;
                sQ[lk][r] = (gi < M && d < D) ? Q[gi * ldq + d] : T(0);
                sR[lk][r] = (gj < r_end && d < D) ? T(R[gj * ldr + d]) : T(0);
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < L1_KC; ++k) {
                T qa[4], rb[4];
#pragma unroll
                for (int a = 0; a < 4; ++a) qa[a] = sQ[k][ty * 4 + a];
#pragma unroll
                for (int b = 0; b < 4; ++b) rb[b] = sR[k][tx * 4 + b];
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int b = 0; b < 4; ++b) acc[a][b] += l1_abs(qa[a] - rb[b]);
            }
        }
        // this lane's four candidates per row in ascending index order, then the 16 lanes that hold
        // the other columns of the same rows
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            T d = T(HKM_INF);
            unsigned i = 0xffffffffu;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int64_t gj = j0 + tx * 4 + b;
                if (gj < r_end) l1_better<T>(d, i, acc[a][b], unsigned(gj));
            }
#pragma unroll
            for (int w = 1; w < 16; w <<= 1) {
                const T od = __shfl_xor(d, w);
                const unsigned oi = unsigned(__shfl_xor(int(i), w));
                l1_better<T>(d, i, od, oi);
            }
            l1_better<T>(bd[a], bi[a], d, i);
        }
    }

    if (tx == 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t gi = i0 + ty * 4 + a;
            if (gi >= M) continue;
            if (F64) {
                part_d[int64_t(blockIdx.y) * M + gi] = double(bd[a]);
                part_i[int64_t(blockIdx.y) * M + gi] = bi[a];
            } else if (keys) {
                // distances are >= 0, so their bit patterns order like the values; a row whose
                // distances were all NaN keeps the initial key
                if (bi[a] != 0xffffffffu)
                    atomicMin(&keys[gi], (unsigned long long)(__float_as_uint(float(bd[a]))) << 32 | bi[a]);
            } else {
                labels[gi] = bi[a] == 0xffffffffu ? 0 : int32_t(bi[a]);
                if (min_dist) min_dist[gi] = float(bd[a]);
            }
        }
    }
}

__global__ void l1_fill_keys_kernel(unsigned long long* __restrict__ keys, int64_t n) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) keys[i] = ~0ull;
}

__global__ void l1_unpack_rows_kernel(const unsigned long long* __restrict__ keys, int64_t n,
                                      int64_t* __restrict__ idx, float* __restrict__ dist) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const unsigned long long k = keys[i];
    idx[i] = (k >> 32) == 0xffffffffull ? 0 : int64_t(unsigned(k));
    if (dist) dist[i] = __uint_as_float(unsigned(k >> 32));
}

// Narrow rows (D <= 16): one point per lane in registers, the centroids in LDS read as wave-wide
// broadcasts, k ascending with a strict '<' so the first index wins ties.  Bound by streaming X.
static constexpr int L1S_THREADS = 256;
static constexpr int L1S_LDS_FLOATS = 8192;

template <int D>
__global__ __launch_bounds__(L1S_THREADS) void l1_assign_small_kernel(
    const float* __restrict__ X, int64_t N, int64_t ldx, const float* __restrict__ C, int K, int64_t ldc,
    int32_t* __restrict__ labels, float* __restrict__ min_dist, int ktile, int64_t nbatches) {
    __shared__ float sC[L1S_LDS_FLOATS];
    const int tid = threadIdx.x;
    const int nkt = (K + ktile - 1) / ktile;
    auto stage = [&](int kt) {
        const int k0 = kt * ktile;
        const int kn = min(ktile, K - k0);
        for (int i = tid; i < kn * D; i += L1S_THREADS) {
            const int r = i / D, c = i - r * D;
            sC[i] = C[int64_t(k0 + r) * ldc + c];
        }
        __syncthreads();
        return kn;
    };
    int kn = 0;
    if (nkt == 1) kn = stage(0);
    for (int64_t b = blockIdx.x; b < nbatches; b += gridDim.x) {
        const int64_t i = b * L1S_THREADS + tid;
        const int64_t ir = i < N ? i : N - 1;
        float x[D];
        const float* xp = X + ir * ldx;
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = xp[d];
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
                const float* c = sC + k * D;
                float dist = fabsf(x[0] - c[0]);
#pragma unroll
                for (int d = 1; d < D; ++d) dist += fabsf(x[d] - c[d]);
                if (dist < m) {
                    m = dist;
                    mi = k0 + k;
                }
            }
        }
        if (i < N) {
            labels[i] = mi;
            if (min_dist) min_dist[i] = m;
        }
    }
}

template <int D>
static int launch_l1_small_t(const float* X, int64_t N, int64_t ldx, const float* C, int32_t K, int64_t ldc,
                             int32_t* labels, float* min_dist, hipStream_t st) {
    const int ktile = L1S_LDS_FLOATS / D;
    const int64_t nbatches = (N + L1S_THREADS - 1) / L1S_THREADS;
    int64_t grid = int64_t(num_cus()) * 8;
    if (grid > nbatches) grid = nbatches;
    hipLaunchKernelGGL(l1_assign_small_kernel<D>, dim3((unsigned)grid), dim3(L1S_THREADS), 0, st, X, N, ldx, C, K,
                       ldc, labels, min_dist, ktile, nbatches);
    return check_launch("l1_assign_small_kernel");
}

int launch_assign_l1(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                     int64_t ldc, int32_t* labels, float* min_dist, hipStream_t st) {
    // narrow rows and few centroids: the 64 x 64 tile would be mostly padding
    if (D <= 16 && int64_t(K) * D <= 1024) {
#define HKM_CASE(d) \
    case d:         \
        return launch_l1_small_t<d>(X, N, ldx, C, K, ldc, labels, min_dist, st);
        switch (D) {
            HKM_CASE(1) HKM_CASE(2) HKM_CASE(3) HKM_CASE(4) HKM_CASE(5) HKM_CASE(6) HKM_CASE(7) HKM_CASE(8)
            HKM_CASE(9) HKM_CASE(10) HKM_CASE(11) HKM_CASE(12) HKM_CASE(13) HKM_CASE(14) HKM_CASE(15) HKM_CASE(16)
        }
#undef HKM_CASE
    }
    const int64_t tiles = (N + L1_T - 1) / L1_T;
    if (tiles > 0x7fffffffLL) return fail(HKM_EUNSUPPORTED, "assign_l1: too many row tiles");
    hipLaunchKernelGGL(l1_argmin_kernel<float>, dim3((unsigned)tiles, 1), dim3(256), 0, st, X, N, ldx, C,
                       int64_t(K), ldc, D, int64_t(K), labels, min_dist,
                       static_cast<unsigned long long*>(nullptr), static_cast<double*>(nullptr),
                       static_cast<unsigned*>(nullptr));
    return check_launch("l1_argmin_kernel");
}

int launch_closest_rows_l1(const float* X, int64_t N, int32_t D, int64_t ldx, const float* Qm,
                           int32_t M, int64_t ldq, int64_t* idx, float* dist,
                           unsigned long long* keys, hipStream_t st) {
    hipLaunchKernelGGL(l1_fill_keys_kernel, dim3((M + 255) / 256), dim3(256), 0, st, keys, int64_t(M));
    int rc = check_launch("l1_fill_keys_kernel");
    if (rc) return rc;
    const int64_t qtiles = (int64_t(M) + L1_T - 1) / L1_T;
    // enough splits of the data rows to fill the device, each a multiple of the tile height
    int64_t want = (int64_t(num_cus()) * 8 + qtiles - 1) / qtiles;
    int64_t rps = (N + want - 1) / want;
    rps = (rps + L1_T - 1) / L1_T * L1_T;
    if (rps < 4 * L1_T) rps = 4 * L1_T;
    const int64_t nsplit = (N + rps - 1) / rps;
    if (nsplit > 65535) return fail(HKM_EUNSUPPORTED, "closest_rows_l1: too many splits");
    if (N > 0)
        hipLaunchKernelGGL(l1_argmin_kernel<float>, dim3((unsigned)qtiles, (unsigned)nsplit), dim3(256), 0, st, Qm,
                           int64_t(M), ldq, X, N, ldx, D, rps, static_cast<int32_t*>(nullptr),
                           static_cast<float*>(nullptr), keys, static_cast<double*>(nullptr),
                           static_cast<unsigned*>(nullptr));
    if ((rc = check_launch("l1_argmin_kernel"))) return rc;
    hipLaunchKernelGGL(l1_unpack_rows_kernel, dim3((M + 255) / 256), dim3(256), 0, st, keys, int64_t(M), idx,
                       dist);
    return check_launch("l1_unpack_rows_kernel");
}

// best (distance, row) of every query over the splits, in split order = ascending row order: on equal
// distances the first row wins
__global__ void l1_merge_splits_kernel(const double* __restrict__ part_d, const unsigned* __restrict__ part_i,
                                       int nsplit, int64_t M, int64_t* __restrict__ idx,
                                       double* __restrict__ dist) {
    const int64_t q = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (q >= M) return;
    double bd = double(HKM_INF);
    unsigned bi = 0xffffffffu;
    for (int s = 0; s < nsplit; ++s) l1_better<double>(bd, bi, part_d[int64_t(s) * M + q], part_i[int64_t(s) * M + q]);
    idx[q] = bi == 0xffffffffu ? 0 : int64_t(bi);
    if (dist) dist[q] = bd;
}

// slots of part_d / part_i: the splits are chosen so that nsplit * qtiles <= CLOSEST64_ITEMS
int64_t closest64_slots(int32_t M) { return int64_t(CLOSEST64_ITEMS) * L1_T + M; }

int launch_closest_rows_l1_q64(const float* X, int64_t N, int32_t D, int64_t ldx, const double* Qm, int32_t M,
                               int64_t* idx, double* dist, double* part_d, unsigned* part_i, hipStream_t st) {
    const int64_t qtiles = (int64_t(M) + L1_T - 1) / L1_T;
    int64_t want = CLOSEST64_ITEMS / qtiles;
    if (want < 1) want = 1;
    int64_t rps = (N + want - 1) / want;
    rps = (rps + L1_T - 1) / L1_T * L1_T;
    if (rps < 4 * L1_T) rps = 4 * L1_T;
    const int64_t nsplit = (N + rps - 1) / rps;
    hipLaunchKernelGGL(l1_argmin_kernel<double>, dim3((unsigned)qtiles, (unsigned)nsplit), dim3(256), 0, st, Qm,
                       int64_t(M), int64_t(D), X, N, ldx, D, rps, static_cast<int32_t*>(nullptr),
                       static_cast<float*>(nullptr), static_cast<unsigned long long*>(nullptr), part_d, part_i);
    int rc = check_launch("l1_argmin_kernel<double>");
    if (rc) return rc;
    hipLaunchKernelGGL(l1_merge_splits_kernel, dim3((M + 255) / 256), dim3(256), 0, st, part_d, part_i, int(nsplit),
                       int64_t(M), idx, dist);
    return check_launch("l1_merge_splits_kernel");
}

// ------------------------------------------------------------------------------------------------
// per-cluster medians by radix selection
// ------------------------------------------------------------------------------------------------
static constexpr int MED_R = 4096;       // rows of one cluster per workgroup and pass
static constexpr int MED_SORT_K = 4096;  // clusters whose cursors fit in LDS during the grouping

__device__ __forceinline__ unsigned to_key(float v) {
    const unsigned b = __float_as_uint(v);
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float from_key(unsigned k) {
    return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu));
}

// eff[i] = labels[i] if the row takes part in the medians, else -1.  With skip_zero a row whose
// entries are all zero is left out, as the reference drops the rows of `x * selection` that sum to
// zero in absolute value (heat/cluster/kmedians.py:93-96).
// LPR lanes share a row (a power of two <= 32, about the feature count: no idle lanes on narrow data).
// VEC: rows are read in 16-byte groups (X 16-byte aligned, ldx % 4 == 0, D % 4 == 0; LPR then counts
// lanes per row of D / 4 groups).
template <int LPR, bool VEC>
__global__ __launch_bounds__(256) void med_eff_label_kernel(const float* __restrict__ X, int64_t N,
                                                            int D, int64_t ldx,
                                                            const int32_t* __restrict__ labels, int K,
                                                            int32_t* __restrict__ eff) {
    constexpr int RPG = 8;  // rows per lane group: that many independent loads in flight per lane
    const int sub = threadIdx.x & (LPR - 1);
    const int64_t row0 = ((int64_t(blockIdx.x) * 256 + threadIdx.x) / LPR) * RPG;
    int nz[RPG];
#pragma unroll
    for (int u = 0; u < RPG; ++u) nz[u] = 0;
    if (VEC) {
        const int ng = D >> 2;
        for (int g = sub; g < ng; g += LPR) {
            float4 v[RPG];
#pragma unroll
            for (int u = 0; u < RPG; ++u)
                v[u] = row0 + u < N ? *reinterpret_cast<const float4*>(X + (row0 + u) * ldx + 4 * g)
                                    : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int u = 0; u < RPG; ++u)
                nz[u] |= (v[u].x != 0.f) | (v[u].y != 0.f) | (v[u].z != 0.f) | (v[u].w != 0.f);
        }
    } else {
        for (int d = sub; d < D; d += LPR) {
            float v[RPG];
#pragma unroll
            for (int u = 0; u < RPG; ++u) v[u] = row0 + u < N ? X[(row0 + u) * ldx + d] : 0.f;
#pragma unroll
            for (int u = 0; u < RPG; ++u) nz[u] |= (v[u] != 0.f);
        }
    }
#pragma unroll
    for (int u = 0; u < RPG; ++u) {
#pragma unroll
        for (int w = 1; w < LPR; w <<= 1) nz[u] |= __shfl_xor(nz[u], w);
    }
    // lane u of the group stores row u
#pragma unroll
    for (int u = 0; u < RPG; ++u) {
        if ((LPR >= RPG ? sub == u : sub == 0) && row0 + u < N) {
            const int l = labels[row0 + u];
            eff[row0 + u] = (l >= 0 && l < K && nz[u]) ? l : -1;
        }
    }
}

// offsets[k] = rows of clusters < k, chunk_start[k] = chunks of clusters < k (one workgroup)
__global__ __launch_bounds__(1024) void med_scan_kernel(const int64_t* __restrict__ counts, int K,
                                                        int64_t* __restrict__ offsets,
                                                        int32_t* __restrict__ chunk_start,
                                                        int32_t* __restrict__ cursor) {
    __shared__ long long so[1024];
    __shared__ int sc[1024];
    const int tid = threadIdx.x;
    const int per = (K + 1023) / 1024;
    const int k0 = tid * per, k1 = min(K, k0 + per);
    long long o = 0;
    int c = 0;
    for (int k = k0; k < k1; ++k) {
        o += counts[k];
        c += int((counts[k] + MED_R - 1) / MED_R);
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
        cursor[k] = 0;
        o += counts[k];
        c += int((counts[k] + MED_R - 1) / MED_R);
    }
}

// perm[offsets[k] + j] = the rows of cluster k in some order.  A workgroup ranks its rows per cluster
// in LDS and reserves a range per cluster with one global atomic.
__global__ __launch_bounds__(256) void med_group_kernel(const int32_t* __restrict__ eff, int64_t N,
                                                        int K, const int64_t* __restrict__ offsets,
                                                        int32_t* __restrict__ cursor,
                                                        int32_t* __restrict__ perm) {
    constexpr int PER = 8;
    extern __shared__ int lcnt[];  // [K] when K <= MED_SORT_K
    const bool lds = K <= MED_SORT_K;
    const int64_t base = int64_t(blockIdx.x) * (256 * PER);
    int lab[PER], pos[PER];
    if (lds) {
        for (int k = threadIdx.x; k < K; k += 256) lcnt[k] = 0;
        __syncthreads();
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int64_t i = base + u * 256 + threadIdx.x;
        lab[u] = i < N ? eff[i] : -1;
        pos[u] = 0;
        if (lab[u] >= 0) pos[u] = lds ? atomicAdd(&lcnt[lab[u]], 1) : atomicAdd(&cursor[lab[u]], 1);
    }
    if (lds) {
        __syncthreads();
        for (int k = threadIdx.x; k < K; k += 256) {
            const int c = lcnt[k];
            lcnt[k] = c ? atomicAdd(&cursor[k], c) : 0;
        }
        __syncthreads();
    }
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        if (lab[u] < 0) continue;
        const int64_t i = base + u * 256 + threadIdx.x;
        perm[offsets[lab[u]] + (lds ? lcnt[lab[u]] : 0) + pos[u]] = int32_t(i);
    }
}

__global__ void med_zero_kernel(unsigned* __restrict__ p, int64_t n) {
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += int64_t(gridDim.x) * blockDim.x)
        p[i] = 0;
}

__device__ __forceinline__ int med_find_cluster(const int32_t* __restrict__ chunk_start, int K, int chunk) {
    int lo = 0, hi = K;  // largest k with chunk_start[k] <= chunk
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (chunk_start[mid] <= chunk) lo = mid;
        else hi = mid;
    }
    return lo;
}

// state per (cluster, coordinate): prefix = the leading bytes of the key found so far.
// MODE 0: histogram of byte `pass` (0 = most significant) of the keys that match the prefix.
// MODE 1: minimum key larger than prefix (the complete key of the lower median).
// A workgroup handles up to MED_R rows of ONE cluster and a slice of `cols` = 2^cl coordinates
// (32, or the next power of two >= D for narrow data, so that no lane idles): 256 / cols rows per
// step.  Consecutive rows of a lane that fall into the same bin are counted in a register and added
// with one LDS atomic per run -- in the first pass nearly every value of a coordinate shares its
// leading byte.
template <int MODE>
__global__ __launch_bounds__(256) void med_pass_kernel(const float* __restrict__ X, int64_t ldx, int D,
                                                       const int32_t* __restrict__ perm,
                                                       const int64_t* __restrict__ offsets,
                                                       const int32_t* __restrict__ chunk_start, int K,
                                                       int pass, int cl,
                                                       const unsigned* __restrict__ prefix,
                                                       unsigned* __restrict__ hist_g,
                                                       unsigned* __restrict__ next_g) {
    __shared__ unsigned lh[32][257];
    __shared__ unsigned lmin[32];
    const int chunk = blockIdx.x;
    if (chunk >= chunk_start[K]) return;
    const int k = med_find_cluster(chunk_start, K, chunk);
    const int64_t r0 = offsets[k] + int64_t(chunk - chunk_start[k]) * MED_R;
    const int64_t r1 = min(offsets[k + 1], r0 + MED_R);
    const int cols = 1 << cl;
    const int col = threadIdx.x & (cols - 1), rl = threadIdx.x >> cl, rstep = 256 >> cl;
    const int d = blockIdx.y * cols + col;
    const bool ok = d < D;
    if (MODE == 0) {
        for (int i = threadIdx.x; i < 32 * 257; i += 256) (&lh[0][0])[i] = 0;
    } else if (threadIdx.x < 32) {
        lmin[threadIdx.x] = 0xffffffffu;
    }
    __syncthreads();
    const unsigned pf = ok ? prefix[int64_t(k) * D + d] : 0;
    const int shift = 24 - 8 * pass;
    unsigned best = 0xffffffffu;
    int run_bin = -1;
    unsigned run_len = 0;
    if (ok) {
        // eight rows in flight per lane: the gather is latency-bound otherwise
        constexpr int UF = 8;
        int64_t r = r0 + rl;
        auto consume = [&](unsigned key) {
            if (MODE == 0) {
                // bytes above `shift + 8` must equal the prefix (nothing to compare in the first pass)
                const bool match = pass == 0 || (key >> (shift + 8)) == pf;
                if (match) {
                    const int bin = int((key >> shift) & 255u);
                    if (bin == run_bin) {
                        ++run_len;
                    } else {
                        if (run_len) atomicAdd(&lh[col][run_bin], run_len);
                        run_bin = bin;
                        run_len = 1;
                    }
                }
            } else if (key > pf) {
                best = min(best, key);
            }
        };
        for (; r + int64_t(UF - 1) * rstep < r1; r += int64_t(UF) * rstep) {
            int row[UF];
            float v[UF];
#pragma unroll
            for (int u = 0; u < UF; ++u) row[u] = perm[r + int64_t(u) * rstep];
#pragma unroll
            for (int u = 0; u < UF; ++u) v[u] = X[int64_t(row[u]) * ldx + d];
#pragma unroll
            for (int u = 0; u < UF; ++u) consume(to_key(v[u]));
        }
        for (; r < r1; r += rstep) consume(to_key(X[int64_t(perm[r]) * ldx + d]));
        if (MODE == 0 && run_len) atomicAdd(&lh[col][run_bin], run_len);
        if (MODE == 1 && best != 0xffffffffu) atomicMin(&lmin[col], best);
    }
    __syncthreads();
    if (MODE == 0) {
        for (int i = threadIdx.x; i < cols * 256; i += 256) {
            const int c = i >> 8, b = i & 255;
            const unsigned v = lh[c][b];
            const int dd = blockIdx.y * cols + c;
            if (v && dd < D) atomicAdd(&hist_g[(int64_t(k) * D + dd) * 256 + b], v);
        }
    } else if (threadIdx.x < cols) {
        const int dd = blockIdx.y * cols + threadIdx.x;
        if (dd < D && lmin[threadIdx.x] != 0xffffffffu)
            atomicMin(&next_g[int64_t(k) * D + dd], lmin[threadIdx.x]);
    }
}

// one wave per (cluster, coordinate): find the bin that holds the wanted rank (each lane owns four
// consecutive bins, an exclusive scan over the lanes gives their first rank), extend the prefix by
// that byte, make the rank relative to the bin, and clear the bins
__global__ __launch_bounds__(256) void med_pick_kernel(unsigned* __restrict__ hist_g, int64_t KD, int D,
                                                       const int64_t* __restrict__ counts, int pass,
                                                       unsigned* __restrict__ prefix,
                                                       int64_t* __restrict__ rank,
                                                       unsigned* __restrict__ eqcnt,
                                                       unsigned* __restrict__ next_g) {
    const int lane = threadIdx.x & 63;
    const int64_t i = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (i >= KD) return;  // whole waves leave together
    const int64_t n = counts[i / D];
    uint4* h4 = reinterpret_cast<uint4*>(hist_g + i * 256) + lane;
    const uint4 c = *h4;
    *h4 = make_uint4(0u, 0u, 0u, 0u);
    int64_t want = pass == 0 ? (n > 0 ? (n - 1) / 2 : 0) : rank[i];
    const unsigned pf = pass == 0 ? 0u : prefix[i];
    // exclusive scan of the lanes' totals (bins are 32-bit counts of at most 2^31 rows)
    const unsigned tot = c.x + c.y + c.z + c.w;
    unsigned incl = tot;
#pragma unroll
    for (int w = 1; w < 64; w <<= 1) {
        const unsigned o = __shfl_up(incl, w);
        if (lane >= w) incl += o;
    }
    const int64_t first = int64_t(incl) - tot;  // rank of this lane's first element
    const unsigned cs[4] = {c.x, c.y, c.z, c.w};
    int digit = -1;
    unsigned in_bin = 0;
    int64_t rel = 0, lo = first;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if (digit < 0 && want >= lo && want < lo + int64_t(cs[q])) {
            digit = 4 * lane + q;
            in_bin = cs[q];
            rel = want - lo;
        }
        lo += cs[q];
    }
    const unsigned long long who = __ballot(digit >= 0);
    if (who == 0) {
        // nothing holds the rank (an empty cluster): digit 0, as a walk over empty bins ends
        if (lane == 0) {
            prefix[i] = pf << 8;
            rank[i] = 0;
            eqcnt[i] = 0;
            if (pass == 0) next_g[i] = 0xffffffffu;
        }
    } else if (digit >= 0) {
        prefix[i] = (pf << 8) | unsigned(digit);
        rank[i] = rel;
        eqcnt[i] = in_bin;
        if (pass == 0) next_g[i] = 0xffffffffu;
    }
}

// mode 0: the reference's median (percentile 50, linear): lower middle for an odd count, for an even
//         count lo + (hi - lo) * 0.5 evaluated in fp64 and rounded to fp32 (heat/core/statistics.py
//         percentile on the fp64 `x * selection`);  mode 1: the lower middle (torch.median).
// An empty cluster takes the data row fallback_rows[k] if given, else keeps C_old[k] if given, else 0.
__global__ __launch_bounds__(256) void med_final_kernel(const unsigned* __restrict__ prefix,
                                                        const int64_t* __restrict__ rank,
                                                        const unsigned* __restrict__ eqcnt,
                                                        const unsigned* __restrict__ next_g,
                                                        const int64_t* __restrict__ counts, int K, int D,
                                                        int mode, const float* __restrict__ X, int64_t ldx,
                                                        int64_t N, const int64_t* __restrict__ fallback_rows,
                                                        const float* __restrict__ C_old,
                                                        float* __restrict__ C_new, int64_t ldcn,
                                                        int64_t* __restrict__ counts_out,
                                                        double* __restrict__ med64) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= int64_t(K) * D) return;
    const int k = int(i / D), d = int(i - int64_t(k) * D);
    const int64_t n = counts[k];
    float v = 0.f;
    double v64 = 0.0;  // the value before it is rounded to fp32 (differs for an even count only)
    bool have64 = false;
    if (n == 0) {
        if (fallback_rows) {
            int64_t r = fallback_rows[k];
            r = r < 0 ? 0 : (r >= N ? N - 1 : r);
            v = N > 0 ? X[r * ldx + d] : 0.f;
        } else if (C_old) {
            v = C_old[int64_t(k) * D + d];
        }
    } else {
        const float lo = from_key(prefix[i]);
        v = lo;
        if (mode == 0 && (n & 1) == 0) {
            // rank of lo inside its run of equal values; the next order statistic is another copy
            // of lo unless lo is the last of the run
            const float hi = (rank[i] + 1 < int64_t(eqcnt[i])) ? lo : from_key(next_g[i]);
            v64 = double(lo) + (double(hi) - double(lo)) * 0.5;
            have64 = true;
            v = float(v64);
        }
    }
    C_new[int64_t(k) * ldcn + d] = v;
    if (med64) med64[i] = have64 ? v64 : double(v);
    if (d == 0 && counts_out) counts_out[k] = n;
}

int launch_update_median(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                         int32_t K, const int64_t* fallback_rows, const float* C_old, float* C_new,
                         int64_t ldcn, int64_t* counts_out, int32_t mode, int32_t skip_zero_rows,
                         const MedianWorkspace& w, hipStream_t st, double* med64) {
    int rc;
    const int32_t* eff = labels;
    if (N > 0 && skip_zero_rows) {
        const bool vec = aligned16(X) && (ldx % 4 == 0) && (D % 4 == 0);
        const int units = vec ? D / 4 : D;  // loads per row
        const int lpr = units <= 2 ? 1 : units <= 6 ? 4 : units <= 12 ? 8 : units <= 24 ? 16 : 32;
        const int64_t blocks = ((N + 7) / 8 * lpr + 255) / 256;  // 8 rows per lane group
        if (blocks > 0x7fffffffLL) return fail(HKM_EUNSUPPORTED, "update_median: N too large");
#define HKM_EFF(L)                                                                                             \
    do {                                                                                                       \
        if (vec)                                                                                               \
            hipLaunchKernelGGL((med_eff_label_kernel<L, true>), dim3((unsigned)blocks), dim3(256), 0, st, X, N, D, \
                               ldx, labels, K, w.eff);                                                         \
        else                                                                                                   \
            hipLaunchKernelGGL((med_eff_label_kernel<L, false>), dim3((unsigned)blocks), dim3(256), 0, st, X, N, D, \
                               ldx, labels, K, w.eff);                                                         \
    } while (0)
        if (lpr == 1) HKM_EFF(1);
        else if (lpr == 4) HKM_EFF(4);
        else if (lpr == 8) HKM_EFF(8);
        else if (lpr == 16) HKM_EFF(16);
        else HKM_EFF(32);
#undef HKM_EFF
        if ((rc = check_launch("med_eff_label_kernel"))) return rc;
        eff = w.eff;
    }
    if ((rc = launch_label_counts(eff, N, K, w.counts, st))) return rc;
    hipLaunchKernelGGL(med_scan_kernel, dim3(1), dim3(1024), 0, st, w.counts, K, w.offsets, w.chunk_start,
                       w.cursor);
    if ((rc = check_launch("med_scan_kernel"))) return rc;
    const int64_t KD = int64_t(K) * D;
    const unsigned kd_blocks = unsigned((KD + 255) / 256);
    if (N > 0) {
        const int64_t gblocks = (N + 2047) / 2048;
        const size_t glds = K <= MED_SORT_K ? size_t(K) * sizeof(int) : 0;
        hipLaunchKernelGGL(med_group_kernel, dim3((unsigned)gblocks), dim3(256), glds, st, eff, N, K,
                           w.offsets, w.cursor, w.perm);
        if ((rc = check_launch("med_group_kernel"))) return rc;
    }
    // sum_k ceil(n_k / R) <= N / R + K chunks; surplus workgroups return at once
    const int64_t max_chunks = N / MED_R + K;
    if (max_chunks > 0x7fffffffLL) return fail(HKM_EUNSUPPORTED, "update_median: too many chunks");
    int cl = 5;
    while (cl > 0 && (1 << (cl - 1)) >= D) --cl;  // 2^cl = min(32, next power of two >= D)
    const unsigned J = unsigned((D + (1 << cl) - 1) >> cl);
    int64_t zblocks = (KD * 256 + 255) / 256;
    if (zblocks > int64_t(num_cus()) * 32) zblocks = int64_t(num_cus()) * 32;
    hipLaunchKernelGGL(med_zero_kernel, dim3((unsigned)zblocks), dim3(256), 0, st, w.hist, KD * 256);
    if ((rc = check_launch("med_zero_kernel"))) return rc;
    for (int pass = 0; pass < 4; ++pass) {
        if (N > 0) {
            hipLaunchKernelGGL(med_pass_kernel<0>, dim3((unsigned)max_chunks, J), dim3(256), 0, st, X, ldx, D,
                               w.perm, w.offsets, w.chunk_start, K, pass, cl, w.prefix, w.hist, w.next);
            if ((rc = check_launch("med_pass_kernel<0>"))) return rc;
        }
        hipLaunchKernelGGL(med_pick_kernel, dim3((unsigned)((KD + 3) / 4)), dim3(256), 0, st, w.hist, KD, D, w.counts, pass,
                           w.prefix, w.rank, w.eqcnt, w.next);
        if ((rc = check_launch("med_pick_kernel"))) return rc;
    }
    if (mode == 0 && N > 0) {
        hipLaunchKernelGGL(med_pass_kernel<1>, dim3((unsigned)max_chunks, J), dim3(256), 0, st, X, ldx, D,
                           w.perm, w.offsets, w.chunk_start, K, 0, cl, w.prefix, w.hist, w.next);
        if ((rc = check_launch("med_pass_kernel<1>"))) return rc;
    }
    hipLaunchKernelGGL(med_final_kernel, dim3(kd_blocks), dim3(256), 0, st, w.prefix, w.rank, w.eqcnt, w.next,
                       w.counts, K, D, mode, X, ldx, N, fallback_rows, C_old, C_new, ldcn, counts_out, med64);
    return check_launch("med_final_kernel");
}

}  // namespace hkm
