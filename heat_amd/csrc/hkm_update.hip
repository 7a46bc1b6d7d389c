// Deterministic per-cluster mean (two passes, no floating-point atomics) and the scalar
// reductions of the Lloyd loop.
//
// Pass 1 (update_partial_kernel): workgroup (s, j, z) owns row chunk s, the 32-column slice j of the
// features and the cluster range z.  It keeps an fp32 accumulator acc[KR][32] in LDS.  Each of its 8
// half-waves OWNS the clusters k with k % 8 == q and is the only one that ever touches their
// accumulator rows; it visits the rows of the chunk in ascending order.  Every accumulator element
// therefore has exactly one writer with a fixed order of additions.
// Pass 2 (update_finalize_kernel): four threads per (k, d) add the chunk partials in a fixed strided
// order in fp64; the result is divided by the count and rounded to fp32.
//
// Arithmetic follows heat/cluster/kmeans.py:88-101: mean in float64 (types.py:945-959 promotes
// x * selection), count clipped to >= 1 and rounded through fp32 (rounding.py:156-164), result
// stored as fp32 (dndarray.py:1778-1779); an empty cluster gives a zero row.
#include "hkm_common.h"

namespace hkm {

static constexpr int UPD_THREADS = 256;
static constexpr int UPD_HALVES = 8;
static constexpr int UPD_KR_MAX = 480;  // 480 x (32 x 4 + 4) B = 61.9 KB of LDS, under the 64 KB dynamic limit

UpdateGeom update_geom(int64_t N, int32_t D, int32_t K) {
    UpdateGeom g;
    g.J = (D + 31) / 32;
    g.Z = (K + UPD_KR_MAX - 1) / UPD_KR_MAX;
    g.KR = (K + g.Z - 1) / g.Z;
    // aim at ~1024 workgroups overall; keep fp32 runs <= 32768 rows and chunks >= 1024 rows
    int64_t want_s = 1024 / (int64_t(g.J) * g.Z);
    if (want_s < 1) want_s = 1;
    int64_t rpc = (N + want_s - 1) / want_s;
    if (rpc < 1024) rpc = 1024;
    if (rpc > 32768) rpc = 32768;
    rpc = (rpc + 63) / 64 * 64;
    g.rows_per_chunk = rpc;
    int64_t s = (N + rpc - 1) / rpc;
    g.S = int32_t(s < 1 ? 1 : s);
    return g;
}

__global__ __launch_bounds__(UPD_THREADS) void update_partial_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const int32_t* __restrict__ labels,
    int K, int KR, int64_t rows_per_chunk, float* __restrict__ part_sum,
    int32_t* __restrict__ part_cnt, int DPAD) {
    extern __shared__ __align__(16) float lds[];
    float* acc = lds;                                       // [KR][32]
    int32_t* cnt = reinterpret_cast<int32_t*>(lds + KR * 32);  // [KR]
    const int tid = threadIdx.x;
    const int s = blockIdx.x, j = blockIdx.y, z = blockIdx.z;
    const int kbase = z * KR;
    const int kend = min(K, kbase + KR);

    for (int i = tid; i < KR * 32; i += UPD_THREADS) acc[i] = 0.f;
    for (int i = tid; i < KR; i += UPD_THREADS) cnt[i] = 0;
    __syncthreads();

    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int col = j * 32 + c;
    const bool col_ok = col < D;
    const int q0 = wave * 2, q1 = wave * 2 + 1;
    const int64_t r_begin = int64_t(s) * rows_per_chunk;
    const int64_t r_end = min(N, r_begin + rows_per_chunk);

    int lab_next = -1;
    if (r_begin + lane < r_end) lab_next = labels[r_begin + lane];
    for (int64_t base = r_begin; base < r_end; base += 64) {
        const int lab = lab_next;
        // the next batch's labels are requested before this batch's rows: one round trip per batch
        lab_next = -1;
        if (base + 64 + lane < r_end) lab_next = labels[base + 64 + lane];
        const bool in_rng = lab >= kbase && lab < kend;
        unsigned long long own0 = __ballot(in_rng && (lab & (UPD_HALVES - 1)) == q0);
        unsigned long long own1 = __ballot(in_rng && (lab & (UPD_HALVES - 1)) == q1);
        while (own0 | own1) {
            // up to 8 rows per half-wave in flight
            constexpr int U = 8;
            int rr[U], ll[U];
            float xv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                int r0 = -1, r1 = -1;
                if (own0) {
                    r0 = __builtin_ctzll(own0);
                    own0 &= own0 - 1;
                }
                if (own1) {
                    r1 = __builtin_ctzll(own1);
                    own1 &= own1 - 1;
                }
                rr[u] = h ? r1 : r0;
                const int src = rr[u] < 0 ? 0 : rr[u];
                ll[u] = __shfl(lab, src);
                xv[u] = 0.f;
                if (rr[u] >= 0 && col_ok) xv[u] = X[(base + rr[u]) * ldx + col];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (rr[u] >= 0) {
                    const int k = ll[u] - kbase;
                    acc[k * 32 + c] += xv[u];
                    if (c == 0 && j == 0) cnt[k] += 1;
                }
            }
        }
    }
    __syncthreads();

    float* ps = part_sum + (int64_t(s) * K + kbase) * DPAD + j * 32;
    for (int i = tid; i < (kend - kbase) * 32; i += UPD_THREADS) {
        const int k = i >> 5, cc = i & 31;
        ps[int64_t(k) * DPAD + cc] = acc[k * 32 + cc];
    }
    if (j == 0)
        for (int i = tid; i < kend - kbase; i += UPD_THREADS)
            part_cnt[int64_t(s) * K + kbase + i] = cnt[i];
}

// 256 threads = 64 (k, d) pairs x 4 strided lanes over the chunks.  Lane q adds chunks q, q+4, ...
// in ascending order (8 loads in flight, additions in order); lane 0 then adds the four lane sums in
// lane order.  The order depends only on S.
__global__ __launch_bounds__(256) void update_finalize_kernel(
    const float* __restrict__ part_sum, const int32_t* __restrict__ part_cnt, int S, int K, int D,
    int DPAD, float* __restrict__ C_new, int64_t ldcn, int64_t* __restrict__ counts) {
    __shared__ double ssum[4][64];
    __shared__ int64_t scnt[4][64];
    const int e = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int64_t i = int64_t(blockIdx.x) * 64 + e;
    const bool ok = i < int64_t(K) * D;
    const int k = ok ? int(i / D) : 0, d = ok ? int(i - int64_t(k) * D) : 0;
    double sum = 0.0;
    int64_t n = 0;
    if (ok) {
        const float* ps = part_sum + int64_t(k) * DPAD + d;
        const int32_t* pc = part_cnt + k;
        const int64_t sstride = int64_t(K) * DPAD;
        int s = q;
        for (; s + 28 < S; s += 32) {
            float t[8];
            int32_t c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                t[u] = ps[(s + 4 * u) * sstride];
                c[u] = pc[int64_t(s + 4 * u) * K];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                sum += double(t[u]);
                n += c[u];
            }
        }
        for (; s < S; s += 4) {
            sum += double(ps[s * sstride]);
            n += pc[int64_t(s) * K];
        }
    }
    ssum[q][e] = sum;
    scnt[q][e] = n;
    __syncthreads();
    if (q == 0 && ok) {
        sum = ((ssum[0][e] + ssum[1][e]) + ssum[2][e]) + ssum[3][e];
        n = scnt[0][e] + scnt[1][e] + scnt[2][e] + scnt[3][e];
        // the reference's count passes through fp32 (clamp of an int64 tensor with a float bound)
        const double cnt = double(float(n < 1 ? 1 : n));
        C_new[int64_t(k) * ldcn + d] = float(sum / cnt);
        if (d == 0 && counts) counts[k] = n;
    }
}

int launch_update(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                  int32_t K, float* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                  hipStream_t st) {
    const UpdateGeom g = update_geom(N, D, K);
    const int dpad = g.J * 32;
    const size_t lds = size_t(g.KR) * 32 * sizeof(float) + size_t(g.KR) * sizeof(int32_t);
    hipLaunchKernelGGL(update_partial_kernel, dim3(g.S, g.J, g.Z), dim3(UPD_THREADS), lds, st, X, N,
                       D, ldx, labels, K, g.KR, g.rows_per_chunk, w.part_sum, w.part_cnt, dpad);
    int rc = check_launch("update_partial_kernel");
    if (rc) return rc;
    const int64_t tot = int64_t(K) * D;
    hipLaunchKernelGGL(update_finalize_kernel, dim3((unsigned)((tot + 63) / 64)), dim3(256), 0, st,
                       w.part_sum, w.part_cnt, g.S, K, D, dpad, C_new, ldcn, counts);
    return check_launch("update_finalize_kernel");
}

// ---- scalar reductions: one workgroup, fixed order ------------------------------------------
// mode 0: sum of (a[i]-b[i])^2 with the square taken in fp32 (heat/cluster/kmeans.py:141)
// mode 1: sum of v[i]                      (sum of clamped squared distances)
// mode 2: sum of sqrtf(v[i])^2, then (sqrtf(total))^2   (heat/cluster/_kcluster.py:367-368)
__device__ __forceinline__ double block_sum_fixed(double v, double* sh) {
    const int tid = threadIdx.x;
    sh[tid] = v;
    __syncthreads();
    for (int w = blockDim.x / 2; w > 0; w >>= 1) {
        if (tid < w) sh[tid] += sh[tid + w];
        __syncthreads();
    }
    const double r = sh[0];
    __syncthreads();
    return r;
}

__global__ __launch_bounds__(256) void shift_kernel(const float* __restrict__ a,
                                                    const float* __restrict__ b, int64_t n,
                                                    float* __restrict__ out) {
    __shared__ double sh[256];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
        const float d = a[i] - b[i];
        acc += double(d * d);
    }
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) *out = float(t);
}

int launch_shift(const float* C_old, const float* C_new, int32_t K, int32_t D, float* shift,
                 hipStream_t st) {
    hipLaunchKernelGGL(shift_kernel, dim3(1), dim3(256), 0, st, C_old, C_new, int64_t(K) * D, shift);
    return check_launch("shift_kernel");
}

__global__ __launch_bounds__(256) void sum_partial_kernel(const float* __restrict__ v, int64_t n,
                                                          int64_t per_block, int mode,
                                                          double* __restrict__ red) {
    __shared__ double sh[256];
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    double acc = 0.0;
    for (int64_t i = b0 + threadIdx.x; i < b1; i += 256) {
        float x = v[i];
        if (mode == 2) {
            const float r = sqrtf(x);
            x = r * r;
        }
        acc += double(x);
    }
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) red[blockIdx.x] = t;
}

__global__ __launch_bounds__(256) void sum_final_kernel(const double* __restrict__ red, int nb,
                                                        int mode, float* __restrict__ out) {
    __shared__ double sh[256];
    double acc = 0.0;
    for (int i = threadIdx.x; i < nb; i += 256) acc += red[i];
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) {
        float f = float(t);
        if (mode == 2) {
            const float r = sqrtf(f);
            f = r * r;
        }
        *out = f;
    }
}

int launch_sum_min_d2(const float* v, int64_t N, float* out, double* red, int mode,
                      hipStream_t st) {
    int nb = int((N + 65535) / 65536);
    if (nb < 1) nb = 1;
    if (nb > RED_SLOTS) nb = RED_SLOTS;
    const int64_t per_block = (N + nb - 1) / nb;
    hipLaunchKernelGGL(sum_partial_kernel, dim3(nb), dim3(256), 0, st, v, N, per_block, mode, red);
    int rc = check_launch("sum_partial_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(sum_final_kernel, dim3(1), dim3(256), 0, st, red, nb, mode, out);
    return check_launch("sum_final_kernel");
}

__global__ void widen_kernel(const int32_t* __restrict__ in, int64_t n, int64_t* __restrict__ out) {
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += int64_t(gridDim.x) * blockDim.x)
        out[i] = in[i];
}

int launch_widen(const int32_t* in, int64_t N, int64_t* out, hipStream_t st) {
    int64_t grid = (N + 255) / 256;
    const int64_t cap = int64_t(num_cus()) * 16;
    if (grid > cap) grid = cap;
    hipLaunchKernelGGL(widen_kernel, dim3((unsigned)grid), dim3(256), 0, st, in, N, out);
    return check_launch("widen_kernel");
}

}  // namespace hkm
