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
static constexpr int UPD_KR_MAX = 448;  // (448 + 1) x (32 x 4 + 4) B + 4.6 KB of row lists = 63.9 KB of LDS (64 KB dynamic limit)

UpdateGeom update_geom(int64_t N, int32_t D, int32_t K, int32_t elem) {
    UpdateGeom g;
    const int kr_max = elem == 8 ? UPD_KR_MAX / 2 : UPD_KR_MAX;  // fp64 accumulator rows are twice as wide
    g.J = (D + 31) / 32;
    g.Z = (K + kr_max - 1) / kr_max;
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

template <typename T>
__global__ __launch_bounds__(UPD_THREADS) void update_partial_kernel(
    const T* __restrict__ X, int64_t N, int D, int64_t ldx, const int32_t* __restrict__ labels,
    int K, int KR, int64_t rows_per_chunk, T* __restrict__ part_sum,
    int32_t* __restrict__ part_cnt, int DPAD, const int32_t* __restrict__ gate, int ngate) {
    // behind the one-sweep MFMA step this pass only runs if some workgroup there raised its flag
    if (gate) {
        int any = 0;
        for (int i = threadIdx.x; i < ngate; i += UPD_THREADS) any |= gate[i];
        if (!__syncthreads_or(any)) return;
    }
    constexpr int U = 4;          // rows per half-wave and pass
    constexpr int LIST = 64 + U;  // a batch has 64 rows; room for the padding to a multiple of U
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* acc = reinterpret_cast<T*>(lds_raw);                           // [KR + 1][32], last row = sink
    int32_t* cnt = reinterpret_cast<int32_t*>(acc + (KR + 1) * 32);   // [KR + 1]
    int2* lists = reinterpret_cast<int2*>(cnt + ((KR + 1 + 1) & ~1)); // [8 half-waves][LIST]
    const int tid = threadIdx.x;
    const int s = blockIdx.x, j = blockIdx.y, z = blockIdx.z;
    const int kbase = z * KR;
    const int kend = min(K, kbase + KR);

    for (int i = tid; i < (KR + 1) * 32; i += UPD_THREADS) acc[i] = T(0);
    for (int i = tid; i < KR + 1; i += UPD_THREADS) cnt[i] = 0;
    __syncthreads();

    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int col = j * 32 + c;
    const bool col_ok = col < D;
    const int q0 = wave * 2, q1 = wave * 2 + 1;
    int2* my_list = lists + (wave * 2 + h) * LIST;  // list of the half-wave this lane belongs to
    int2* list0 = lists + q0 * LIST;
    int2* list1 = lists + q1 * LIST;
    const bool count_here = (c == 0) && (j == 0);
    const int64_t r_begin = int64_t(s) * rows_per_chunk;
    const int64_t r_end = min(N, r_begin + rows_per_chunk);
    const T* xcol = X + (col_ok ? col : 0);

    int lab_next = -1;
    if (r_begin + lane < r_end) lab_next = labels[r_begin + lane];
    for (int64_t base = r_begin; base < r_end; base += 64) {
        const int lab = lab_next;
        // the next batch's labels are requested before this batch's rows
        lab_next = -1;
        if (base + 64 + lane < r_end) lab_next = labels[base + 64 + lane];

        // Each half-wave collects the rows of the batch whose cluster it owns, in ascending row order,
        // as (row, local cluster) pairs in its LDS list; the list is padded to a multiple of U with
        // entries that add row 0 of the batch to the sink row.
        const bool in_rng = lab >= kbase && lab < kend;
        const bool p0 = in_rng && (lab & (UPD_HALVES - 1)) == q0;
        const bool p1 = in_rng && (lab & (UPD_HALVES - 1)) == q1;
        const unsigned long long m0 = __ballot(p0), m1 = __ballot(p1);
        const int n0 = __popcll(m0), n1 = __popcll(m1);
        const int rank0 = __builtin_amdgcn_mbcnt_hi(unsigned(m0 >> 32), __builtin_amdgcn_mbcnt_lo(unsigned(m0), 0));
        const int rank1 = __builtin_amdgcn_mbcnt_hi(unsigned(m1 >> 32), __builtin_amdgcn_mbcnt_lo(unsigned(m1), 0));
        if (p0) list0[rank0] = make_int2(lane, lab - kbase);
        if (p1) list1[rank1] = make_int2(lane, lab - kbase);
        const int nmax = max(n0, n1);
        const int npad = (nmax + U - 1) / U * U;
        if (lane < npad - n0) list0[n0 + lane] = make_int2(0, KR);
        if (lane < npad - n1) list1[n1 + lane] = make_int2(0, KR);
        wave_lds_sync();  // the lists are read by other lanes than those that wrote them

        for (int t = 0; t < npad; t += U) {
            int2 e[U];
            T xv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) e[u] = my_list[t + u];
#pragma unroll
            for (int u = 0; u < U; ++u) xv[u] = xcol[(base + e[u].x) * ldx];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                acc[e[u].y * 32 + c] += col_ok ? xv[u] : T(0);
                if (count_here) cnt[e[u].y] += 1;
            }
        }
        wave_lds_sync();  // the next batch overwrites the lists
    }
    __syncthreads();

    T* ps = part_sum + (int64_t(s) * K + kbase) * DPAD + j * 32;
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
// With fsum != NULL the partials of the one-sweep MFMA step ([G][K][D] fp64, [G][K] counts) are used
// unless one of its workgroups raised its flag; then the fp32 partials of pass 1 are.
template <typename T>
__global__ __launch_bounds__(256) void update_finalize_kernel(
    const T* __restrict__ part_sum, const int32_t* __restrict__ part_cnt, int S, int K, int D,
    int DPAD, T* __restrict__ C_new, int64_t ldcn, int64_t* __restrict__ counts,
    const T* __restrict__ C_old, double* __restrict__ shift_part,
    const double* __restrict__ fsum, const int32_t* __restrict__ fcnt,
    const int32_t* __restrict__ fflags, int G) {
    __shared__ double ssum[4][64];
    __shared__ double ssq[64];
    __shared__ int64_t scnt[4][64];
    const int e = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int64_t i = int64_t(blockIdx.x) * 64 + e;
    const bool ok = i < int64_t(K) * D;
    const int k = ok ? int(i / D) : 0, d = ok ? int(i - int64_t(k) * D) : 0;
    double sum = 0.0;
    int64_t n = 0;
    bool fused = fsum != nullptr;
    if (fused) {
        int any = 0;
        for (int g = threadIdx.x; g < G; g += 256) any |= fflags[g];
        fused = !__syncthreads_or(any);
    }
    if (ok && fused) {
        const double* ps = fsum + int64_t(k) * D + d;
        const int32_t* pc = fcnt + k;
        const int64_t sstride = int64_t(K) * D;
        int s = q;
        for (; s + 28 < G; s += 32) {
            double t[8];
            int32_t c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                t[u] = ps[(s + 4 * u) * sstride];
                c[u] = pc[int64_t(s + 4 * u) * K];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                sum += t[u];
                n += c[u];
            }
        }
        for (; s < G; s += 4) {
            sum += ps[s * sstride];
            n += pc[int64_t(s) * K];
        }
    } else if (ok) {
        const T* ps = part_sum + int64_t(k) * DPAD + d;
        const int32_t* pc = part_cnt + k;
        const int64_t sstride = int64_t(K) * DPAD;
        int s = q;
        for (; s + 28 < S; s += 32) {
            T t[8];
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
        const T cnew = T(sum / cnt);
        C_new[int64_t(k) * ldcn + d] = cnew;
        if (d == 0 && counts) counts[k] = n;
        if (C_old) {
            const T df = C_old[int64_t(k) * D + d] - cnew;  // square taken in the data type (kmeans.py:141)
            ssq[e] = double(df * df);
        }
    }
    if (C_old) {
        // this block's share of sum((C - C_new)^2), added in element order
        if (q == 0 && !ok) ssq[e] = 0.0;
        __syncthreads();
        if (threadIdx.x == 0) {
            double t = 0.0;
            for (int i = 0; i < 64; ++i) t += ssq[i];
            shift_part[blockIdx.x] = t;
        }
    }
}

// one workgroup adds the per-block shares in block order
template <typename T>
__global__ __launch_bounds__(256) void shift_final_kernel(const double* __restrict__ part, int nb,
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

template <typename T>
static int launch_update_t(const T* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                           int32_t K, T* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                           const T* C_old, T* shift, hipStream_t st) {
    const UpdateGeom g = update_geom(N, D, K, int32_t(sizeof(T)));
    const int dpad = g.J * 32;
    const size_t lds = size_t(g.KR + 1) * 32 * sizeof(T) + size_t((g.KR + 2) & ~1) * sizeof(int32_t) +
                       size_t(UPD_HALVES) * (64 + 8) * sizeof(int2);
    T* part = reinterpret_cast<T*>(w.part_sum);
    hipLaunchKernelGGL(update_partial_kernel<T>, dim3(g.S, g.J, g.Z), dim3(UPD_THREADS), lds, st, X, N,
                       D, ldx, labels, K, g.KR, g.rows_per_chunk, part, w.part_cnt, dpad,
                       static_cast<const int32_t*>(nullptr), 0);
    int rc = check_launch("update_partial_kernel");
    if (rc) return rc;
    const int64_t tot = int64_t(K) * D;
    const int nb = int((tot + 63) / 64);
    hipLaunchKernelGGL(update_finalize_kernel<T>, dim3(nb), dim3(256), 0, st, static_cast<const T*>(part),
                       static_cast<const int32_t*>(w.part_cnt), g.S, K, D, dpad, C_new, ldcn, counts, C_old,
                       w.shift_part, static_cast<const double*>(nullptr),
                       static_cast<const int32_t*>(nullptr), static_cast<const int32_t*>(nullptr), 0);
    rc = check_launch("update_finalize_kernel");
    if (rc || !C_old) return rc;
    hipLaunchKernelGGL(shift_final_kernel<T>, dim3(1), dim3(256), 0, st, static_cast<const double*>(w.shift_part),
                       nb, shift);
    return check_launch("shift_final_kernel");
}

int launch_update_f64(const double* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                      int32_t K, double* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                      const double* C_old, double* shift, hipStream_t st) {
    return launch_update_t<double>(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, C_old, shift, st);
}

int launch_update(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                  int32_t K, float* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                  const float* C_old, float* shift, hipStream_t st) {
    return launch_update_t<float>(X, N, D, ldx, labels, K, C_new, ldcn, counts, w, C_old, shift, st);
}

// Second half of the one-sweep MFMA step: the two-pass update gated by the flags of the fused kernel
// (normally every workgroup returns at once), then the finalize that reads whichever partials hold.
int launch_update_fused(const float* X, int64_t N, int32_t D, int64_t ldx, const int32_t* labels,
                        int32_t K, float* C_new, int64_t ldcn, int64_t* counts, const Workspace& w,
                        int fgrid, const float* C_old, float* shift, hipStream_t st) {
    const UpdateGeom g = update_geom(N, D, K, 4);
    const int dpad = g.J * 32;
    const size_t lds = size_t(g.KR + 1) * 32 * sizeof(float) + size_t((g.KR + 2) & ~1) * sizeof(int32_t) +
                       size_t(UPD_HALVES) * (64 + 8) * sizeof(int2);
    hipLaunchKernelGGL(update_partial_kernel<float>, dim3(g.S, g.J, g.Z), dim3(UPD_THREADS), lds, st, X, N,
                       D, ldx, labels, K, g.KR, g.rows_per_chunk, w.part_sum, w.part_cnt, dpad,
                       static_cast<const int32_t*>(w.fflags), fgrid);
    int rc = check_launch("update_partial_kernel");
    if (rc) return rc;
    const int64_t tot = int64_t(K) * D;
    const int nb = int((tot + 63) / 64);
    hipLaunchKernelGGL(update_finalize_kernel<float>, dim3(nb), dim3(256), 0, st,
                       static_cast<const float*>(w.part_sum), static_cast<const int32_t*>(w.part_cnt), g.S, K,
                       D, dpad, C_new, ldcn, counts, C_old, w.shift_part, static_cast<const double*>(w.fsum),
                       static_cast<const int32_t*>(w.fcnt), static_cast<const int32_t*>(w.fflags), fgrid);
    rc = check_launch("update_finalize_kernel");
    if (rc || !C_old) return rc;
    hipLaunchKernelGGL(shift_final_kernel<float>, dim3(1), dim3(256), 0, st,
                       static_cast<const double*>(w.shift_part), nb, shift);
    return check_launch("shift_final_kernel");
}

// ---- scalar reductions: one workgroup, fixed order ------------------------------------------
// mode 0: sum of (a[i]-b[i])^2 with the square taken in fp32 (heat/cluster/kmeans.py:141)
// mode 1: sum of v[i]                      (sum of clamped squared distances)
// mode 2: sum of sqrtf(v[i])^2, then (sqrtf(total))^2   (heat/cluster/_kcluster.py:367-368)
// mode 3: sum of sqrtf(v[i])               (clustering cost of k-means||, _kcluster.py:163-170,312-316)

__device__ __forceinline__ float hkm_sqrt(float v) { return sqrtf(v); }
__device__ __forceinline__ double hkm_sqrt(double v) { return sqrt(v); }

template <typename T>
__global__ __launch_bounds__(256) void shift_kernel(const T* __restrict__ a,
                                                    const T* __restrict__ b, int64_t n,
                                                    T* __restrict__ out) {
    __shared__ double sh[256];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
        const T d = a[i] - b[i];
        acc += double(d * d);
    }
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) *out = T(t);
}

int launch_shift(const float* C_old, const float* C_new, int32_t K, int32_t D, float* shift,
                 hipStream_t st) {
    hipLaunchKernelGGL(shift_kernel<float>, dim3(1), dim3(256), 0, st, C_old, C_new, int64_t(K) * D, shift);
    return check_launch("shift_kernel");
}

int launch_shift_f64(const double* C_old, const double* C_new, int32_t K, int32_t D, double* shift,
                     hipStream_t st) {
    hipLaunchKernelGGL(shift_kernel<double>, dim3(1), dim3(256), 0, st, C_old, C_new, int64_t(K) * D, shift);
    return check_launch("shift_kernel");
}

// mode 0: plain sum, 2: sum of sqrt(x)^2, 3: sum of sqrt(x)
template <typename T>
__device__ __forceinline__ double sum_term(T x, int mode) {
    if (mode == 2) {
        const T r = hkm_sqrt(x);
        x = r * r;
    } else if (mode == 3) {
        x = hkm_sqrt(x);
    }
    return double(x);
}

// A block sums its contiguous range with four independent 16-byte loads in flight per thread (VEC:
// float data, 16-byte aligned; per_block is a multiple of 4096 elements), each feeding its own fp64
// accumulator in a fixed order -- a single dependent 4-byte load per trip ran at a twentieth of the
// memory rate.  The partials are combined in a fixed order: the result is reproducible.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sum_partial_kernel(const T* __restrict__ v, int64_t n,
                                                          int64_t per_block, int mode,
                                                          double* __restrict__ red) {
    __shared__ double sh[256];
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    double acc = 0.0;
    int64_t i0 = b0;
    if (VEC) {
        double a[4] = {0.0, 0.0, 0.0, 0.0};
        for (; i0 + 4096 <= b1; i0 += 4096) {
            float4 q[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                q[t] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(v) + i0 + t * 1024 + threadIdx.x * 4);
#pragma unroll
            for (int t = 0; t < 4; ++t)
                a[t] += ((sum_term<float>(q[t].x, mode) + sum_term<float>(q[t].y, mode)) +
                         (sum_term<float>(q[t].z, mode) + sum_term<float>(q[t].w, mode)));
        }
        acc = (a[0] + a[1]) + (a[2] + a[3]);
    }
    for (int64_t i = i0 + threadIdx.x; i < b1; i += 256) acc += sum_term<T>(v[i], mode);
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) red[blockIdx.x] = t;
}

template <typename T>
__global__ __launch_bounds__(256) void sum_final_kernel(const double* __restrict__ red, int nb,
                                                        int mode, T* __restrict__ out) {
    __shared__ double sh[256];
    double acc = 0.0;
    for (int i = threadIdx.x; i < nb; i += 256) acc += red[i];
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) {
        T f = T(t);
        if (mode == 2) {
            const T r = hkm_sqrt(f);
            f = r * r;
        }
        *out = f;
    }
}

template <typename T>
static int launch_sum_t(const T* v, int64_t N, T* out, double* red, int mode, hipStream_t st) {
    int nb = int((N + 16383) / 16384);
    if (nb < 1) nb = 1;
    if (nb > RED_SLOTS) nb = RED_SLOTS;
    const int64_t per_block = ((N > 0 ? (N + nb - 1) / nb : 1) + 4095) / 4096 * 4096;
    nb = int((N + per_block - 1) / per_block);
    if (nb < 1) nb = 1;
    if (sizeof(T) == 4 && aligned16(v))
        hipLaunchKernelGGL((sum_partial_kernel<T, true>), dim3(nb), dim3(256), 0, st, v, N, per_block, mode, red);
    else
        hipLaunchKernelGGL((sum_partial_kernel<T, false>), dim3(nb), dim3(256), 0, st, v, N, per_block, mode, red);
    int rc = check_launch("sum_partial_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(sum_final_kernel<T>, dim3(1), dim3(256), 0, st, static_cast<const double*>(red), nb, mode,
                       out);
    return check_launch("sum_final_kernel");
}

// dmin[i] = min(dmin[i], dnew[i]) and the partial sums of sqrt(dmin[i]) in one pass: the running minimum
// of a k-means|| round merged with the cost of the next one.  Same blocking and order as
// sum_partial_kernel, so the sum equals hkm_min_dist_sum_f32 of the merged array bit for bit.
template <bool VEC>
__global__ __launch_bounds__(256) void min_merge_partial_kernel(float* __restrict__ dmin, const float* __restrict__ dnew,
                                                                int64_t n, int64_t per_block,
                                                                double* __restrict__ red) {
    __shared__ double sh[256];
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    double acc = 0.0;
    int64_t i0 = b0;
    if (VEC) {
        double a[4] = {0.0, 0.0, 0.0, 0.0};
        for (; i0 + 4096 <= b1; i0 += 4096) {
            float4 q[4], r[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                q[t] = *reinterpret_cast<const float4*>(dmin + i0 + t * 1024 + threadIdx.x * 4);
                r[t] = *reinterpret_cast<const float4*>(dnew + i0 + t * 1024 + threadIdx.x * 4);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                q[t].x = fminf(q[t].x, r[t].x);
                q[t].y = fminf(q[t].y, r[t].y);
                q[t].z = fminf(q[t].z, r[t].z);
                q[t].w = fminf(q[t].w, r[t].w);
                *reinterpret_cast<float4*>(dmin + i0 + t * 1024 + threadIdx.x * 4) = q[t];
                a[t] += ((sum_term<float>(q[t].x, 3) + sum_term<float>(q[t].y, 3)) +
                         (sum_term<float>(q[t].z, 3) + sum_term<float>(q[t].w, 3)));
            }
        }
        acc = (a[0] + a[1]) + (a[2] + a[3]);
    }
    for (int64_t i = i0 + threadIdx.x; i < b1; i += 256) {
        const float m = fminf(dmin[i], dnew[i]);
        dmin[i] = m;
        acc += sum_term<float>(m, 3);
    }
    const double t = block_sum_fixed(acc, sh);
    if (threadIdx.x == 0) red[blockIdx.x] = t;
}

int launch_min_merge_sum(float* dmin, const float* dnew, int64_t N, float* out, double* red, hipStream_t st) {
    int nb = int((N + 16383) / 16384);
    if (nb < 1) nb = 1;
    if (nb > RED_SLOTS) nb = RED_SLOTS;
    const int64_t per_block = ((N > 0 ? (N + nb - 1) / nb : 1) + 4095) / 4096 * 4096;
    nb = int((N + per_block - 1) / per_block);
    if (nb < 1) nb = 1;
    if (aligned16(dmin) && aligned16(dnew))
        hipLaunchKernelGGL(min_merge_partial_kernel<true>, dim3(nb), dim3(256), 0, st, dmin, dnew, N, per_block, red);
    else
        hipLaunchKernelGGL(min_merge_partial_kernel<false>, dim3(nb), dim3(256), 0, st, dmin, dnew, N, per_block, red);
    int rc = check_launch("min_merge_partial_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(sum_final_kernel<float>, dim3(1), dim3(256), 0, st, static_cast<const double*>(red), nb, 3, out);
    return check_launch("sum_final_kernel");
}

int launch_sum_min_d2(const float* v, int64_t N, float* out, double* red, int mode, hipStream_t st) {
    return launch_sum_t<float>(v, N, out, red, mode, st);
}

int launch_sum_min_d2_f64(const double* v, int64_t N, double* out, double* red, int mode, hipStream_t st) {
    return launch_sum_t<double>(v, N, out, red, mode, st);
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
