// The whole Lloyd loop of KMeans.fit (heat/cluster/kmeans.py:131-146) as ONE launch, for data small enough to
// stay in the registers of a few dozen workgroups (a few hundred thousand narrow rows).  Such fits are bound by
// launch and hand-over latency, not by memory or arithmetic: a step of the one-sweep kernels takes two dependent
// launches and a look from the host, a dozen microseconds for half a microsecond of memory time.  Here
//
//   * X is read from memory once per FIT: every thread keeps its PPT rows in registers for all iterations;
//   * an iteration is: assign the thread's rows (the same chain as the one-sweep kernel: D fused multiply-adds
//     that start at |c|^2 on rows of -2c, |x|^2 joins the minimum only, lazy clamp, first index wins), bring
//     the workgroup's per-cluster sums up to date, publish them, ONE hand-over between the workgroups, and then
//     every workgroup adds all published rows itself, forms the new centroids and the shift, and evaluates
//     `shift <= tol` -- all workgroups run the same instructions on the same numbers, so they agree on when to
//     stop without another exchange;
//   * the per-cluster sums are exact 64-bit integer sums: a coordinate enters as rint(x * 2^(43 - E)) with 2^E
//     above the largest |value| of its COLUMN over the whole data set (found once, before the first iteration;
//     per column, so that features of very different magnitudes each keep their 43 bits).  Integer
//     additions are exact, so (i) LDS atomics and the addition of the workgroups' rows may happen in any order,
//     (ii) the sums depend on the labels alone -- two iterations with the same labels give the same centroids
//     bit for bit, which is where the reference stops with a shift of exactly 0 -- and (iii) they can be
//     kept UP TO DATE instead of being formed again: a thread touches the table only for rows whose label
//     changed (subtract from the old cluster, add to the new one), which after the first iterations is a small
//     part of the rows.  A mean is the integer sum scaled back and divided by the count (rounded through fp32
//     like the reference, heat/core/rounding.py:156-164).  A value of at least 2^-20 of its column's largest enters
//     exactly; a smaller one with an error of at most 2^-44 of that largest value, far below the fp32 rounding
//     of the mean itself.
//
// The hand-over.  The chip's eight L2 caches are not coherent with each other for ordinary accesses, so what
// workgroups hand to each other is written and read with device-scope atomic accesses, which go past the caches.
// A round trip between workgroups on different dies costs about a microsecond and a half, so an iteration makes
// exactly one: every 64-bit word a workgroup publishes carries, in its two top bits, a stamp of the iteration it
// belongs to (the sums need 62 bits: N * 2^43 < 2^61), and a reader simply loads the words it needs until each
// shows the stamp it expects -- no arrival counter, no flag, no wait for the stores to be acknowledged; a word is
// written by one 8-byte store, so a word with the right stamp is the right word.  The rows live in two buffers
// that alternate by iteration, and a buffer's stamps go 1, 3, 1, ... resp. 2, 0, 2, ...: what a buffer held two
// iterations ago never passes for the current row.  A workgroup cannot publish row it + 2 before every other
// workgroup has read row it (it needs their rows it + 1 first, which they publish after that read).  Before the
// first iteration every workgroup clears its own two rows (stamp 0, which iterations 0 and 1 do not expect) and
// all meet once at an arrival counter, where the column maxima are exchanged too.
//
// Every wait is bounded.  A workgroup that has waited longer than the limit the host passed (device clock ticks
// of 10 ns) raises the abort flag and leaves; every other workgroup sees the flag in its own wait and leaves
// too, so the grid always drains.  The status word then says so and the caller runs the loop step by step.
// The grid is at most FIT_MAX_GRID workgroups of 1024 threads, one per CU: all of them are resident at once
// on an idle device, and on a busy one they arrive as CUs become free.
#include "hkm_common.h"

namespace hkm {

static constexpr int FIT_T = 1024;
static constexpr int FIT_QB = 43;  // bits kept below 2^E: N * 2^43 stays below 2^61 for N <= FIT_MAX_ROWS
static constexpr unsigned long long FIT_VALUE_MASK = (1ull << 62) - 1;  // a published word: 62 bits of sum, 2 of stamp
static constexpr unsigned long long FIT_MAGIC = 0x4338000000000000ull;  // bits of 1.5 * 2^52

// rows per thread: as few as give a grid of at most FIT_MAX_GRID workgroups
static int fit_ppt(int64_t N, int32_t D) {
    const int pmax = D <= 4 ? 4 : D <= 8 ? 2 : 1;  // what the registers of a 1024-thread workgroup hold
    for (int p = 1; p <= pmax; p *= 2)
        if ((N + int64_t(FIT_T) * p - 1) / (int64_t(FIT_T) * p) <= FIT_MAX_GRID) return p;
    return 0;
}

bool fit_eligible(int64_t N, int32_t D, int32_t K) {
    return N >= 1 && N <= FIT_MAX_ROWS && small_eligible(D, K) && fit_ppt(N, D) != 0;
}

int fit_grid(int64_t N, int32_t D) {
    const int p = fit_ppt(N, D);
    return p ? int((N + int64_t(FIT_T) * p - 1) / (int64_t(FIT_T) * p)) : 0;
}

// what workgroups hand to each other goes past the caches
__device__ __forceinline__ void peer_store(unsigned long long* p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long peer_load(const unsigned long long* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned peer_load32(const unsigned* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// every store this thread issued has been acknowledged
__device__ __forceinline__ void wait_stores() { __builtin_amdgcn_s_waitcnt(0x0f70); }

struct FitArgs {
    const float* X;
    int64_t N, ldx;
    const float* C0;
    int K, max_iter, has_tol, G;
    double tol;
    float* C_out;            // K x D dense
    int64_t* labels;         // N
    float* shift_out;        // device scalar
    int32_t* info;           // [0] iterations run, or a negative status; [1] bits of the last shift (may be host memory)
    unsigned long long* rows;  // [2][G][slots] what the workgroups publish
    unsigned* bar;           // [0] arrivals, [1] abort flag, [2 + d] bits of the largest |value| of column d
    unsigned long long wait_limit;  // ticks of the constant 100 MHz clock a wait may last
};

__global__ void fit_init_kernel(unsigned* bar) {
    if (threadIdx.x < 32) bar[threadIdx.x] = 0u;
}

// Counts the workgroup in and waits until `target` arrivals have been counted.  Called by every thread; true
// if the wait succeeded, false if it ran out or another workgroup gave up (the caller then leaves).
__device__ __forceinline__ bool grid_handover(unsigned* bar, unsigned target, unsigned long long limit, int* s_ok) {
    wait_stores();
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(&bar[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long t0 = wall_clock64();
        int ok = 1;
        while (peer_load32(&bar[0]) < target) {
            if (peer_load32(&bar[1]) != 0u) {
                ok = 0;
                break;
            }
            if (wall_clock64() - t0 > limit) {
                __hip_atomic_store(&bar[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = 0;
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
        *s_ok = ok;
    }
    __syncthreads();
    return *s_ok != 0;
}

template <int D, int PPT>
__global__ __launch_bounds__(FIT_T) void lloyd_fit_kernel(const FitArgs a) {
    constexpr int T = FIT_T;
    constexpr int SC = (D + 1 + 3) / 4 * 4;  // LDS centroid row: D coordinates of -2c, |c|^2, pad
    constexpr int R = 8;                     // copies of the integer table (a lane uses copy lane % R)
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int K = a.K, slots = K * (D + 1);
    float* sC = reinterpret_cast<float*>(lds_raw);                               // [K][SC]
    float* sCraw = sC + K * SC;                                                  // [K][D] centroids as they are
    unsigned long long* itab = reinterpret_cast<unsigned long long*>(sCraw + ((K * D + 3) & ~3));  // [slots][R]
    unsigned long long* tot = itab + slots * R;                                  // [slots]
    unsigned long long* strided = tot + ((slots + 1) & ~1);                      // [T]
    double* red = reinterpret_cast<double*>(strided + T);                        // [2][256]
    __shared__ int s_ok;
    __shared__ int s_max[D];
    __shared__ int s_exp[D];  // E of every column: 2^E is above its largest |value|
    const int tid = threadIdx.x, lane = tid & 63;
    const int G = a.G;

    // ---- the thread's rows, for the whole fit ----
    float x[PPT][D];
    float xn[PPT];
    int lab[PPT];
    int row[PPT];  // N <= FIT_MAX_ROWS
    if (tid < D) s_max[tid] = 0;
#pragma unroll
    for (int p = 0; p < PPT; ++p) {
        row[p] = (p * G + int(blockIdx.x)) * T + tid;
        lab[p] = -1;
        const bool have = row[p] < a.N;
        const float* xr = a.X + int64_t(have ? row[p] : 0) * a.ldx;
        float s = 0.f;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            x[p][d] = have ? xr[d] : 0.f;
            s = __fadd_rn(s, __fmul_rn(x[p][d], x[p][d]));
        }
        xn[p] = s;
    }
    for (int i = tid; i < slots * R; i += T) itab[i] = 0ull;
    __syncthreads();
    // bits of non-negative floats order like integers (NaN and inf on top)
#pragma unroll
    for (int d = 0; d < D; ++d) {
        int mx = 0;
#pragma unroll
        for (int p = 0; p < PPT; ++p) mx = max(mx, __float_as_int(x[p][d]) & 0x7fffffff);
#pragma unroll
        for (int w = 32; w > 0; w >>= 1) mx = max(mx, __shfl_xor(mx, w));
        if (lane == 0) atomicMax(&s_max[d], mx);
    }
    __syncthreads();
    if (tid < D) __hip_atomic_fetch_max(&a.bar[2 + tid], unsigned(s_max[tid]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // whatever an earlier call left in this workgroup's two rows must not pass for a row of this one
    for (int i = tid; i < 2 * slots; i += T)
        peer_store(a.rows + (size_t(i / slots) * G + blockIdx.x) * slots + (i % slots), 0ull);
    if (!grid_handover(a.bar, unsigned(G), a.wait_limit, &s_ok)) {
        if (tid == 0) a.info[0] = -1;
        return;
    }
    // a column with a non-finite value has no bound: every workgroup sees the same maxima and leaves the same
    // way, the caller runs such data step by step
    int nonfinite = 0;
    if (tid < D) {
        const int ebits = int((peer_load32(&a.bar[2 + tid]) >> 23) & 0xff);
        nonfinite = ebits == 255;
        s_exp[tid] = ebits - 127 + 1;
    }
    if (__syncthreads_or(nonfinite)) {
        if (tid == 0 && blockIdx.x == 0) a.info[0] = -2;
        return;
    }
    const double magic = __longlong_as_double((long long)FIT_MAGIC);

    for (int i = tid; i < K * D; i += T) sCraw[i] = a.C0[i];
    __syncthreads();
    // centroid rows for the scan: -2c (exact) and |c|^2, as the one-sweep kernel stages them
    auto stage_scan_rows = [&]() {
        for (int r = (tid >= 256 ? tid - 256 : tid); r < K; r += T) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const float c = sCraw[r * D + d];
                s = __fadd_rn(s, __fmul_rn(c, c));
                sC[r * SC + d] = -2.0f * c;
            }
            sC[r * SC + D] = s;
        }
    };
    stage_scan_rows();
    __syncthreads();
    __shared__ int s_fail;
    if (tid == 0) s_fail = 0;

    const int SP = slots;            // threads per group of rows in the gather
    const int J = T / SP;            // groups: thread (j, s) adds rows j, j + J, ... of slot s
    int n_iter = 0;
    float shift = 0.f;
#ifdef HKM_FIT_TRACE
    unsigned long long* trace = a.rows + size_t(2) * FIT_MAX_GRID * slots;
    unsigned long long tprev = clock64();
#define FIT_TP(i)                                                        \
    if (tid == 0 && blockIdx.x == 0) {                                   \
        const unsigned long long tn = clock64();                         \
        if (it >= 4) trace[i] += tn - tprev;                             \
        tprev = tn;                                                      \
    }
#else
#define FIT_TP(i)
#endif
    for (int it = 0; it < a.max_iter; ++it) {
        FIT_TP(0)
        // ---- assignment (heat/spatial/distance.py:59-64 + the argmin of heat/cluster/_kcluster.py:352-370) ----
        float m[PPT];
        int mi[PPT];
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            m[p] = HKM_INF;
            mi[p] = 0;
        }
#pragma unroll 2
        for (int k = 0; k < K; ++k) {
            float c[SC];
#pragma unroll
            for (int q = 0; q < SC / 4; ++q) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(sC + k * SC + 4 * q);
                c[4 * q] = v[0];
                c[4 * q + 1] = v[1];
                c[4 * q + 2] = v[2];
                c[4 * q + 3] = v[3];
            }
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                float dist = fmaf(x[p][0], c[0], c[D]);
#pragma unroll
                for (int d = 1; d < D; ++d) dist = fmaf(x[p][d], c[d], dist);
                mi[p] = dist < m[p] ? k : mi[p];
                m[p] = fminf(m[p], dist);
            }
        }
        bool neg = false;
#pragma unroll
        for (int p = 0; p < PPT; ++p) neg |= (m[p] + xn[p] < 0.f);
        if (__any(neg)) {
            // a row that coincides with a centroid up to rounding: the scan again with the clamp at 0 on every
            // value, as the reference orders them (the wave decides together, like the one-sweep kernel)
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                m[p] = HKM_INF;
                mi[p] = 0;
            }
            for (int k = 0; k < K; ++k) {
#pragma unroll
                for (int p = 0; p < PPT; ++p) {
                    float dist = fmaf(x[p][0], sC[k * SC], sC[k * SC + D]);
#pragma unroll
                    for (int d = 1; d < D; ++d) dist = fmaf(x[p][d], sC[k * SC + d], dist);
                    dist = fmaxf(dist + xn[p], 0.0f);
                    mi[p] = dist < m[p] ? k : mi[p];
                    m[p] = fminf(m[p], dist);
                }
            }
        }

        FIT_TP(1)
        // ---- the workgroup's sums follow the labels that changed ----
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            if (row[p] < a.N && mi[p] != lab[p]) {
                unsigned long long* to = itab + size_t(mi[p]) * (D + 1) * R + (lane & (R - 1));
                unsigned long long* from = itab + size_t(lab[p] < 0 ? 0 : lab[p]) * (D + 1) * R + (lane & (R - 1));
                const bool had = lab[p] >= 0;
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    const double scale = __hiloint2double((1023 + FIT_QB - s_exp[d]) << 20, 0);
                    const unsigned long long bits =
                        (unsigned long long)__double_as_longlong(fma(double(x[p][d]), scale, magic));
                    atomicAdd(to + d * R, bits);
                    if (had) atomicAdd(from + d * R, 0ull - bits);
                }
                atomicAdd(to + D * R, 1ull);
                if (had) atomicAdd(from + D * R, 0ull - 1ull);
                lab[p] = mi[p];
            }
        }
        __syncthreads();

        FIT_TP(2)
        // ---- publish the workgroup's row; add everybody's rows as they show this iteration's stamp ----
        const unsigned long long stamp = (unsigned long long)((it + 1) & 3) << 62;
        unsigned long long* mine = a.rows + (size_t(it & 1) * G + blockIdx.x) * slots;
        for (int s = tid; s < slots; s += T) {
            unsigned long long v = 0ull;
#pragma unroll
            for (int r = 0; r < R; ++r) v += itab[s * R + r];
            peer_store(mine + s, (v & FIT_VALUE_MASK) | stamp);
        }
        FIT_TP(3)
        {
            const unsigned long long* all = a.rows + size_t(it & 1) * G * slots;
            const int s = tid % SP, j = tid / SP;
            unsigned long long v = 0ull;
            bool failed = false;
            if (j < J) {
                for (int g = j; g < G && !failed; g += 8 * J) {
                    unsigned pending = 0u;
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        if (g + u * J < G) pending |= 1u << u;
                    unsigned long long t0 = 0ull;
                    unsigned polls = 0u;
                    while (pending) {
                        unsigned long long t[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u)
                            if (pending & (1u << u)) t[u] = peer_load(all + size_t(g + u * J) * slots + s);
#pragma unroll
                        for (int u = 0; u < 8; ++u)
                            if ((pending & (1u << u)) && (t[u] & ~FIT_VALUE_MASK) == stamp) {
                                v += t[u];
                                pending &= ~(1u << u);
                            }
                        if (pending && (++polls & 15u) == 0u) {
                            // a word is late: somebody gave up, or the wait has lasted too long
                            const unsigned long long now = wall_clock64();
                            if (t0 == 0ull) t0 = now;
                            if (peer_load32(&a.bar[1]) != 0u || now - t0 > a.wait_limit) {
                                failed = true;
                                break;
                            }
                        }
                    }
                }
            }
            strided[tid] = v;
            if (failed) s_fail = 1;
        }
        __syncthreads();
        if (s_fail) {
            if (tid == 0) {
                __hip_atomic_store(&a.bar[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                a.info[0] = -1;
            }
            return;
        }
        FIT_TP(4)
        // ---- the new centroids and the shift (heat/cluster/kmeans.py:76-103,141) ----
        double sq = 0.0;
        if (tid < K * D) {
            const int k = tid / D, d = tid - k * D;
            unsigned long long un = 0ull, us = 0ull;  // the J strided sums of the count and of the coordinate
            for (int q = 0; q < J; ++q) {
                un += strided[q * SP + k * (D + 1) + D];
                us += strided[q * SP + k * (D + 1) + d];
            }
            const long long n = (long long)(un & FIT_VALUE_MASK);
            // the table holds the sum of bit patterns, modulo 2^62: n times the pattern of 1.5 * 2^52 plus the sum
            // of the integers, which lies within +-2^61 (sign-extended from bit 61)
            const long long isum = (long long)((us - (unsigned long long)n * FIT_MAGIC) << 2) >> 2;
            const double cnt = double(float(n < 1 ? 1 : n));
            const double quantum = __hiloint2double((1023 - FIT_QB + s_exp[d]) << 20, 0);
            const float c = float(double(isum) * quantum / cnt);
            const float df = sCraw[tid] - c;
            sq = double(df * df);
            sCraw[tid] = c;  // only this thread reads or writes entry tid between the barriers around
        }
        // The squared differences of the K * D <= 240 coordinates, added in a fixed order by EVERY wave for itself
        // (four per lane, then a butterfly over the lanes): all threads of all workgroups get the same bits
        // without another exchange.  Two buffers by iteration parity: a wave may still be reading one when the
        // fastest writes the next iteration's.
        double* rd = red + (it & 1) * 256;
        if (tid < 256) rd[tid] = sq;
        __syncthreads();
        if (tid >= 256) stage_scan_rows();  // the next iteration's scan rows (threads 256 .. 256 + K - 1)
        {
            double r = (rd[lane] + rd[lane + 64]) + (rd[lane + 128] + rd[lane + 192]);
#pragma unroll
            for (int w = 32; w > 0; w >>= 1) r += __shfl_xor(r, w);
            shift = float(r);
        }
        n_iter = it + 1;
        __syncthreads();  // the scan rows are staged; strided and the table are free again
        FIT_TP(5)
        if (a.has_tol && double(shift) <= a.tol) break;
    }

    // ---- results: the labels of the LAST assignment, the centroids after the last update, the last shift ----
#pragma unroll
    for (int p = 0; p < PPT; ++p)
        if (row[p] < a.N) a.labels[row[p]] = lab[p];
    if (blockIdx.x == 0) {
        for (int i = tid; i < K * D; i += T) a.C_out[i] = sCraw[i];
        if (tid == 0) {
            *a.shift_out = shift;
            a.info[1] = __float_as_int(shift);
            wait_stores();
            a.info[0] = n_iter;
        }
    }
}

static size_t fit_lds_bytes(int32_t D, int32_t K) {
    const int sc = (D + 1 + 3) / 4 * 4, slots = K * (D + 1);
    return size_t(K) * sc * 4 + size_t((K * D + 3) & ~3) * 4 + size_t(slots) * 8 * 8 + size_t((slots + 1) & ~1) * 8 +
           size_t(FIT_T) * 8 + 2 * 256 * 8;
}

size_t fit_workspace_bytes(int32_t D, int32_t K) {
    return 256 + size_t(2) * FIT_MAX_GRID * size_t(K) * (D + 1) * sizeof(unsigned long long);
}

template <int D>
static int launch_fit_d(const FitArgs& a, int ppt, size_t lds, hipStream_t st) {
    const dim3 grid((unsigned)a.G), block(FIT_T);
    if (ppt == 1) hipLaunchKernelGGL((lloyd_fit_kernel<D, 1>), grid, block, lds, st, a);
    else if (ppt == 2 && D <= 8) hipLaunchKernelGGL((lloyd_fit_kernel<D, D <= 8 ? 2 : 1>), grid, block, lds, st, a);
    else if constexpr (D <= 4) {
        if (ppt == 4) hipLaunchKernelGGL((lloyd_fit_kernel<D, 4>), grid, block, lds, st, a);
        else return fail(HKM_EUNSUPPORTED, "lloyd_fit: %d rows per thread", ppt);
    } else return fail(HKM_EUNSUPPORTED, "lloyd_fit: %d rows per thread with %d features", ppt, D);
    return check_launch("lloyd_fit_kernel");
}

int launch_lloyd_fit(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C0, int32_t K, int32_t max_iter,
                     int32_t use_tol, double tol, float* C_out, int64_t* labels, float* shift_out, int32_t* info,
                     void* ws, uint64_t wait_limit_ticks, hipStream_t st) {
    const int ppt = fit_ppt(N, D);
    if (!fit_eligible(N, D, K) || ppt == 0) return fail(HKM_EUNSUPPORTED, "lloyd_fit: N = %lld, D = %d, K = %d", (long long)N, D, K);
    FitArgs a;
    a.X = X;
    a.N = N;
    a.ldx = ldx;
    a.C0 = C0;
    a.K = K;
    a.max_iter = max_iter;
    a.has_tol = use_tol ? 1 : 0;
    a.G = fit_grid(N, D);
    a.tol = tol;
    a.C_out = C_out;
    a.labels = labels;
    a.shift_out = shift_out;
    a.info = info;
    a.bar = static_cast<unsigned*>(ws);
    a.rows = reinterpret_cast<unsigned long long*>(static_cast<char*>(ws) + 256);
    a.wait_limit = wait_limit_ticks;
    const size_t lds = fit_lds_bytes(D, K);
    hipLaunchKernelGGL(fit_init_kernel, dim3(1), dim3(64), 0, st, a.bar);
    int rc = check_launch("fit_init_kernel");
    if (rc) return rc;
    prof_begin(st);
    switch (D) {
#define HKM_FIT_CASE(d) \
    case d: rc = launch_fit_d<d>(a, ppt, lds, st); break;
        HKM_FIT_CASE(1) HKM_FIT_CASE(2) HKM_FIT_CASE(3) HKM_FIT_CASE(4) HKM_FIT_CASE(5) HKM_FIT_CASE(6) HKM_FIT_CASE(7)
        HKM_FIT_CASE(8) HKM_FIT_CASE(9) HKM_FIT_CASE(10) HKM_FIT_CASE(11) HKM_FIT_CASE(12) HKM_FIT_CASE(13)
        HKM_FIT_CASE(14) HKM_FIT_CASE(15) HKM_FIT_CASE(16)
#undef HKM_FIT_CASE
        default: rc = fail(HKM_EUNSUPPORTED, "lloyd_fit: D = %d", D);
    }
    prof_end(st);
    return rc;
}

}  // namespace hkm
