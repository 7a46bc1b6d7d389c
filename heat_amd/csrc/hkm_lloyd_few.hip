// Few clusters of wide rows (K <= 16, 16 < D <= 64) on the vector ALU: the assignment alone, or the one-sweep step
// (labels + per-cluster sums from a single read of X).
//
// With so few centroids the matrix cores are the wrong tool: their work comes in blocks of 32 centroid rows, so at
// K = 8 a quarter of it is useful, and the argmin's vector instructions are paid in matrix time on top.  The vector
// ALU needs K (D + 4) instructions per point -- less than the time X takes to arrive from memory -- so the
// assignment is bound by HBM: 4 D + 4 bytes per point.
//
// A lane owns one row, held in registers (D/4 16-byte loads straight from its row -- plain loads: with 16
// contiguous bytes per lane, loads that pass the caches fetch every line several times and are 2-3 times slower);
// the next round's rows are requested before the current ones are scanned.  (Fetching a wave's 64 rows in whole
// cache lines and handing every lane its row through LDS was built and measured: no faster in this kernel.)
// The centroids
// are the same for every lane, so they are read through the scalar unit (uniform loads from the constant address
// space) and enter the multiply-adds as scalar operands: no LDS traffic and no vector registers for them.  The
// distance follows heat/spatial/distance.py:59-64: the dot product x.c as D fused multiply-adds (four partial
// sums over every fourth feature, added pairwise), then |c|^2 - 2 x.c in one more; |x|^2 joins the minimum only; the clamp at 0 is lazy; first index wins
// ties like torch.min, heat/core/statistics.py:177.
//
// The per-cluster sums are those of the one-sweep matrix-core step, with the same guarantees and the same outputs
// (fp64 partial sums and counts per workgroup, one flag per workgroup), so the same finishing kernels take over:
// a row is rounded to 28 bits below its largest coordinate (or below a floor derived from the centroid norms) and
// added to fp64 accumulators in LDS with ds_add_f64; all additions are then exact while the rows of a workgroup
// span at most 53 - 28 - ceil(log2 rows) bits of magnitude, so their order cannot matter; a workgroup that sees more,
// or a non-finite row, raises its flag and the two-pass update, which always follows and otherwise returns at
// once, recomputes the step's sums.  The D additions per row are what this step costs beyond the assignment, and
// LDS banks are what they wait for: the accumulators exist in R copies, lane l uses copy l mod R, and the strides
// are chosen for the banks: with R = 32 a copy starts one 8-byte bank after the previous one and a cluster's row is
// a multiple of 32 banks long, so the lanes of a wave touch each bank exactly twice whatever their labels; with
// fewer copies (more clusters or features than LDS has room for) the copies are 32 / R banks apart and an odd row
// length lets the labels spread the lanes.
#include "hkm_common.h"
#include "hkm_mfma_util.h"

namespace hkm {

static constexpr int FEW_QBITS = 28;  // as the one-sweep matrix-core step
static constexpr size_t FEW_LDS_HALF = 78 * 1024;  // two workgroups per compute unit
static constexpr size_t FEW_LDS_ALL = 156 * 1024;  // one

// Measured against the matrix-core kernels at N = 10M: this kernel's step is 5 to 40 % faster up to 16 clusters of
// at most 40 features and up to 12 clusters of at most 64; beyond, the vector ALU's K (D + 4) instructions per
// point no longer hide behind the memory.
bool few_eligible(int32_t D, int32_t K) { return D > 16 && D <= 64 && K >= 1 && K <= (D <= 40 ? 16 : 12); }

// padded width: whole 16-byte groups
static inline int few_dp(int32_t D) { return (D + 3) & ~3; }

// row length of a cluster's accumulators, in doubles
static inline int few_lda(int32_t D, int rep) { return rep == 32 ? (few_dp(D) + 31) & ~31 : few_dp(D) + 1; }

// distance between two copies, in doubles: the smallest length that holds [K][lda] and is 32 / rep banks past a
// multiple of 32
static inline int few_copy_stride(int32_t D, int32_t K, int rep) {
    const int need = K * few_lda(D, rep), want = (32 / rep) & 31;
    return need + ((want - need) & 31);
}

// LDS: norms; in the fused kernel R copies of the accumulators, R copies of the counts, eight words of bookkeeping
static size_t few_lds_bytes(int32_t D, int32_t K, int rep) {
    size_t b = (size_t(K) * 4 + 15) & ~size_t(15);
    if (rep > 0) b += size_t(rep) * few_copy_stride(D, K, rep) * 8 + (size_t(rep) * K + 8) * 4;
    return b;
}

// Launch geometry (measured): two workgroups of 256 lanes per compute unit where 32 copies of the accumulators fit
// in half the LDS; otherwise one workgroup with all of it -- of 1024 lanes where the scan is long enough to want
// four waves per SIMD and the rows leave the registers for them (at most 52 features), of 512 otherwise.  The
// assignment alone needs no LDS to speak of: 512 lanes from 9 clusters on.
struct FewGeometry {
    int threads, per_cu, rep;
};

static FewGeometry few_geometry(int32_t D, int32_t K, bool fused) {
    FewGeometry g{256, 2, 1};
    if (!fused) {
        if (K > 8) g.threads = 512;
        return g;
    }
    g.rep = 32;
    if (few_lds_bytes(D, K, 32) > FEW_LDS_HALF) {
        g.threads = (K > 10 && few_dp(D) <= 52) ? 1024 : 512;
        g.per_cu = 1;
        while (g.rep > 1 && few_lds_bytes(D, K, g.rep) > FEW_LDS_ALL) g.rep >>= 1;
    }
    return g;
}

int few_grid(int64_t N, int32_t D, int32_t K) {
    const FewGeometry g = few_geometry(D, K, true);
    const int64_t tiles = (N + g.threads - 1) / g.threads;
    int64_t grid = int64_t(num_cus()) * g.per_cu;
    if (grid > FUSED_MAX_GRID) grid = FUSED_MAX_GRID;
    if (grid > tiles) grid = tiles;
    return int(grid < 1 ? 1 : grid);
}

typedef const __attribute__((address_space(4))) float* few_cptr;  // uniform reads go through the scalar unit

template <int DP, bool FUSED, bool WANT_MIN, int T>
__global__ __launch_bounds__(T) void lloyd_few_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K, int64_t ldc,
    int32_t* __restrict__ labels, float* __restrict__ min_d2, int64_t ntiles, double* __restrict__ fsum,
    int32_t* __restrict__ fcnt, int32_t* __restrict__ flags, int range_bits, int nrep, int lda, int cstride,
    int mode, const int32_t* __restrict__ gate, int ngate) {
    constexpr int NV = DP / 4;
    extern __shared__ __align__(16) float lds[];
    float* sCn = lds;                                                     // [K]
    double* sA = reinterpret_cast<double*>(lds + ((K + 3) & ~3));         // [nrep][cstride], a copy = [K][lda]
    int* sN = reinterpret_cast<int*>(sA + (FUSED ? nrep * cstride : 0));  // [nrep][K], then the bookkeeping
    int* sMeta = sN + (FUSED ? nrep * K : 0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (gate) {
        // the labels a step ran without are only wanted if one of its workgroups raised its flag
        int up = 0;
        for (int i = tid; i < ngate; i += T) up |= gate[i];
        if (!__syncthreads_or(up)) return;
    }
    const bool vec = (mode & 1) != 0;     // rows are whole aligned 16-byte groups
    const few_cptr Cc = (few_cptr)C;

    for (int r = tid; r < K; r += T) {
        float s = 0.f;
        const float* c = C + int64_t(r) * ldc;
        for (int d = 0; d < D; ++d) s = __fadd_rn(s, __fmul_rn(c[d], c[d]));
        sCn[r] = s;
    }
    if (FUSED) {
        for (int i = tid; i < nrep * cstride; i += T) sA[i] = 0.0;
        for (int i = tid; i < nrep * K; i += T) sN[i] = 0;
        if (tid == 0) {
            sMeta[0] = 0x7fffffff;
            sMeta[1] = -0x7fffffff;
            sMeta[2] = 0;
            sMeta[3] = 0;
            sMeta[4] = 0x7fffffff;
        }
    }
    __syncthreads();
    int e_floor = -0x3fffffff;
    if (FUSED) {
        // the floor of the rounding quantum, from the squared centroid norms (as the one-sweep matrix-core step)
        for (int r = tid; r < K; r += T) {
            const int b = __float_as_int(sCn[r]) & 0x7fffffff;
            atomicMax(&sMeta[3], b);
            if (b != 0) atomicMin(&sMeta[4], b);
        }
        __syncthreads();
        const int cexp = (sMeta[3] >> 23) & 0xff, cexp_min = (sMeta[4] >> 23) & 0xff;
        if (cexp != 0 && cexp != 255) {
            const int e_ref = ((cexp - 127) >> 1) + 2, e_min = ((cexp_min - 127) >> 1) + 2;
            const int head = range_bits < 4 ? (range_bits < 0 ? 0 : range_bits) : 4;
            e_floor = min(e_ref + head - range_bits, e_min + 4);
        }
    }
    double* sA_lane = sA + (lane & (nrep - 1)) * cstride;
    int* sN_lane = sN + (lane & (nrep - 1)) * K;
    int emin = 0x7fffffff, emax = -0x7fffffff, nonfinite = 0;

    auto fetch = [&](int64_t tile, floatx4 (&dst)[NV]) {
        const int64_t row = tile * T + wave * 64 + lane;
        const int64_t r = row < N ? row : N - 1;
        const float* xr = X + r * ldx;
        if (vec) {
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const floatx4* q = reinterpret_cast<const floatx4*>(xr + 4 * j);
                dst[j] = *q;
            }
        } else {
#pragma unroll
            for (int j = 0; j < NV - 1; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) dst[j][t] = xr[4 * j + t];
#pragma unroll
            for (int t = 0; t < 4; ++t) dst[NV - 1][t] = 4 * (NV - 1) + t < D ? xr[4 * (NV - 1) + t] : 0.f;
        }
    };

    auto scan = [&](const floatx4 (&x)[NV], float xn, bool clamp, float& m, int& mi) {
        m = HKM_INF;
        mi = 0;
#pragma unroll DP <= 32 ? 2 : 1
        for (int k = 0; k < K; ++k) {
            const few_cptr c = Cc + int64_t(k) * ldc;
            // four partial sums (features t, t + 4, ...), then pairwise: a quarter of one chain's rounding
            float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NV - 1; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) s4[t] = fmaf(x[j][t], c[4 * j + t], s4[t]);
            if (D == DP) {
#pragma unroll
                for (int t = 0; t < 4; ++t) s4[t] = fmaf(x[NV - 1][t], c[4 * (NV - 1) + t], s4[t]);
            } else {
                // the last group reaches beyond the row: x is 0 there, the centroid's last feature stands in
#pragma unroll
                for (int t = 0; t < 4; ++t) s4[t] = fmaf(x[NV - 1][t], c[min(4 * (NV - 1) + t, D - 1)], s4[t]);
            }
            const float s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
            float dist = fmaf(-2.0f, s, sCn[k]);
            if (clamp) dist = fmaxf(dist + xn, 0.0f);
            mi = dist < m ? k : mi;
            m = fminf(m, dist);
        }
    };

    auto step = [&](int64_t tile, const floatx4 (&x)[NV], floatx4 (&xnext)[NV]) {
        if (tile + gridDim.x < ntiles) fetch(tile + gridDim.x, xnext);
        const int64_t row = tile * T + wave * 64 + lane;
        const bool valid = row < N;
        float xn = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j)
#pragma unroll
            for (int t = 0; t < 4; ++t) xn = __fadd_rn(xn, __fmul_rn(x[j][t], x[j][t]));
        float m;
        int mi;
        scan(x, xn, false, m, mi);
        m += xn;
        // a row that coincides with a centroid up to rounding: the scan again with the clamp on every value
        if (__any(m < 0.f)) scan(x, xn, true, m, mi);
        // labels may be absent: a stream of 4 bytes per row next to the reads costs more read bandwidth than its
        // share, so the fit's steps do without and compute the last iteration's labels once
        if (valid) {
            if (labels) labels[row] = mi;
            if (WANT_MIN) min_d2[row] = m;
        }
        if (FUSED && valid) {
            atomicAdd(&sN_lane[mi], 1);
            if (xn != 0.f) {  // an all-zero row adds nothing
                const int e2 = (__float_as_int(xn) >> 23) - 127;
                nonfinite |= int((e2 & 0xff) == 128);
                const int E = max((e2 >> 1) + 2, e_floor);
                emin = min(emin, E);
                emax = max(emax, E);
                const double B = __hiloint2double(((1023 + 52 - FEW_QBITS + E) << 20) | 0x80000, 0);
                double* acc = sA_lane + mi * lda;
                // (the padding beyond D is 0 in x and has its own accumulators, which nobody reads)
#pragma unroll
                for (int j = 0; j < NV; ++j)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const double v = (double(x[j][t]) + B) - B;
                        __hip_atomic_fetch_add(acc + 4 * j + t, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
            }
        }
    };

    floatx4 x0[NV], x1[NV];
    if (int64_t(blockIdx.x) < ntiles) fetch(blockIdx.x, x0);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += 2 * int64_t(gridDim.x)) {
        step(tile, x0, x1);
        if (tile + gridDim.x < ntiles) step(tile + gridDim.x, x1, x0);
    }

    if (FUSED) {
        atomicMin(&sMeta[0], emin);
        atomicMax(&sMeta[1], emax);
        if (nonfinite) atomicOr(&sMeta[2], 1);
        __syncthreads();
        double* gs = fsum + size_t(blockIdx.x) * K * D;
        for (int i = tid; i < K * D; i += T) {
            const int k = i / D, d = i - k * D;
            double v = 0.0;  // exact whatever the order (or the flag is up and the value unused)
            for (int r = 0; r < nrep; ++r) v += sA[r * cstride + k * lda + d];
            gs[i] = v;
        }
        for (int i = tid; i < K; i += T) {
            int c = 0;
            for (int r = 0; r < nrep; ++r) c += sN[r * K + i];
            fcnt[size_t(blockIdx.x) * K + i] = c;
        }
        if (tid == 0) {
            const int lo = sMeta[0], hi = sMeta[1];
            flags[blockIdx.x] = ((hi >= lo && hi - lo > range_bits) || sMeta[2]) ? 1 : 0;
        }
    }
}

template <int DP, int T>
static int launch_few_t(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K, int64_t ldc,
                        int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt, int32_t* flags,
                        const int32_t* gate, int ngate, hipStream_t st) {
    const bool fused = fsum != nullptr;
    const FewGeometry g = few_geometry(D, K, fused);
    const int64_t ntiles = (N + T - 1) / T;
    int64_t grid64 = int64_t(num_cus()) * g.per_cu;
    if (grid64 > FUSED_MAX_GRID) grid64 = FUSED_MAX_GRID;
    if (grid64 > ntiles) grid64 = ntiles;
    const int grid = int(grid64);
    const bool vec = aligned16(X) && ldx % 4 == 0 && D % 4 == 0;
    const int nrep = g.rep;
    const size_t lds = few_lds_bytes(D, K, fused ? nrep : 0);
    const int lda = few_lda(D, nrep), cstride = few_copy_stride(D, K, nrep);
    const int mode = vec ? 1 : 0;
    // rows one workgroup adds up, as a power of two
    const int64_t per_wg = (ntiles + grid - 1) / grid * T;
    int lg = 0;
    while ((int64_t(1) << lg) < per_wg) ++lg;
    const int range_bits = 53 - FEW_QBITS - lg;
#define HKM_FEW_GO(F, M)                                                                                      \
    do {                                                                                                      \
        auto kern = lloyd_few_kernel<DP, F, M, T>;                                                             \
        if (lds > 64 * 1024) {                                                                                \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                           \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));         \
            if (e != hipSuccess) return fail(HKM_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));      \
        }                                                                                                     \
        if (!gate) prof_begin(st); /* (a gated launch that returns at once is no sample of the kernel's time) */ \
        hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(T), lds,     st, X, N, D, ldx, C, K, ldc, labels, \
                           min_d2, ntiles, fsum, fcnt, flags, range_bits, nrep, lda, cstride, mode, gate,    \
                           ngate);                                                                            \
    } while (0)
    if (fused) {
        if (min_d2) HKM_FEW_GO(true, true);
        else HKM_FEW_GO(true, false);
    } else {
        if (min_d2) HKM_FEW_GO(false, true);
        else HKM_FEW_GO(false, false);
    }
#undef HKM_FEW_GO
    if (!gate) prof_end(st);
    return check_launch("lloyd_few_kernel");
}

// fsum == nullptr: the assignment alone.  labels == nullptr (the step only): none are stored.  gate != nullptr: the
// launch does nothing unless one of gate[0 .. ngate) is non-zero.
int launch_few(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K, int64_t ldc,
               int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt, int32_t* flags, hipStream_t st,
               const int32_t* gate, int ngate) {
    if (N == 0) return HKM_OK;
    const int threads = few_geometry(D, K, fsum != nullptr).threads;
    switch (few_dp(D)) {
#define HKM_FEW_CASE(d)                                                                                   \
    case d:                                                                                               \
        switch (threads) {                                                                                \
            case 256: return launch_few_t<d, 256>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, gate, ngate, st); \
            case 512: return launch_few_t<d, 512>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, gate, ngate, st); \
            default:                                                                                      \
                return launch_few_t<d, (d <= 52 ? 1024 : 512)>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, \
                                                               flags, gate, ngate, st);                   \
        }
        HKM_FEW_CASE(20) HKM_FEW_CASE(24) HKM_FEW_CASE(28) HKM_FEW_CASE(32) HKM_FEW_CASE(36) HKM_FEW_CASE(40)
        HKM_FEW_CASE(44) HKM_FEW_CASE(48) HKM_FEW_CASE(52) HKM_FEW_CASE(56) HKM_FEW_CASE(60) HKM_FEW_CASE(64)
#undef HKM_FEW_CASE
        default: return fail(HKM_EUNSUPPORTED, "lloyd_few: D=%d", D);
    }
}

}  // namespace hkm
