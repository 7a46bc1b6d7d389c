// Resident distance + argmin (and the one-sweep Lloyd step) with the cross term x.c evaluated on the
// bf16 matrix cores from fp32 operands split three ways -- an opt-in alternative to the fp32 MFMA
// kernels of hkm_assign_mfma.hip (environment HKM_PRODUCTS=bf16x3, see hkm_api.hip).
//
// Every fp32 value v is written as v1 + v2 + v3 with v1 = bf16(v), v2 = bf16(v - v1),
// v3 = bf16(v - v1 - v2) (round to nearest even; the differences are exact in fp32, and the three
// 8-bit significands cover the 24 bits of v up to 2^-24 |v|).  The product x.c is the sum of the six
// partial products x_i c_j with i + j <= 4; a product of two bf16 values is exact in fp32 and the
// matrix core accumulates in fp32.  What is dropped (x2 c3 + x3 c2 + x3 c3) is below
// 2^-23 sum_k |x_k c_k|, the size of the rounding error of ONE fp32 multiply-add per term -- the
// fp32 MFMA path and an sgemm commit such an error D times.  The small products are accumulated
// first.  v_mfma_f32_32x32x16_bf16 retires 16 features per instruction in half the time the fp32
// MFMA needs for 2: the six partial products cost 3/8 of the fp32 path's matrix time, and -- unlike
// the fp32 MFMA -- the bf16 MFMA runs concurrently with the vector instructions of the argmin scan.
//
// Everything else is the fp32 resident kernel: centroids (-2c, three bf16 planes) and their squared
// norms live in LDS, the accumulators start at |c|^2, |x|^2 joins the minimum only, lazy clamp with
// exact rescan, first index wins ties; the fused variant adds the rows to fp64 LDS accumulators after
// pre-rounding them, exactly as lloyd_mfma_resident_kernel does (same workspace layout, same fallback).
#include "hkm_common.h"
#include "hkm_mfma_util.h"

namespace hkm {

static constexpr int SPLIT_QBITS = 28;
static constexpr int SPLIT_FUSED_THREADS = 512;  // 2 waves per SIMD: room for the split operands without spills

// LDS row stride of a centroid plane in bf16 elements: 16 bytes of padding keep the 16-byte operand
// reads of 16 consecutive lanes on different banks
__host__ __device__ constexpr int split_ldb(int dp) { return dp + 8; }

// The six partial products of one centroid block (32 rows, parts cs) with one point block (parts xq),
// smallest products first, starting from the squared norms c0.
template <int NS>
__device__ __forceinline__ floatx16 split_products(const uintx4 (&cs)[3][NS], const uintx4 (&xq)[3][NS],
                                                   const floatx16& c0) {
    constexpr int XP[6] = {2, 0, 1, 1, 0, 0};
    constexpr int CP[6] = {0, 2, 1, 0, 1, 0};
    floatx16 acc = c0;
#pragma unroll
    for (int t = 0; t < 6; ++t)
#pragma unroll
        for (int s = 0; s < NS; ++s) acc = MFMA_BF16(as_bf16x8(cs[CP[t]][s]), as_bf16x8(xq[XP[t]][s]), acc);
    return acc;
}

// block_argmin without its branch, so that it can share a basic block with matrix instructions: the
// position is looked up unconditionally and taken if the block minimum improves the running one
__device__ __forceinline__ void block_argmin_flat(const floatx16& d, int kb, float& m, int& mi) {
    const float t0 = fminf(fminf(d[0], d[1]), d[2]);
    const float t1 = fminf(fminf(d[3], d[4]), d[5]);
    const float t2 = fminf(fminf(d[6], d[7]), d[8]);
    const float t3 = fminf(fminf(d[9], d[10]), d[11]);
    const float t4 = fminf(fminf(d[12], d[13]), d[14]);
    const float bm = fminf(fminf(fminf(t0, t1), t2), fminf(fminf(t3, t4), d[15]));
    int bi = 8 * (15 >> 2) + (15 & 3);
#pragma unroll
    for (int v = 14; v >= 0; --v) bi = (d[v] == bm) ? 8 * (v >> 2) + (v & 3) : bi;
    const bool lt = bm < m;
    mi = lt ? kb + bi : mi;
    m = lt ? bm : m;
}

// asks the scheduler to order the region that ends here as N groups of one matrix instruction
// followed by VALU vector instructions
template <int N, int VALU>
__device__ __forceinline__ void interleave_mfma_valu() {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, VALU, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
}

// Scan of all centroid blocks for PB = 2 point blocks as a software pipeline.  A wave issues in
// order, and the bf16 matrix core runs concurrently with the vector ALU only for what is issued
// between its instructions, so the vector instructions of one argmin scan are placed BETWEEN the
// matrix instructions of the next product block (about four per matrix instruction):
//   phase B of block cb:   products (cb, point block 1)   with the scan of (cb, point block 0)
//   phase A of block cb+1: products (cb+1, point block 0) with the scan of (cb, point block 1)
// CLAMP applies max(. + |x|^2, 0) to every value (the rescan of a tile whose lazy minimum came out
// negative).
template <int DP, bool CLAMP>
__device__ __forceinline__ void split_scan(const __bf16* planes, int plane_stride, const float* sCn, int ncb, int p,
                                           int h, const uintx4 (&xs)[2][3][DP / 16], const float (&xn)[2],
                                           float (&m)[2], int (&mi)[2]) {
    constexpr int LDB = split_ldb(DP);
    constexpr int NS = DP / 16;
    constexpr int NM = 6 * NS;
    constexpr int VPM = CLAMP ? 7 : 4;  // vector instructions per matrix instruction
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        m[pb] = HKM_INF;
        mi[pb] = 0;
    }
    auto load_cs = [&](int cb, uintx4 (&cs)[3][NS]) {
        const int row_off = (cb * 32 + p) * LDB + h * (DP / 2);
#pragma unroll
        for (int part = 0; part < 3; ++part)
#pragma unroll
            for (int s = 0; s < NS; ++s)
                cs[part][s] = *reinterpret_cast<const uintx4*>(planes + part * plane_stride + row_off + 8 * s);
    };
    auto scan = [&](floatx16& acc, int pb, int kb) {
        if (CLAMP) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = fmaxf(acc[v] + xn[pb], 0.0f);
        }
        block_argmin_flat(acc, kb, m[pb], mi[pb]);
    };
    uintx4 cs[3][NS];
    load_cs(0, cs);
    floatx16 c0 = load_cn16(sCn + 4 * h);
    floatx16 acc0 = split_products<NS>(cs, xs[0], c0);  // prologue: (block 0, point block 0)
    __builtin_amdgcn_sched_barrier(0);
    floatx16 acc1;
    // (no branch inside the loop body: the scheduler orders one basic block at a time)
    for (int cb = 0; cb + 1 < ncb; ++cb) {
        // phase B of block cb
        acc1 = split_products<NS>(cs, xs[1], c0);
        scan(acc0, 0, cb * 32);
        interleave_mfma_valu<NM, VPM>();
        // phase A of block cb + 1
        load_cs(cb + 1, cs);
        c0 = load_cn16(sCn + (cb + 1) * 32 + 4 * h);
        acc0 = split_products<NS>(cs, xs[0], c0);
        scan(acc1, 1, cb * 32);
        interleave_mfma_valu<NM, VPM>();
    }
    // last block: phase B, then the scan that has nothing left to hide behind
    acc1 = split_products<NS>(cs, xs[1], c0);
    scan(acc0, 0, (ncb - 1) * 32);
    interleave_mfma_valu<NM, VPM>();
    scan(acc1, 1, (ncb - 1) * 32);
    if (!CLAMP) {
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) m[pb] += xn[pb];
    }
}

// FUSED: also the per-cluster sums (fsum / fcnt / flags as in lloyd_mfma_resident_kernel)
template <int DP, int PB, bool VEC, bool FUSED>
__global__ __launch_bounds__(FUSED ? SPLIT_FUSED_THREADS : 256) void split_resident_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, int32_t* __restrict__ labels, float* __restrict__ min_d2, int64_t ntiles,
    double* __restrict__ fsum, int32_t* __restrict__ fcnt, int32_t* __restrict__ flags, int range_bits) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int LDB = split_ldb(DP);
    constexpr int LDA = DP + 1;
    constexpr int NJ = DP / 8;   // 16-byte groups of fp32 per lane-half
    constexpr int NS = DP / 16;  // k-steps of the bf16 MFMA
    const int KP = (K + 31) & ~31;
    const int plane_stride = KP * LDB;
    __bf16* planes = reinterpret_cast<__bf16*>(lds_raw);                                   // [3][KP][LDB]
    float* sCn = reinterpret_cast<float*>(lds_raw + size_t(3) * plane_stride * 2);         // [KP]
    double* sA = reinterpret_cast<double*>(sCn + KP);                                      // FUSED: [K][LDA]
    int* sN = reinterpret_cast<int*>(sA + (FUSED ? size_t(K) * LDA : 0));                  // FUSED: [K] + 2
    const int tid = threadIdx.x, nthr = blockDim.x;

    for (int i = tid; i < KP * (DP / 2); i += nthr) {
        const int r = i / (DP / 2), c = (i - r * (DP / 2)) * 2;
        float a = 0.f, b = 0.f;
        if (r < K) {
            if (c < D) a = -2.0f * C[int64_t(r) * ldc + c];
            if (c + 1 < D) b = -2.0f * C[int64_t(r) * ldc + c + 1];
        }
        unsigned p1, p2, p3;
        split_pair(a, b, p1, p2, p3);
        unsigned* dst = reinterpret_cast<unsigned*>(planes + r * LDB + c);
        dst[0] = p1;
        dst[plane_stride / 2] = p2;
        dst[plane_stride] = p3;
    }
    for (int r = tid; r < KP; r += nthr) {
        float s = HKM_INF;  // padding rows can never win
        if (r < K) {
            s = 0.f;
            const float* c = C + int64_t(r) * ldc;
            for (int d = 0; d < D; ++d) s = fmaf(c[d], c[d], s);
        }
        sCn[r] = s;
    }
    if (FUSED) {
        for (int i = tid; i < K * LDA; i += nthr) sA[i] = 0.0;
        for (int i = tid; i < K; i += nthr) sN[i] = 0;
        if (tid == 0) {
            sN[K] = 0x7fffffff;
            sN[K + 1] = -0x7fffffff;
        }
    }
    __syncthreads();

    const int lane = tid & 63, wave = tid >> 6, nw = nthr >> 6;
    const int p = lane & 31, h = lane >> 5;
    const int ncb = KP >> 5;
    const int64_t tile_rows = int64_t(nw) * PB * 32;
    int emin = 0x7fffffff, emax = -0x7fffffff;

    floatx4 bn[PB][NJ];
    auto fetch = [&](int64_t tile) {
        const int64_t row0 = tile * tile_rows + wave * (PB * 32);
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            int64_t r = row0 + pb * 32 + p;
            r = r < N ? r : N - 1;
            const float* xr = X + r * ldx;
#pragma unroll
            for (int j = 0; j < NJ; ++j) bn[pb][j] = load_row4<VEC>(xr, h * (DP / 2) + 4 * j, D);
        }
    };
    if (int64_t(blockIdx.x) < ntiles) fetch(blockIdx.x);

    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int64_t row0 = tile * tile_rows + wave * (PB * 32);
        floatx4 b[PB][NJ];
        uintx4 xs[PB][3][NS];
        float xnr[PB], m[PB];
        int mi[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                b[pb][j] = bn[pb][j];
#pragma unroll
                for (int t = 0; t < 4; ++t) s = fmaf(b[pb][j][t], b[pb][j][t], s);
            }
            xnr[pb] = s + __shfl_xor(s, 32);
#pragma unroll
            for (int st = 0; st < NS; ++st)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    // features 8 st + 2q, + 1 of this lane-half: group 2 st + q / 2, elements 2 (q % 2), + 1
                    const floatx4 g = b[pb][2 * st + (q >> 1)];
                    unsigned p1, p2, p3;
                    split_pair(g[2 * (q & 1)], g[2 * (q & 1) + 1], p1, p2, p3);
                    xs[pb][0][st][q] = p1;
                    xs[pb][1][st][q] = p2;
                    xs[pb][2][st][q] = p3;
                }
        }
        if (tile + gridDim.x < ntiles) fetch(tile + gridDim.x);

        split_scan<DP, false>(planes, plane_stride, sCn, ncb, p, h, xs, xnr, m, mi);
        bool neg = false;
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) neg |= m[pb] < 0.f;
        if (__any(neg)) split_scan<DP, true>(planes, plane_stride, sCn, ncb, p, h, xs, xnr, m, mi);

#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            mi[pb] += 4 * h;
            merge_halves(m[pb], mi[pb]);
            const int64_t r = row0 + pb * 32 + p;
            const bool valid = r < N;
            if (h == 0 && valid) {
                labels[r] = mi[pb];
                if (min_d2) min_d2[r] = m[pb];
                if (FUSED) atomicAdd(&sN[mi[pb]], 1);
            }
            if (FUSED && valid && xnr[pb] != 0.f) {  // an all-zero row adds nothing
                const int e2 = (__float_as_int(xnr[pb]) >> 23) - 127;
                const int E = (e2 >> 1) + 2;
                emin = min(emin, E);
                emax = max(emax, E);
                const double B = __hiloint2double(((1023 + 52 - SPLIT_QBITS + E) << 20) | 0x80000, 0);
                double* row = sA + size_t(mi[pb]) * LDA + h * (DP / 2);
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const double v = (double(b[pb][j][t]) + B) - B;
                        __hip_atomic_fetch_add(row + 4 * j + t, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
            }
        }
    }

    if (FUSED) {
        atomicMin(&sN[K], emin);
        atomicMax(&sN[K + 1], emax);
        __syncthreads();
        double* gs = fsum + size_t(blockIdx.x) * K * D;
        for (int i = tid; i < K * D; i += nthr) {
            const int k = i / D, d = i - k * D;
            gs[i] = sA[size_t(k) * LDA + d];
        }
        for (int i = tid; i < K; i += nthr) fcnt[size_t(blockIdx.x) * K + i] = sN[i];
        if (tid == 0) {
            const int lo = sN[K], hi = sN[K + 1];
            flags[blockIdx.x] = (hi >= lo && hi - lo > range_bits) ? 1 : 0;
        }
    }
}

// feature padding of the split kernels: whole k-steps of 16
int split_dp(int32_t D) { return D <= 32 ? 32 : D <= 48 ? 48 : 64; }

size_t split_lds_bytes(int32_t D, int32_t K, bool fused) {
    const size_t kp = (size_t(K) + 31) / 32 * 32;
    const int dp = split_dp(D);
    size_t b = size_t(3) * kp * split_ldb(dp) * 2 + kp * sizeof(float);
    if (fused) b += size_t(K) * (dp + 1) * sizeof(double) + (size_t(K) + 4) * sizeof(int);
    return b;
}

bool split_eligible(int32_t D, int32_t K, bool fused) {
    // up to 32 features for now: wider rows need more registers for the split point operands than
    // two waves per SIMD leave
    return D > 16 && D <= 32 && split_lds_bytes(D, K, fused) <= (fused ? size_t(160) : size_t(64)) * 1024;
}

int split_fused_grid(int64_t N) {
    constexpr int PB = 2;
    const int64_t tile_rows = int64_t(SPLIT_FUSED_THREADS / 64) * PB * 32;
    const int64_t ntiles = (N + tile_rows - 1) / tile_rows;
    int64_t grid = num_cus();
    if (grid > FUSED_MAX_GRID) grid = FUSED_MAX_GRID;
    if (grid > ntiles) grid = ntiles;
    return int(grid < 1 ? 1 : grid);
}

template <int DP, bool VEC, bool FUSED>
static int launch_split_t(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt,
                          int32_t* flags, hipStream_t st) {
    constexpr int PB = 2;
    const int threads = FUSED ? SPLIT_FUSED_THREADS : 256;
    const int64_t tile_rows = int64_t(threads / 64) * PB * 32;
    const int64_t ntiles = (N + tile_rows - 1) / tile_rows;
    int64_t grid = FUSED ? split_fused_grid(N) : int64_t(num_cus()) * 3;
    if (grid > ntiles) grid = ntiles;
    const size_t lds = split_lds_bytes(D, K, FUSED);
    auto kern = split_resident_kernel<DP, PB, VEC, FUSED>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return fail(HKM_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    const int64_t per_wg = (ntiles + grid - 1) / grid * tile_rows;
    int lg = 0;
    while ((int64_t(1) << lg) < per_wg) ++lg;
    const int range_bits = 53 - SPLIT_QBITS - lg;
    prof_begin(st);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(threads), lds, st, X, N, D, ldx, C, K, ldc, labels,
                       min_d2, ntiles, fsum, fcnt, flags, range_bits);
    prof_end(st);
    return check_launch("split_resident_kernel");
}

// fsum == NULL: distance + argmin only
int launch_split_resident(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt,
                          int32_t* flags, hipStream_t st) {
    const bool vec = aligned16(X) && (ldx % 4 == 0) && (D % 4 == 0);
    const int dp = split_dp(D);
    const bool fused = fsum != nullptr;
#define HKM_CASE(d)                                                                                              \
    case d:                                                                                                      \
        if (fused)                                                                                               \
            return vec ? launch_split_t<d, true, true>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, st)  \
                       : launch_split_t<d, false, true>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, st); \
        return vec ? launch_split_t<d, true, false>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, st)     \
                   : launch_split_t<d, false, false>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, st);
    switch (dp) {
        HKM_CASE(32)
        default:
            return fail(HKM_EUNSUPPORTED, "split_resident: D=%d", D);
    }
#undef HKM_CASE
}

}  // namespace hkm
