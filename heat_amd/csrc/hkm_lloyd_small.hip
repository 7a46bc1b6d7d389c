// One-sweep Lloyd step for small feature counts (D <= 16) and small K*(D+1): X is read from HBM
// exactly once per iteration (4D bytes per point) and only the labels are written (4 bytes).
//
// Assignment: a lane owns PPT consecutive points in registers; the centroids and their squared norms are
// wave-uniform operands -- LDS broadcasts of rows scaled by -2 (exact), or, where a row is one scalar load,
// scalar registers filled straight from C (scan_centroids_sload); 12 to 16 centroids of 4 or 8 coordinates
// are instead one A operand of v_mfma_f32_16x16x4_f32 and the minimum is found in registers after a
// transpose across the lanes (the matrix-core scan in the kernel body); a dozen or more centroids of up to
// 3 coordinates are taken four at a time (scan_centroids_blocked).  The quadratic expansion of
// heat/spatial/distance.py:59-64, d2 = |x|^2 + |c|^2 - 2 x.c, is evaluated as a chain of D fused
// multiply-adds that starts at |c|^2; |x|^2, the same for every centroid, is added to the minimum only.
// First index wins ties (torch.min, heat/core/statistics.py:177).  The clamp at 0 is applied lazily: a
// negative minimum (a point that coincides with a centroid up to rounding) triggers a rescan with the
// clamp applied to every candidate, so the result equals clamping first.
//
// Update (heat/cluster/kmeans.py:76-103), per-cluster sums whose value does not depend on the order in
// which the hardware happens to run things:
//   K*(D+1) <= 48 and D <= 8: every lane owns a private fp32 column per (cluster, coordinate) in LDS and adds
//     its own points in program order; the read-add-write round trips of a round are deferred to the
//     next round and interleaved with its arithmetic.  At the end lanes' columns are added in a fixed
//     fp64 tree.
//   otherwise, large N: every coordinate is added as a 64-bit integer, rint(x * 2^(32 - Ec)) with 2^Ec
//     the bound of the step's largest centroid coordinate, to one of several copies of an integer table
//     in LDS with ds_add_u64.  Integer addition is exact, so the atomics may land in any order; it costs
//     two vector instructions per coordinate, a fraction of the assignment.  A workgroup that meets a row
//     outside the scale's range (|x| >= 2^(Ec + headroom), inf, NaN) or has no usable scale raises a flag,
//     and a second launch -- the same sweep with one of the two ordered strategies below, which returns at
//     once when no flag is up -- redoes the step.
//   otherwise, K <= 32 and D <= 8: the sums are a matrix product, (one-hot labels)^T x [X, 1], evaluated on the
//     fp32 matrix cores with v_mfma_f32_16x16x4_f32 over the wave's points of the round (read back from
//     the staging buffer); the fp32 accumulators move into the wave's private fp64 row in LDS every
//     eight rounds.
//   otherwise: for every cluster k and coordinate d the wavefront forms
//     sum over lanes of [label == k] * x_d with a fixed DPP tree (row shifts, then row broadcasts;
//     the total lands in lane 63) and lane 63 adds it to the wave's private fp64 row in LDS.
// Either way the workgroup writes one fp64 partial row; a single-workgroup kernel adds the rows in a
// fixed order, divides by the count (rounded through fp32 like the reference,
// heat/core/rounding.py:156-164) and computes the centroid shift (kmeans.py:141).
#include <type_traits>

#include "hkm_common.h"
#include "hkm_mfma_util.h"

// Fewest centroids for which the matrix-core scan of the narrow kernel is used (8 / 4 coordinates).  Its cost
// does not depend on K and equals that of the vector scan over 11 to 12 centroids (50M rows, kernel without
// label stores, 8 coordinates: 0.345-0.352 ms whatever K is, against 0.342 / 0.358 / 0.370 ms of the vector
// scan at K = 11 / 12 / 13; 4 coordinates: 0.222 against 0.219 / 0.231 ms at K = 12 / 13).
#ifndef HKM_MSCAN_MIN_K8
#define HKM_MSCAN_MIN_K8 12
#endif
#ifndef HKM_MSCAN_MIN_K4
#define HKM_MSCAN_MIN_K4 13
#endif

namespace hkm {

// STREAM: the matrix is larger than the last-level cache, so its lines are not worth keeping there.  A template
// parameter: a run-time choice between a non-temporal and a plain load of one address is compiled into a single
// plain load.
template <bool STREAM>
__device__ __forceinline__ floatx4 ldg4(const float* p) {
    const floatx4* q = reinterpret_cast<const floatx4*>(p);
    if constexpr (STREAM) return __builtin_nontemporal_load(q);
    else return *q;
}

template <int D>
struct SmallCfg {
    // points per lane so that a lane's chunk is a whole number of 16-byte vectors
    static constexpr int PPT = (D % 4 == 0) ? 2 : (D % 2 == 0) ? 2 : 4;
    static constexpr int SC = (D + 1 + 3) / 4 * 4;  // LDS centroid row: D coords, |c|^2, pad
    // Centroid rows by scalar loads instead of LDS broadcasts, where a row is ONE scalar load (1, 4 or 8
    // values): measured on 30-100 M rows with 16-100 clusters, the step is then 4-26 % faster; rows of
    // 2, 3, 5 or 7 values take several loads per centroid and run 6-10 % slower that way.
    static constexpr bool SLOAD = D == 1 || D == 4 || D == 8;
    // Up to 16 centroids of 4 or 8 coordinates are one A operand of v_mfma_f32_16x16x4_f32 (one or two steps
    // over the coordinates): the cross terms of 16 points then cost one or two matrix instructions.
    static constexpr bool MSCAN = D == 4 || D == 8;
    // The scan four centroids at a time, where a centroid row is one 16-byte LDS read: the assignment of
    // 100M rows takes 1.39 instead of 2.05 ms with 1 coordinate and 100 centroids, 0.66 instead of 1.01 ms
    // with 2 and 64, 0.53 instead of 0.67 ms with 3 and 40; from a dozen centroids on it is never slower.
    // Rows of 5 to 7 coordinates (two reads per row, more registers) run 0-18 % slower that way.
    static constexpr bool BLOCKED = D <= 3;
    // The wave's staging buffer holds a round as 64 rows, one per lane, of the lane's PPT points (RL floats); the
    // rows are RLP floats apart, a multiple of 4 whose quarter is odd: the 16 lanes that read 16 bytes each
    // together then meet no LDS bank twice (with rows of 16 floats back to back they met four times, with 32 eight
    // times).  Point q of the round starts at stage_off(q).
    static constexpr int RL = PPT * D;
    static constexpr int RLP = (RL / 4) % 2 == 1 ? RL : RL + 4;
    static constexpr int stage_off(int q) { return (q / PPT) * RLP + (q % PPT) * D; }
};

bool small_eligible(int32_t D, int32_t K) { return D <= 16 && K * (D + 1) <= 240; }
static constexpr int SMALL_T = 256;

// ---- the integer accumulation (acc_mode 4) ----
// A coordinate is added as the integer rint(x * 2^(QB - Ec)), where 2^Ec bounds the largest centroid
// coordinate of the step: integer additions are exact, so LDS atomics may deliver them in any order.
static constexpr int SMALL_QB = 32;
// copies of every accumulator per workgroup (a lane uses copy lane % R): fewer lanes of one instruction
// meet at one address, and with the copies side by side none in a bank more than their share
__host__ __device__ constexpr int small_replicas(int K) { return K <= 16 ? 16 : K <= 32 ? 8 : 4; }
// entries per cluster row of the table
__host__ __device__ constexpr int small_int_stride(int D) { return D + 1; }

// LDS of one workgroup; acc_mode as in the kernel (0 labels only, 1 lane columns, 2 wave rows by the
// DPP tree, 3 wave rows by the matrix cores, 4 integer tables)
static size_t small_lds_bytes(int32_t D, int32_t K, int acc_mode) {
    const int ppt = (D % 2 == 0) ? 2 : 4;
    const int sc = (D + 1 + 3) / 4 * 4, rl = ppt * D, rlp = (rl / 4) % 2 == 1 ? rl : rl + 4, slots = K * (D + 1);  // as SmallCfg
    const size_t xch = (D == 4 || D == 8) ? size_t(SMALL_T / 64) * 256 * sizeof(float) : 0;  // as SmallCfg::MSCAN
    return size_t(((K + 3) & ~3) * sc) * sizeof(float) + size_t(SMALL_T / 64) * 64 * rlp * sizeof(float) + xch +
           (acc_mode == 2   ? size_t(SMALL_T / 64) * slots * sizeof(double)
            : acc_mode == 3 ? size_t(SMALL_T / 64) * (slots * sizeof(double) + 64 * ppt * sizeof(int))
            : acc_mode == 1 ? size_t(slots + D + 1) * SMALL_T * sizeof(float)
            : acc_mode == 4 ? size_t(small_replicas(K)) * K * small_int_stride(D) * 8 + 16
                            : 0);
}
// The ordered strategies: per-lane LDS columns while they fit (slots * 1 KB), the matrix-core product up
// to 32 clusters, the DPP tree otherwise.
static int small_ordered_mode(int32_t D, int32_t K) { return D > 8 ? 2 : K * (D + 1) <= 48 ? 1 : K <= 32 ? 3 : 2; }

// Fewest centroids for which the scan goes four at a time (HKM_SMALL_BLOCKED_MIN_K overrides; looked up per call)
static int small_blocked_min_k() {
    const char* e = getenv("HKM_SMALL_BLOCKED_MIN_K");
    return e ? atoi(e) : 12;
}

// HKM_SMALL_SUMS = ordered | integer (looked up per call) overrides the choice by size; tests use it
static int small_sums_override() {
    const char* e = getenv("HKM_SMALL_SUMS");
    if (!e) return 0;
    return e[0] == 'o' ? 1 : e[0] == 'i' ? 2 : 0;
}

// Beyond 48 slots the ordered strategies cost more than the assignment itself; the integer tables cost a
// fraction of it but need a second launch (a re-run in the ordered way that normally returns at once), so
// they start where a launch no longer shows: from 2^20 rows where the ordered way is the matrix-core
// product, from 2^17 where it is the wave-wide tree (more than 32 clusters or more than 8 features:
// 1M x 16, 14 clusters: 0.039 against 0.075 ms per step; 500k x 16, 8: 0.026 against 0.033 ms).
bool small_integer_sums(int64_t N, int32_t D, int32_t K) {
    if (K * (D + 1) <= 48) return false;
    const int o = small_sums_override();
    if (o) return o == 2;
    return N >= ((K > 32 || D > 8) ? (int64_t(1) << 17) : (int64_t(1) << 20));
}
static int small_acc_mode(int64_t N, int32_t D, int32_t K) {
    return small_integer_sums(N, D, K) ? 4 : small_ordered_mode(D, K);
}

int small_grid(int64_t N, int32_t D, int32_t K) {
    const int ppt = (D % 2 == 0) ? 2 : 4;
    const int64_t groups = (N + ppt - 1) / ppt;
    // one group per lane until every CU holds as many workgroups as fit (4 by registers, fewer if the
    // accumulating variant's LDS says so: a grid beyond that would run in two uneven batches), then
    // grid-stride
    int64_t want = (groups + SMALL_T - 1) / SMALL_T;
    int64_t per_cu = int64_t(160 * 1024) / int64_t(small_lds_bytes(D, K, small_acc_mode(N, D, K)));
    if (per_cu > 4) per_cu = 4;
    if (per_cu < 1) per_cu = 1;
    int64_t cap = int64_t(num_cus()) * per_cu;
    if (cap > SMALL_MAX_GRID) cap = SMALL_MAX_GRID;
    if (want > cap) want = cap;
    if (want < 1) want = 1;
    return int(want);
}

// Exchanges between the four rows of 16 lanes of a wave (one instruction each): rows 2, 3 of a with rows 0, 1
// of b; odd rows of a with even rows of b.
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void lane_rows_swap32(float& a, float& b) {
    const uintx2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void lane_rows_swap16(float& a, float& b) {
    const uintx2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
}

// sum over the 64 lanes with a fixed tree; the total is valid in lane 63
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
#define HKM_DPP_ADD(ctrl, rmask, bmask)                                                              \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, \
                                                               rmask, bmask, true))
    HKM_DPP_ADD(0x111, 0xf, 0xf);  // row_shr:1
    HKM_DPP_ADD(0x112, 0xf, 0xf);  // row_shr:2
    HKM_DPP_ADD(0x114, 0xf, 0xf);  // row_shr:4
    HKM_DPP_ADD(0x118, 0xf, 0xf);  // row_shr:8  -> lane 15 of each row holds the row sum
    HKM_DPP_ADD(0x142, 0xa, 0xf);  // row_bcast:15 into rows 1 and 3
    HKM_DPP_ADD(0x143, 0xc, 0xf);  // row_bcast:31 into rows 2 and 3
#undef HKM_DPP_ADD
    return v;
}

template <int D, int PPT, bool CLAMP>
__device__ __forceinline__ void scan_centroids(const float* sC, int k0, int k1,
                                               const float (&x)[PPT][D], const float (&xn)[PPT],
                                               float (&m)[PPT], int (&mi)[PPT]) {
    constexpr int SC = SmallCfg<D>::SC;
#pragma unroll 2
    for (int k = k0; k < k1; ++k) {
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
            // c holds -2*c_k and |c_k|^2: the chain ends as |c|^2 - 2 x.c, D instructions per distance
            float dist = fmaf(x[p][0], c[0], c[D]);
#pragma unroll
            for (int d = 1; d < D; ++d) dist = fmaf(x[p][d], c[d], dist);
            if (CLAMP) dist = fmaxf(dist + xn[p], 0.0f);
            mi[p] = dist < m[p] ? k : mi[p];
            m[p] = fminf(m[p], dist);
        }
    }
}

// The scan for more than a few centroids, four at a time: the running minimum absorbs a block's four
// distances with two three-input minima, and of the block only its number is kept where the minimum fell
// (one compare, one select) -- 4 instead of 12 instructions per four distances besides the products.
// Which of the four it was is looked up once per point at the end: the lane reads the four rows of ITS
// block from LDS, evaluates the same chains again (same operands, same order: same bits) and takes the
// first that equals the minimum.  Strict '<' on blocks and the first equal position inside one give the
// first centroid that reaches the minimum, as the one-by-one scan does; NaN distances are skipped by the
// minima, and a point with nothing below +inf keeps index 0.  Rows K .. 4 * ceil(K / 4) - 1 of sC hold
// zero coordinates and the norm +inf.  m must come in as +inf.
template <int D, int PPT>
__device__ __forceinline__ void scan_centroids_blocked(const float* sC, int K, const float (&x)[PPT][D],
                                                       float (&m)[PPT], int (&mi)[PPT]) {
    constexpr int SC = SmallCfg<D>::SC;
    int blk[PPT];
#pragma unroll
    for (int p = 0; p < PPT; ++p) blk[p] = 0;
    const int nb = (K + 3) >> 2;
    for (int b = 0; b < nb; ++b) {
        float dist[4][PPT];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float c[SC];
#pragma unroll
            for (int q = 0; q < SC / 4; ++q) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(sC + (4 * b + j) * SC + 4 * q);
                c[4 * q] = v[0];
                c[4 * q + 1] = v[1];
                c[4 * q + 2] = v[2];
                c[4 * q + 3] = v[3];
            }
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                float d2 = fmaf(x[p][0], c[0], c[D]);
#pragma unroll
                for (int d = 1; d < D; ++d) d2 = fmaf(x[p][d], c[d], d2);
                dist[j][p] = d2;
            }
        }
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            const float nm = fminf(fminf(fminf(fminf(dist[0][p], dist[1][p]), dist[2][p]), dist[3][p]), m[p]);
            blk[p] = nm < m[p] ? b : blk[p];
            m[p] = nm;
        }
    }
#pragma unroll
    for (int p = 0; p < PPT; ++p) {
        const float* cb = sC + blk[p] * (4 * SC);
        int pos = 0;
#pragma unroll
        for (int j = 3; j >= 0; --j) {
            float c[SC];
#pragma unroll
            for (int q = 0; q < SC / 4; ++q) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(cb + j * SC + 4 * q);
                c[4 * q] = v[0];
                c[4 * q + 1] = v[1];
                c[4 * q + 2] = v[2];
                c[4 * q + 3] = v[3];
            }
            float d2 = fmaf(x[p][0], c[0], c[D]);
#pragma unroll
            for (int d = 1; d < D; ++d) d2 = fmaf(x[p][d], c[d], d2);
            pos = d2 == m[p] ? j : pos;
        }
        mi[p] = m[p] < HKM_INF ? 4 * blk[p] + pos : 0;
    }
}

// The same scan with the centroid rows fetched straight from the caller's C at wave-uniform addresses:
// the compiler turns such reads into scalar loads, so a row arrives in scalar registers through the scalar
// cache and costs neither LDS bandwidth (a broadcast read still returns 64 copies) nor vector registers.
// The rows in C carry no factor -2, so the chain runs on t = x.c - |c|^2 / 2 and looks for the LARGEST t:
// every intermediate value is the other chain's divided by -2 (a power of two commutes with rounding), so
// the comparisons, the ties and -2 t_max = the minimum are the same bits.  |c|^2 still comes from LDS.
template <int D, int PPT, bool CLAMP>
__device__ __forceinline__ void scan_centroids_sload(const float* __restrict__ C, int64_t ldc, const float* sC,
                                                     int k0, int k1, const float (&x)[PPT][D],
                                                     const float (&xn)[PPT], float (&m)[PPT], int (&mi)[PPT]) {
    constexpr int SC = SmallCfg<D>::SC;
    // m is a minimum of distances on entry and on return; in between the plain scan tracks the largest t
    // (= m / -2, exact both ways), the clamped one the smallest clamped distance
    float best[PPT];
#pragma unroll
    for (int p = 0; p < PPT; ++p) best[p] = CLAMP ? m[p] : -0.5f * m[p];
    constexpr int UNROLL_K = PPT == 2 ? 4 : 2;  // centroid rows in flight: bounded by the scalar registers
#pragma unroll UNROLL_K
    for (int k = k0; k < k1; ++k) {
        const float* ck = C + int64_t(k) * ldc;
        float c[D];
#pragma unroll
        for (int d = 0; d < D; ++d) c[d] = ck[d];
        const float hcn = -0.5f * sC[k * SC + D];
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            float t = fmaf(x[p][0], c[0], hcn);
#pragma unroll
            for (int d = 1; d < D; ++d) t = fmaf(x[p][d], c[d], t);
            if (CLAMP) {
                const float dist = fmaxf(fmaf(-2.0f, t, xn[p]), 0.0f);
                mi[p] = dist < best[p] ? k : mi[p];
                best[p] = fminf(best[p], dist);
            } else {
                mi[p] = t > best[p] ? k : mi[p];
                best[p] = fmaxf(best[p], t);
            }
        }
    }
#pragma unroll
    for (int p = 0; p < PPT; ++p) m[p] = CLAMP ? best[p] : -2.0f * best[p];
}

// The same scan with the centroids in registers that are uniform over the wave (KT rows, those
// beyond K hold |c|^2 = +inf and never win): no LDS reads and no loop in the round.
template <int D, int PPT, int KT, bool CLAMP>
__device__ __forceinline__ void scan_centroids_reg(const float (&cs)[KT][D + 1], int k0, int k1,
                                                   const float (&x)[PPT][D], const float (&xn)[PPT],
                                                   float (&m)[PPT], int (&mi)[PPT]) {
#pragma unroll
    for (int k = k0; k < k1; ++k) {
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            float dist = fmaf(x[p][0], cs[k][0], cs[k][D]);
#pragma unroll
            for (int d = 1; d < D; ++d) dist = fmaf(x[p][d], cs[k][d], dist);
            if (CLAMP) dist = fmaxf(dist + xn[p], 0.0f);
            mi[p] = dist < m[p] ? k : mi[p];
            m[p] = fminf(m[p], dist);
        }
    }
}

// ACC: 0 = labels only, 1 = per-lane private LDS columns, 2 = DPP wave tree + per-wave fp64 rows,
//      3 = matrix-core product (one-hot labels x points) + per-wave fp64 rows,
//      4 = integer tables in LDS, added to with atomics
// KT: 0 = centroid rows fetched in a loop over K; otherwise K <= KT and they sit in registers
// flags / aux: ACC == 4 writes flags[workgroup] = 1 if its sums cannot be trusted (a row too large for the
//   integer scale, or no usable scale), aux = how many bits above the largest centroid coordinate a row
//   may reach.  The ordered modes, given flags, are the re-run after an ACC == 4 launch of aux workgroups:
//   they return at once unless one of those raised its flag.
template <int D, int ACC, bool WANT_MIN, bool WANT_SSE, int KT, bool STREAM>
__global__ __launch_bounds__(SMALL_T) void lloyd_small_kernel(
    const float* __restrict__ X, int64_t N, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, int32_t* __restrict__ labels, float* __restrict__ min_d2,
    double* __restrict__ part, int vec, int32_t* __restrict__ flags, int aux) {
    constexpr int T = SMALL_T;
    constexpr int PPT = SmallCfg<D>::PPT;
    constexpr int SC = SmallCfg<D>::SC;
    constexpr int NV = PPT * D / 4;  // 16-byte vectors per lane
    constexpr int NW = T / 64;
    extern __shared__ __align__(16) float lds[];
    float* sC = lds;  // [K][SC]
    const int slots = K * (D + 1);
    constexpr bool ACCUM = ACC != 0;
    const int KP = (K + 3) & ~3;                                     // rows of sC: K, then +inf-norm rows up to a multiple of four
    constexpr int RL = SmallCfg<D>::RL, RLP = SmallCfg<D>::RLP;
    float* stage = lds + KP * SC;                                    // [NW][64][RLP] transpose buffer
    // matrix-core scan: [NW][128] (minimum, index) pairs on their way from the lane that found them to the
    // lane that owns the point
    float* xch_all = stage + NW * 64 * RLP;
    float* after = xch_all + (SmallCfg<D>::MSCAN ? NW * 256 : 0);
    double* wacc_all = reinterpret_cast<double*>(after);             // ACC==2: [NW][slots]
    float* cols = after;                                             // ACC==1: [slots][T]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    double* wacc = wacc_all + wave * slots;
    // ACC == 4: [K][LDI][R] 64-bit integers (column D of a row counts its points; the R copies of an entry
    // lie side by side, so a lane's copy -- lane mod R -- decides its LDS bank and the 64 lanes of an
    // instruction spread evenly over the banks whatever their labels are), then the bits of the largest
    // |centroid coordinate| and the workgroup's flag
    constexpr int LDI = small_int_stride(D);
    const int nrep = small_replicas(K);
    unsigned long long* iacc = reinterpret_cast<unsigned long long*>(after);
    int* imeta = reinterpret_cast<int*>(iacc + nrep * K * LDI);
    if ((ACC == 2 || ACC == 3) && flags) {
        int any = 0;
        for (int g = tid; g < aux; g += T) any |= flags[g];
        if (!__syncthreads_or(any)) return;
    }
    int* wlab = reinterpret_cast<int*>(wacc_all + NW * slots) + wave * (64 * PPT);  // ACC==3: [4][16*PPT]
    float* wstage = stage + wave * 64 * RLP;

    const int64_t groups = (N + PPT - 1) / PPT;
    const int64_t full = (vec & 1) ? N / PPT : 0;  // groups served by the 16-byte vector path
    const int64_t stride = int64_t(gridDim.x) * T;
    const int64_t wg0 = int64_t(blockIdx.x) * T;
    int64_t base = wg0;
    // A wave's 64 groups are NV*1024 contiguous bytes: fetched as NV fully coalesced 16-byte
    // loads per lane, then redistributed through a wave-private LDS buffer so that every lane
    // ends up with its own PPT consecutive points.  The first rounds are requested here, before the
    // centroids are staged: for a matrix of a few megabytes the kernel is two memory latencies long,
    // and this way they overlap.
    // rounds in flight: enough bytes per CU to cover the HBM latency, within the registers a wide row leaves
    constexpr int PF = NV <= 4 ? 3 : NV <= 8 ? 2 : 1;
    floatx4 nxt[PF][NV];
    const float* wsrc = X + (base + wave * 64) * (PPT * D) + lane * 4;
    const int64_t rstride = stride * (PPT * D);
#pragma unroll
    for (int f = 0; f < PF; ++f) {
        if (base + f * stride + T <= full) {
#pragma unroll
            for (int v = 0; v < NV; ++v) nxt[f][v] = ldg4<STREAM>(wsrc + f * rstride + v * 256);
        }
    }

    for (int i = tid; i < K * SC; i += T) {
        const int r = i / SC, c = i - r * SC;
        sC[i] = c < D ? C[int64_t(r) * ldc + c] : 0.f;  // scaled by -2 once the norms are taken
    }
    if (ACC == 2 || ACC == 3)
        for (int i = tid; i < NW * slots; i += T) wacc_all[i] = 0.0;
    if (ACC == 1)
        for (int i = tid; i < (slots + D + 1) * T; i += T) cols[i] = 0.f;
    if (ACC == 4) {
        for (int i = tid; i < nrep * K * LDI; i += T) iacc[i] = 0ull;
        if (tid < 2) imeta[tid] = 0;
    }
    __syncthreads();
    if (ACC == 4) {
        // bits of non-negative floats order like integers; NaN and inf end up on top
        int mx = 0;
        for (int i = tid; i < K * SC; i += T) mx = max(mx, __float_as_int(sC[i]) & 0x7fffffff);
        atomicMax(&imeta[0], mx);
        __syncthreads();  // the scaling below overwrites what the maximum was taken of
    }
    for (int r = tid; r < K; r += T) {
        float s = 0.f;
#pragma unroll
        for (int d = 0; d < D; ++d) s = __fadd_rn(s, __fmul_rn(sC[r * SC + d], sC[r * SC + d]));
        sC[r * SC + D] = s;
#pragma unroll
        for (int d = 0; d < D; ++d) sC[r * SC + d] *= -2.0f;  // exact
    }
    for (int i = K * SC + tid; i < KP * SC; i += T) sC[i] = (i % SC) == D ? HKM_INF : 0.f;
    __syncthreads();

    // ACC == 4: 2^Ec > every |centroid coordinate|.  A coordinate x enters as the 64-bit pattern of
    // fma(x, 2^(QB - Ec), 1.5 * 2^52): for |x| < 2^(Ec + 51 - QB) that is the pattern of the constant plus
    // the integer rint(x * 2^(QB - Ec)), so the sum of n patterns minus n times the constant's is the exact
    // sum of the integers (all modulo 2^64; the true sum fits because aux also accounts for the number of
    // rows a workgroup adds).  A row is inside the range if |x|^2 < 2^(2 (Ec + aux)).
    double iscale = 0.0, iquantum = 0.0;
    float xn_limit = 0.f;
    bool bad = false;
    if (ACC == 4) {
        const int ebits = (imeta[0] >> 23) & 0xff;
        const int Ec = ebits - 127 + 1;
        bad = ebits == 0 || ebits == 255;  // all centroids zero (or denormal), or a non-finite one: no scale
        iscale = __hiloint2double((1023 + SMALL_QB - Ec) << 20, 0);
        iquantum = __hiloint2double((1023 - SMALL_QB + Ec) << 20, 0);
        const int e2 = 2 * (Ec + aux);
        xn_limit = e2 > 127 ? HKM_INF : e2 < -126 ? 0.f : __int_as_float((e2 + 127) << 23);
    }

    // 0 < KT <= 8: one copy of the centroid table per wave, in scalar registers
    // KT = 16 / 32 (ACC == 3 only): one / two blocks of 16 clusters in the matrix-core accumulation
    constexpr bool REGC = KT > 0 && KT <= 8;
    constexpr int KR = REGC ? KT : 1;
    constexpr int MB = KT == 32 ? 2 : 1;
    float cs[KR][D + 1];
    if (REGC) {
#pragma unroll
        for (int k = 0; k < KR; ++k)
#pragma unroll
            for (int d = 0; d <= D; ++d) {
                const float v = k < K ? sC[k * SC + d] : (d == D ? HKM_INF : 0.f);
                cs[k][d] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
            }
    }

    // The matrix-core scan (K <= 16, D = 4 or 8, PPT = 2): 16 points x 16 centroids per v_mfma_f32_16x16x4_f32,
    // one instruction per four coordinates.  A = the centroid table (lane: row lane % 16, coordinate 4 s +
    // lane / 16 of -2c; rows beyond K are zero), held in registers for the whole kernel; C = |c|^2 of the four
    // rows 4 (lane / 16) + r the lane's results belong to (+inf beyond K: never the minimum); B = 16 points
    // read back from the staging buffer.
    constexpr bool MSCAN = SmallCfg<D>::MSCAN && !REGC;
    const bool mscan = MSCAN && K <= 16 && K >= (D == 8 ? HKM_MSCAN_MIN_K8 : HKM_MSCAN_MIN_K4);
    float ma[MSCAN ? D / 4 : 1];
    floatx4 mcn = {HKM_INF, HKM_INF, HKM_INF, HKM_INF};
    if (mscan) {
        const int i = lane & 15, kk = lane >> 4;
#pragma unroll
        for (int st = 0; st < D / 4; ++st) ma[st] = i < K ? sC[i * SC + 4 * st + kk] : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (4 * kk + r < K) mcn[r] = sC[(4 * kk + r) * SC + D];
    }
    float* xch = xch_all + wave * 256;

    double sse = 0.0;

    // ACC == 1: the additions of a round are deferred to the NEXT round and interleaved with its
    // arithmetic, so that the LDS read -> add -> write round trips of the PPT points (which must stay
    // sequential: two points of a lane may share a cluster) hide behind independent work.  A lane's
    // pending points live in pcol (column offset of their cluster, or of a dummy cluster that
    // collects nothing useful) and px.
    const int dummy_col = slots * T + tid;
    int pcol[PPT];
    float px[PPT][D + 1];
#pragma unroll
    for (int p = 0; p < PPT; ++p) {
        pcol[p] = dummy_col;
#pragma unroll
        for (int d = 0; d <= D; ++d) px[p][d] = 0.f;
    }
    auto rmw_read = [&](int p, float (&r)[D + 1]) {
#pragma unroll
        for (int d = 0; d <= D; ++d) r[d] = cols[pcol[p] + d * T];
    };
    auto rmw_write = [&](int p, const float (&r)[D + 1]) {
#pragma unroll
        for (int d = 0; d <= D; ++d) cols[pcol[p] + d * T] = r[d] + px[p][d];
    };

    // ACC == 3: fp32 accumulators of the matrix-core product (lane: cluster rows 4*(lane/16) + r of
    // block mb, column lane%16), moved into the wave's fp64 row every eight rounds (1024 points at
    // most in fp32) -- every (cluster, column) has one owner, so plain read-add-write.
    floatx4 macc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) macc[mb] = floatx4{0.f, 0.f, 0.f, 0.f};
    int since_flush = 0;
    auto flush_macc = [&]() {
        const int col = lane & 15;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * mb + 4 * (lane >> 4) + r;
                if (row < K && col <= D) wacc[row * (D + 1) + col] += double(macc[mb][r]);
                macc[mb][r] = 0.f;
            }
        since_flush = 0;
    };

    // label + accumulate one group of PPT points held in registers.  Executed by ALL lanes of the
    // wave (the DPP tree needs them); GUARD: rows >= N contribute nothing and store nothing.
    auto process = [&](int64_t i0, const float (&x)[PPT][D], auto guard_tag) {
        constexpr bool GUARD = decltype(guard_tag)::value;
        float xn[PPT], m[PPT];
        int mi[PPT];
        float r[D + 1];
        if (ACC == 1) rmw_read(0, r);
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) s = __fadd_rn(s, __fmul_rn(x[p][d], x[p][d]));
            xn[p] = s;
            m[p] = HKM_INF;
            mi[p] = 0;
        }
        const int kh = REGC ? KT / 2 : K >> 1;
        const bool blocked = !REGC && SmallCfg<D>::BLOCKED && (vec & 4) != 0;
        if (ACC == 1 && PPT == 4) {
            rmw_write(0, r);
            rmw_read(1, r);
        }
        bool scanned = false;
        if constexpr (MSCAN) {
            if (mscan) {
                scanned = true;
                // The wave's 128 points of the round sit in the staging buffer as rows; 64 at a time, four
                // groups of 16 go through the matrix cores.  A lane then holds, of each group, the distances
                // of point lane % 16 to centroids 4 (lane / 16) + r; two swaps of lane rows per register
                // (across the halves of the wave, then between neighbouring rows) transpose that, so that
                // lane 16 g + n ends up with all sixteen distances of point n of group g, in centroid order.
                const float* brow = wstage + SmallCfg<D>::stage_off(lane & 15) + (lane >> 4);  // (16 j, 64 half: whole rows)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    floatx4 acc[4];
                    float bv[4][D / 4];  // all requested before the first matrix instruction waits for one
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int st = 0; st < D / 4; ++st) bv[j][st] = brow[SmallCfg<D>::stage_off(half * 64 + 16 * j) + 4 * st];
                    wave_lds_sync();
#pragma unroll
                    for (int st = 0; st < D / 4; ++st)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ma[st], bv[j][st], st == 0 ? mcn : acc[j], 0, 0, 0);
                    float dk[4][4];  // [group -> centroid quad after the transpose][r]
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) dk[j][q] = acc[j][q];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        lane_rows_swap32(dk[0][q], dk[2][q]);
                        lane_rows_swap32(dk[1][q], dk[3][q]);
                        lane_rows_swap16(dk[0][q], dk[1][q]);
                        lane_rows_swap16(dk[2][q], dk[3][q]);
                    }
                    floatx16 dv;
#pragma unroll
                    for (int k = 0; k < 16; ++k) dv[k] = dk[k >> 2][k & 3];
                    const float best = block_min16(dv);
                    const int pos = block_pos16(dv, best);  // 8 * (k / 4) + k % 4 for the first k that holds it
                    const int idx = (pos & 3) | ((pos >> 3) << 2);
                    // nothing below +inf (all distances inf or NaN): index 0, as the running scan leaves it
                    const bool any = best < HKM_INF;
                    float2 out;
                    out.x = any ? best : HKM_INF;
                    out.y = __int_as_float(any ? idx : 0);
                    reinterpret_cast<float2*>(xch)[half * 64 + lane] = out;
                }
                wave_lds_sync();
                const floatx4 mine = reinterpret_cast<const floatx4*>(xch)[lane];  // points 2 lane, 2 lane + 1
                wave_lds_sync();
                m[0] = mine[0];
                mi[0] = __float_as_int(mine[1]);
                m[PPT - 1] = mine[2];
                mi[PPT - 1] = __float_as_int(mine[3]);
            }
        }
        if (!scanned) {
            if constexpr (!REGC && SmallCfg<D>::BLOCKED) {
                if (blocked) scan_centroids_blocked<D, PPT>(sC, K, x, m, mi);
            }
            if (!blocked) {
                if constexpr (REGC) scan_centroids_reg<D, PPT, KR, false>(cs, 0, KR / 2, x, xn, m, mi);
                else if constexpr (SmallCfg<D>::SLOAD) scan_centroids_sload<D, PPT, false>(C, ldc, sC, 0, kh, x, xn, m, mi);
                else scan_centroids<D, PPT, false>(sC, 0, kh, x, xn, m, mi);
            }
        }
        if (ACC == 1) {
            rmw_write(PPT == 4 ? 1 : 0, r);
            rmw_read(PPT == 4 ? 2 : 1, r);
        }
        if (!scanned && !blocked) {
            if constexpr (REGC) scan_centroids_reg<D, PPT, KR, false>(cs, KR / 2, KR, x, xn, m, mi);
            else if constexpr (SmallCfg<D>::SLOAD) scan_centroids_sload<D, PPT, false>(C, ldc, sC, kh, K, x, xn, m, mi);
            else scan_centroids<D, PPT, false>(sC, kh, K, x, xn, m, mi);
        }
        if (ACC == 1 && PPT == 4) {
            rmw_write(2, r);
            rmw_read(3, r);
        }
        // |x|^2 is the same for every centroid: it joins the minimum only
        bool neg = false;
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            m[p] += xn[p];
            neg |= (m[p] < 0.f);
        }
        if (__any(neg)) {
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                m[p] = HKM_INF;
                mi[p] = 0;
            }
            if constexpr (REGC) scan_centroids_reg<D, PPT, KR, true>(cs, 0, KR, x, xn, m, mi);
            else if constexpr (SmallCfg<D>::SLOAD) scan_centroids_sload<D, PPT, true>(C, ldc, sC, 0, K, x, xn, m, mi);
            else scan_centroids<D, PPT, true>(sC, 0, K, x, xn, m, mi);
        }

        // labels == NULL: the caller only wants the sums (a fit needs the labels of its last
        // iteration only and can recompute those)
        // (vec & 8: `labels` points to 64-bit integers, the type the reference returns its labels in)
        const bool lab64 = (vec & 8) != 0;
        if constexpr (!GUARD) {
            if (labels && lab64) {
                longlong2* out = reinterpret_cast<longlong2*>(reinterpret_cast<long long*>(labels) + i0);
#pragma unroll
                for (int q = 0; q < PPT / 2; ++q) out[q] = make_longlong2(mi[2 * q], mi[2 * q + 1]);
            } else if (labels) {
                if constexpr (PPT == 4) {
                    *reinterpret_cast<int4*>(labels + i0) = make_int4(mi[0], mi[1], mi[2], mi[3]);
                } else {
                    *reinterpret_cast<int2*>(labels + i0) = make_int2(mi[0], mi[1]);
                }
            }
        }
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            const bool ok = !GUARD || i0 + p < N;
            if (ok) {
                if (GUARD && labels) {
                    if (lab64) reinterpret_cast<long long*>(labels)[i0 + p] = mi[p];
                    else labels[i0 + p] = mi[p];
                }
                if (WANT_MIN) min_d2[i0 + p] = m[p];
                if (WANT_SSE) sse += double(m[p]);
            } else {
                mi[p] = -1;  // matches no cluster below
            }
        }
        if (ACC == 1) {
            rmw_write(PPT - 1, r);
            // this round's points become the pending ones
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                pcol[p] = (GUARD && mi[p] < 0) ? dummy_col : (mi[p] * (D + 1)) * T + tid;
#pragma unroll
                for (int d = 0; d < D; ++d) px[p][d] = x[p][d];
                px[p][D] = 1.0f;
            }
        }
        if (ACC == 4) {
            const double magic = __hiloint2double(0x43380000, 0);  // 1.5 * 2^52
            const int rep = lane & (nrep - 1);
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                bad |= !(xn[p] < xn_limit);  // too large for the scale, or not finite
                if (!GUARD || mi[p] >= 0) {
                    unsigned long long* row = iacc + mi[p] * (LDI * nrep) + rep;
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        const double t = fma(double(x[p][d]), iscale, magic);
                        __hip_atomic_fetch_add(row + d * nrep, (unsigned long long)__double_as_longlong(t), __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                    __hip_atomic_fetch_add(row + D * nrep, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        }
        if (ACC == 3) {
            // Per-cluster sums as a matrix product on the fp32 matrix cores: (one-hot labels, 16 x 4
            // points) x (4 points x [coordinates, 1]) per v_mfma_f32_16x16x4_f32, accumulated over the
            // wave's 64*PPT points of the round.  The points are read back from the wave's staging
            // buffer (row q = point q of the round), the labels go through LDS transposed so that a
            // lane fetches those of four steps at once.
            constexpr int G = 16 * PPT;  // MFMA steps per round
#pragma unroll
            for (int p = 0; p < PPT; ++p) {
                const int q = lane * PPT + p;
                wlab[(q & 3) * G + (q >> 2)] = mi[p];  // -1 for rows beyond N: matches no cluster
            }
            wave_lds_sync();
            const int kk = lane >> 4, col = lane & 15;
            const float bconst = col == D ? 1.0f : 0.0f;
            const int cread = col < D ? col : D - 1;  // lanes of the padding columns read a valid address
#pragma unroll
            for (int g4 = 0; g4 < G; g4 += 4) {
                const int4 lb = *reinterpret_cast<const int4*>(wlab + kk * G + g4);
                const int lbs[4] = {lb.x, lb.y, lb.z, lb.w};
                float bv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) bv[u] = wstage[SmallCfg<D>::stage_off(4 * (g4 + u) + kk) + cread];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float bval = col < D ? bv[u] : bconst;
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const float a = lbs[u] == col + 16 * mb ? 1.0f : 0.0f;
                        macc[mb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bval, macc[mb], 0, 0, 0);
                    }
                }
            }
            wave_lds_sync();  // the next round overwrites the staging buffer and the labels
            if (++since_flush == 8) flush_macc();
        }
        if (ACC == 2) {
            for (int k = 0; k < K; ++k) {
                float f[PPT], v[D + 1];
#pragma unroll
                for (int p = 0; p < PPT; ++p) f[p] = (mi[p] == k) ? 1.0f : 0.0f;
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    v[d] = f[0] * x[0][d];
#pragma unroll
                    for (int p = 1; p < PPT; ++p) v[d] = fmaf(f[p], x[p][d], v[d]);
                }
                v[D] = f[0];
#pragma unroll
                for (int p = 1; p < PPT; ++p) v[D] += f[p];
#pragma unroll
                for (int d = 0; d <= D; ++d) v[d] = wave_sum_to_lane63(v[d]);
                if (lane == 63) {
#pragma unroll
                    for (int d = 0; d <= D; ++d) wacc[k * (D + 1) + d] += double(v[d]);
                }
            }
        }
    };

    // Main loop, identical trip count for every lane of the workgroup.  Rounds in which the whole
    // workgroup lies inside the vector-loadable range take the fast path; the next round's rows are
    // requested before the current round is processed.
    {
        // The loop is unrolled PF times so that each round's buffer is a fixed set of registers: a
        // register rotation would make every round wait for ALL outstanding loads.  (The requests sit under a
        // condition, so the compiler's wait for a round's rows also covers most of the later rounds' loads; the
        // loop without conditions, with all PF rounds truly in flight, was measured and is 3-18 % slower.)
        bool more = base + T <= full;
        while (more) {
#pragma unroll
            for (int f = 0; f < PF; ++f) {
                if (more) {
                    float x[PPT][D];
                    // lanes exchange data through the wave's buffer: the fences tell the compiler
                    // that other lanes read what this lane wrote (and wrote what it reads); the
                    // hardware runs a wave's LDS operations in order
                    wave_lds_sync();
#pragma unroll
                    for (int v = 0; v < NV; ++v)
                        *reinterpret_cast<floatx4*>(wstage + ((v * 256 + lane * 4) / RL) * RLP + (v * 256 + lane * 4) % RL) =
                            nxt[f][v];  // (piece v * 64 + lane of the round, in memory order, into its lane's row)
                    wave_lds_sync();
                    if (base + PF * stride + T <= full) {
#pragma unroll
                        for (int v = 0; v < NV; ++v) nxt[f][v] = ldg4<STREAM>(wsrc + PF * rstride + v * 256);
                    }
                    wsrc += rstride;
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const floatx4 q =
                            *reinterpret_cast<const floatx4*>(wstage + lane * RLP + 4 * v);
#pragma unroll
                        for (int t = 0; t < 4; ++t) x[(4 * v + t) / D][(4 * v + t) % D] = q[t];
                    }
                    process((base + tid) * PPT, x, std::false_type{});
                    base += stride;
                    more = base + T <= full;
                }
            }
        }
    }
    // remaining rounds: unaligned / strided inputs and the ragged end, rows clamped and guarded
    for (; base < groups; base += stride) {
        const int64_t i0 = (base + tid) * PPT;
        float x[PPT][D];
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            const int64_t r = (i0 + p < N) ? i0 + p : N - 1;
#pragma unroll
            for (int d = 0; d < D; ++d) x[p][d] = X[r * ldx + d];
        }
        if (ACC == 3 || mscan) {
            // the matrix-core accumulation and the matrix-core scan read the round's points from the staging buffer
            wave_lds_sync();
#pragma unroll
            for (int p = 0; p < PPT; ++p)
#pragma unroll
                for (int d = 0; d < D; ++d) wstage[lane * RLP + p * D + d] = x[p][d];
            wave_lds_sync();
        }
        process(i0, x, std::true_type{});
    }

    if (ACC == 1) {
        // the last round's points are still pending
#pragma unroll
        for (int p = 0; p < PPT; ++p) {
            float r[D + 1];
            rmw_read(p, r);
            rmw_write(p, r);
        }
    }
    if (ACC == 3) flush_macc();
    if (ACC == 4 && bad) atomicOr(&imeta[1], 1);
    if (ACCUM || WANT_SSE) {
        __syncthreads();
        double* prow = part + int64_t(blockIdx.x) * (slots + 1);
        if (ACC == 4) {
            for (int s = tid; s < slots; s += T) {
                const int k = s / (D + 1), d = s - k * (D + 1);
                unsigned long long bits = 0ull, cnt = 0ull;
                for (int r = 0; r < nrep; ++r) {
                    bits += iacc[(k * LDI + d) * nrep + r];
                    cnt += iacc[(k * LDI + D) * nrep + r];
                }
                const long long sum = (long long)(bits - cnt * 0x4338000000000000ull);
                prow[s] = d == D ? double(cnt) : double(sum) * iquantum;
            }
            if (tid == 0) flags[blockIdx.x] = imeta[1];
        }
        if (ACC == 2 || ACC == 3) {
            for (int s = tid; s < slots; s += T) {
                double v = 0.0;
#pragma unroll
                for (int w = 0; w < NW; ++w) v += wacc_all[w * slots + s];
                prow[s] = v;
            }
        }
        if (ACC == 1) {
            // lanes add their T/64 columns in ascending order, then a butterfly over the 64 lanes
            for (int s = wave; s < slots; s += NW) {
                double v = 0.0;
                for (int t = lane; t < T; t += 64) v += double(cols[s * T + t]);
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
                if (lane == 0) prow[s] = v;
            }
        }
        if (WANT_SSE) {
            __shared__ double ssh[NW];
            double v = sse;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
            if (lane == 0) ssh[wave] = v;
            __syncthreads();
            if (tid == 0) {
                double t = 0.0;
                for (int w = 0; w < NW; ++w) t += ssh[w];
                prow[slots] = t;
            }
        }
    }
}

// One workgroup of 1024 threads finishes the step.  Thread (j, s) adds the partial rows g = j, j+J,
// ... of slot s in ascending order (up to 32 independent loads in flight, additions still in row order);
// thread (0, s) then adds the J strided sums in ascending j.  The order depends only on (G, slots).
__global__ __launch_bounds__(1024) void lloyd_small_finalize_kernel(
    const double* __restrict__ part, int G, int K, int D, const float* __restrict__ C_old,
    float* __restrict__ C_new, int64_t ldcn, int64_t* __restrict__ counts,
    float* __restrict__ shift, float* __restrict__ sse_out, int have_sse, int spad) {
    __shared__ double strided[1024];
    __shared__ double tot[256];
    __shared__ double red[256];
    const int tid = threadIdx.x;
    const int slots = K * (D + 1);
    const int nslot = slots + 1;  // last = sum of min d2
    const int J = 1024 / spad;  // spad = nslot: as many row groups as fit the workgroup
    const int s = tid % spad, j = tid / spad;
    // the old coordinate this thread will compare its mean with (K * D <= 240 < 1024: one per thread), asked
    // for before the partial rows so that its latency hides behind theirs
    float c_old = 0.0f;
    if (C_old && tid < K * D) c_old = C_old[tid];
    double v = 0.0;
    if (j < J && s < nslot && (s < slots || have_sse)) {
        // a thread's rows are requested 32 at a time, the last batch with the rows beyond G left out: the
        // kernel is nothing but the latency of these reads, and a few hundred rows should cost one round
        // trip, not one per eight rows and one per row of the remainder
        for (int g = j; g < G; g += 32 * J) {
            double t[32];
#pragma unroll
            for (int u = 0; u < 32; ++u) t[u] = g + u * J < G ? part[int64_t(g + u * J) * nslot + s] : 0.0;
#pragma unroll
            for (int u = 0; u < 32; ++u)
                if (g + u * J < G) v += t[u];
        }
    }
    strided[tid] = v;
    __syncthreads();
    if (j == 0 && s < nslot) {  // (threads of j == 0 are tid < spad)
        double t = 0.0;
        for (int q = 0; q < J; ++q) t += strided[q * spad + s];
        tot[s] = t;
    }
    __syncthreads();
    double sq = 0.0;
    for (int i = tid; i < K * D; i += 1024) {
        const int k = i / D, d = i - k * D;
        const int64_t n = (int64_t)tot[k * (D + 1) + D];
        const double cnt = double(float(n < 1 ? 1 : n));
        const float c = float(tot[k * (D + 1) + d] / cnt);
        C_new[int64_t(k) * ldcn + d] = c;
        if (C_old) {
            const float df = c_old - c;  // i == tid here
            sq += double(df * df);
        }
        if (d == 0 && counts) counts[k] = n;
    }
    // The pairwise tree over 1024 slots (t += t + w for w = 512 ... 1), of which only the first K * D <= 240
    // are not zero: the two widest levels add zeros and are left out, two levels go through LDS, the last
    // six stay inside the first wave.  Same association, same bits.
    if (tid < 256) red[tid] = sq;
    __syncthreads();
    if (tid < 128) red[tid] += red[tid + 128];
    __syncthreads();
    if (tid < 64) {
        double r = red[tid] + red[tid + 64];
#pragma unroll
        for (int w = 32; w > 0; w >>= 1) r += __shfl_down(r, w);
        if (tid == 0) {
            if (shift) *shift = float(r);
            if (sse_out && have_sse) *sse_out = float(tot[slots]);
        }
    }
}

// First level of the finish for many wide partial rows: workgroup b adds rows b * R0 .. of `part` in ascending
// order (16 loads in flight, additions still in row order) into row b of `out`.  One workgroup walking a
// thousand rows of 145 values is 30 us of latency; 32 workgroups walking 32 rows each and one walking their
// 32 results are 10.  The order depends only on (G, R0).
__global__ __launch_bounds__(256) void lloyd_small_prereduce_kernel(const double* __restrict__ part, int G, int nslot,
                                                                    int R0, double* __restrict__ out) {
    const int g0 = blockIdx.x * R0, g1 = min(G, g0 + R0);
    for (int s = threadIdx.x; s < nslot; s += 256) {
        double v = 0.0;
        for (int g = g0; g < g1; g += 16) {
            double t[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) t[u] = g + u < g1 ? part[int64_t(g + u) * nslot + s] : 0.0;
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (g + u < g1) v += t[u];
        }
        out[int64_t(blockIdx.x) * nslot + s] = v;
    }
}

// acc_mode: 0 labels only, else the accumulation strategy; flags / aux as in the kernel
template <int D>
static int launch_small_t(const float* X, int64_t N, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, double* part, bool want_sse,
                          int acc_mode, int grid, int32_t* flags, int aux, bool timed, bool labels64, hipStream_t st) {
    const bool want_min = min_d2 != nullptr;
    const size_t lds = small_lds_bytes(D, K, acc_mode);
    // bit 0: 16-byte vector path; bit 1: X exceeds the 256 MB last-level cache -> streaming loads;
    // bit 2: the scan takes the centroids four at a time; bit 3: labels are stored as 64-bit integers
    const int vec = ((ldx == D) && aligned16(X) && aligned16(labels) ? 1 : 0) |
                    (N * int64_t(D) * 4 > (int64_t(256) << 20) ? 2 : 0) | (K >= small_blocked_min_k() ? 4 : 0) |
                    (labels64 ? 8 : 0);
    // the register-resident centroid table: K <= 8 rows of at most 5 values
    constexpr int KT8 = D <= 4 ? 8 : 0;
    const bool reg = KT8 > 0 && K <= KT8;
    // streaming loads only in the modes that large matrices run in (labels only, per-lane columns, integer sums)
#define HKM_LAUNCH(A, M, S, KTV, STRM)                                                                            \
    hipLaunchKernelGGL((lloyd_small_kernel<D, A, M, S, KTV, STRM>), dim3(grid), dim3(SMALL_T), lds, st, X, N, ldx, C, \
                       K, ldc, labels, min_d2, part, vec, flags, aux)
#define HKM_GO2(A, M, S, KTV)                                          \
    do {                                                               \
        if constexpr (A == 0 || A == 1 || A == 4) {                    \
            if (vec & 2) HKM_LAUNCH(A, M, S, KTV, true);               \
            else HKM_LAUNCH(A, M, S, KTV, false);                      \
        } else {                                                       \
            HKM_LAUNCH(A, M, S, KTV, false);                           \
        }                                                              \
    } while (0)
#define HKM_GO(A, M, S)                                  \
    do {                                                 \
        if (A == 3 && K > 16) HKM_GO2(A, M, S, (A == 3 ? 32 : 0));       \
        else if (A == 3) HKM_GO2(A, M, S, (A == 3 ? 16 : 0));            \
        else if (reg && A != 4) HKM_GO2(A, M, S, (A != 4 ? KT8 : 0));    \
        else HKM_GO2(A, M, S, 0);                                        \
    } while (0)
    if (timed) prof_begin(st);
    if (acc_mode == 2) {
        if (want_sse) HKM_GO(2, false, true);
        else HKM_GO(2, false, false);
    } else if (acc_mode == 4) {
        if (want_sse) HKM_GO(4, false, true);
        else HKM_GO(4, false, false);
    } else if (acc_mode == 0) {
        if (want_min) HKM_GO(0, true, false);
        else HKM_GO(0, false, false);
    } else {
        // per-lane columns and the matrix-core product exist up to 8 features (small_ordered_mode)
        if constexpr (D <= 8) {
            if (acc_mode == 1) {
                if (want_sse) HKM_GO(1, false, true);
                else HKM_GO(1, false, false);
            } else {
                if (want_sse) HKM_GO(3, false, true);
                else HKM_GO(3, false, false);
            }
        } else {
            return fail(HKM_EUNSUPPORTED, "lloyd_small: accumulation mode %d with D=%d", acc_mode, D);
        }
    }
    if (timed) prof_end(st);
#undef HKM_GO
#undef HKM_GO2
#undef HKM_LAUNCH
    return check_launch("lloyd_small_kernel");
}

// how many bits above the largest centroid coordinate a row may reach in the integer accumulation:
// the fused multiply-add needs |x| * 2^(QB - Ec) < 2^51, the 64-bit sum of a workgroup's rows 2^62
static int small_headroom_bits(int64_t N, int32_t D, int grid) {
    const int ppt = (D % 2 == 0) ? 2 : 4;
    const int64_t groups = (N + ppt - 1) / ppt;
    const int64_t per_wg = int64_t(SMALL_T) * ppt;
    const int64_t rounds = (groups + int64_t(grid) * SMALL_T - 1) / (int64_t(grid) * SMALL_T);
    const int64_t rows = rounds * per_wg;
    int lg = 0;
    while ((int64_t(1) << lg) < rows) ++lg;
    return std::min(51 - SMALL_QB, 62 - SMALL_QB - lg);
}

// mode bit 0: accumulate per-cluster sums into `part`; bit 1: also the sum of min d2.
// flags: [grid] scratch for the integer accumulation (may be NULL: then the ordered strategies run).
int launch_small(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                 int64_t ldc, int32_t* labels, float* min_d2, double* part, int mode, int32_t* flags,
                 hipStream_t st, bool labels64) {
    const int grid = small_grid(N, D, K);
    const bool accum = mode & 1, want_sse = mode & 2;
    const int headroom = small_headroom_bits(N, D, grid);
    const bool integer = accum && flags && headroom >= 4 && small_integer_sums(N, D, K);
    const int ordered = small_ordered_mode(D, K);
#define HKM_T(d)                                                                                           \
    case d: {                                                                                              \
        if (!integer)                                                                                      \
            return launch_small_t<d>(X, N, ldx, C, K, ldc, labels, min_d2, part, want_sse, accum ? ordered : 0, \
                                     grid, nullptr, 0, true, labels64, st);                                \
        int rc = launch_small_t<d>(X, N, ldx, C, K, ldc, labels, min_d2, part, want_sse, 4, grid, flags,   \
                                   headroom, true, labels64, st);                                          \
        if (rc) return rc;                                                                                 \
        /* the same sweep in the ordered way if a workgroup raised its flag; returns at once otherwise */  \
        return launch_small_t<d>(X, N, ldx, C, K, ldc, labels, min_d2, part, want_sse, ordered, grid, flags, \
                                 grid, false, labels64, st);                                               \
    }
    switch (D) {
        HKM_T(1) HKM_T(2) HKM_T(3) HKM_T(4) HKM_T(5) HKM_T(6) HKM_T(7) HKM_T(8)
        HKM_T(9) HKM_T(10) HKM_T(11) HKM_T(12) HKM_T(13) HKM_T(14) HKM_T(15) HKM_T(16)
        default:
            return fail(HKM_EUNSUPPORTED, "lloyd_small: D=%d outside 1..16", D);
    }
#undef HKM_T
}

int launch_small_finalize(const double* part, int grid, int32_t K, int32_t D, const float* C_old,
                          float* C_new, int64_t ldcn, int64_t* counts, float* shift, float* sse,
                          hipStream_t st) {
    const int spad = K * (D + 1) + 1;  // <= 241 because K*(D+1) <= 240
    // many wide rows: two levels (the first writes behind the rows it reads; the workspace holds SMALL_MAX_GRID)
    if (int64_t(grid) * spad >= 32768 && grid + 32 <= SMALL_MAX_GRID) {
        const int r0 = (grid + 31) / 32, nb = (grid + r0 - 1) / r0;
        double* out = const_cast<double*>(part) + int64_t(grid) * spad;
        hipLaunchKernelGGL(lloyd_small_prereduce_kernel, dim3(nb), dim3(256), 0, st, part, grid, spad, r0, out);
        int rc = check_launch("lloyd_small_prereduce_kernel");
        if (rc) return rc;
        part = out;
        grid = nb;
    }
    hipLaunchKernelGGL(lloyd_small_finalize_kernel, dim3(1), dim3(1024), 0, st, part, grid, K, D,
                       C_old, C_new, ldcn, counts, shift, sse, sse ? 1 : 0, spad);
    return check_launch("lloyd_small_finalize_kernel");
}

}  // namespace hkm
