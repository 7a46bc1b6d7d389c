// k nearest rows without the distance matrix: the cdist -> topk(largest=False) -> label vote chain of
// heat/classification/kneighborsclassifier.py:114-132.
//
//   * knn_tile_kernel: a workgroup owns 64 query rows and walks its share of the reference rows in
//     tiles of 64 (4 x 4 register block per lane, both tiles staged through LDS in chunks of 16
//     features, sum (q - r)^2 in fp32 -- the direct form, no cancellation).  Every lane keeps the KL
//     best (distance, row) pairs of its four query rows, sorted, in registers; a candidate is only
//     looked at when it beats the row's threshold, the smallest k-th entry among the 16 lanes that
//     share the row (that lane alone holds k closer rows, so nothing above it can rank).  At the end
//     the 16 lists of a row are merged with shuffles.  Reference rows can be split over several
//     workgroups (grid.y); their lists are merged by knn_merge_kernel.  More than KL neighbours are
//     found in passes: a pass only admits pairs that rank after the last pair of the pass before.
//   * order: ascending (squared distance, row index) -- the first row wins exact ties.
//   * knn_vote_kernel: sum of the label rows of the k neighbours, argmax with the first class on ties.
//
//   * knn_mfma_kernel (16 <= D <= 128): the same walk with the products q.x on the matrix cores and the
//     squared distance as (|q|^2 + |x|^2) - 2 q.x clamped at zero, the form torch.cdist itself takes above
//     25 rows.  A wave owns 32 query rows, held in registers for the whole kernel; a tile of 32 reference
//     rows goes from global memory straight into the A operand (lane = row, half of the features each:
//     the order of the features inside the sum is free as long as both operands agree), 32x32x2 fp32
//     MFMAs leave every lane with 16 candidates of ONE query row, so a lane keeps one list and the
//     two lanes of a query row merge at the end.  |x|^2 comes from knn_norms_kernel.
//
// Bound: knn_tile_kernel the vector ALU, 2 operations (subtract, fused multiply-add) per (query, row,
// feature); knn_mfma_kernel the fp32 matrix cores, 2 flops per (query, row, feature).
#include "hkm_mfma_util.h"

namespace hkm {

static constexpr int KNN_T = 64;
static constexpr int KNN_KC = 16;
static constexpr int KNN_MAX_SPLITS = 64;
static constexpr int KNN_MAX_TARGET = 1536;
static constexpr unsigned KNN_NONE = 0xffffffffu;

__device__ __forceinline__ bool knn_less(float d, unsigned i, float e, unsigned j) {
    return d < e || (d == e && i < j);
}

template <int KL>
__device__ __forceinline__ void knn_insert(float (&ld)[KL], unsigned (&li)[KL], float d, unsigned i) {
    // candidates of one lane arrive in ascending row order, so '<' on the distance alone keeps ties stable
#pragma unroll
    for (int s = KL - 1; s >= 0; --s) {
        const bool up = s > 0 && d < ld[s > 0 ? s - 1 : 0];
        const bool here = !up && d < ld[s];
        const float nd = up ? ld[s > 0 ? s - 1 : 0] : (here ? d : ld[s]);
        const unsigned ni = up ? li[s > 0 ? s - 1 : 0] : (here ? i : li[s]);
        ld[s] = nd;
        li[s] = ni;
    }
}

// The lists live in registers and must be updated in place: a branch per lane around the insertion makes
// the compiler copy a whole list at every candidate, so the branch is taken by the wave as a whole (any
// lane with a hit) and lanes without one insert +inf, which changes nothing.
// x = take ? y : x, written so that x stays in its register (the compiler's own selects end up in fresh
// registers and the list is copied back at every candidate)
__device__ __forceinline__ void knn_keep_or(float& x, float y, unsigned long long take) {
    asm("v_cndmask_b32_e64 %0, %0, %1, %2" : "+v"(x) : "v"(y), "s"(take));
}
__device__ __forceinline__ void knn_keep_or(unsigned& x, unsigned y, unsigned long long take) {
    asm("v_cndmask_b32_e64 %0, %0, %1, %2" : "+v"(x) : "v"(y), "s"(take));
}

// the insertion of knn_insert slot by slot from the end: slot s takes the candidate if it is smaller, and
// the pair in front of it instead if the candidate is smaller than that one too
template <int KL>
__device__ __forceinline__ void knn_insert_in_place(float (&ld)[KL], unsigned (&li)[KL], float d, unsigned i) {
    unsigned long long lt[KL];
#pragma unroll
    for (int s = 0; s < KL; ++s) lt[s] = __builtin_amdgcn_ballot_w64(d < ld[s]);
#pragma unroll
    for (int s = KL - 1; s >= 0; --s) {
        knn_keep_or(ld[s], d, lt[s]);
        knn_keep_or(li[s], i, lt[s]);
        if (s > 0) {
            knn_keep_or(ld[s], ld[s - 1], lt[s - 1]);
            knn_keep_or(li[s], li[s - 1], lt[s - 1]);
        }
    }
}

template <int KL>
__device__ __forceinline__ void knn_offer(float (&ld)[KL], unsigned (&li)[KL], bool ok, float d, unsigned i) {
    if (__builtin_amdgcn_ballot_w64(ok) != 0) knn_insert_in_place(ld, li, ok ? d : HKM_INF, i);
}

template <int KL>
__global__ __launch_bounds__(256) void knn_tile_kernel(
    const float* __restrict__ Q, int64_t M, int64_t ldq, const float* __restrict__ R, int64_t Nn, int64_t ldr,
    int D, int64_t rows_per_split, int has_bound, float* __restrict__ last_d2, unsigned* __restrict__ last_i,
    float* __restrict__ part_d, unsigned* __restrict__ part_i, int64_t* __restrict__ out_i, int64_t ldi,
    float* __restrict__ out_d, int64_t ldd, int col0, int kcount) {
    __shared__ float sQ[KNN_KC][KNN_T + 4];
    __shared__ float sR[KNN_KC][KNN_T + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int lk = tid & 15, lr = tid >> 4;
    const int64_t i0 = int64_t(blockIdx.x) * KNN_T;
    const int64_t r_begin = int64_t(blockIdx.y) * rows_per_split;
    const int64_t r_end = min(Nn, r_begin + rows_per_split);

    float ld[4][KL];
    unsigned li[4][KL];
    float bd[4];
    unsigned bi[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int s = 0; s < KL; ++s) {
            ld[a][s] = HKM_INF;
            li[a][s] = KNN_NONE;
        }
        const int64_t gi = i0 + ty * 4 + a;
        bd[a] = -1.0f;
        bi[a] = 0;
        if (has_bound && gi < M) {
            bd[a] = last_d2[gi];
            bi[a] = last_i[gi];
        }
    }

    for (int64_t j0 = r_begin; j0 < r_end; j0 += KNN_T) {
        float acc[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[a][b] = 0.0f;
        for (int d0 = 0; d0 < D; d0 += KNN_KC) {
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int r = lr + 16 * q;
                const int d = d0 + lk;
                const int64_t gi = i0 + r, gj = j0 + r;
                sQ[lk][r] = (gi < M && d < D) ? Q[gi * ldq + d] : 0.0f;
                sR[lk][r] = (gj < r_end && d < D) ? R[gj * ldr + d] : 0.0f;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < KNN_KC; ++k) {
                float qa[4], rb[4];
#pragma unroll
                for (int a = 0; a < 4; ++a) qa[a] = sQ[k][ty * 4 + a];
#pragma unroll
                for (int b = 0; b < 4; ++b) rb[b] = sR[k][tx * 4 + b];
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const float df = qa[a] - rb[b];
                        acc[a][b] = fmaf(df, df, acc[a][b]);
                    }
            }
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            // every list entry stems from an earlier tile, i.e. from a smaller row index than any
            // candidate of this one: a candidate at exactly the threshold ranks after KL entries
            float thr = ld[a][KL - 1];
#pragma unroll
            for (int s = 0; s < KL - 1; ++s) thr = s == kcount - 1 ? ld[a][s] : thr;  // only kcount entries are asked for
#pragma unroll
            for (int w = 1; w < 16; w <<= 1) thr = fminf(thr, __shfl_xor(thr, w));
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int64_t gj = j0 + tx * 4 + b;
                const float d = acc[a][b];
                bool ok = gj < r_end && d < thr;
                if (has_bound) ok = ok && (d > bd[a] || (d == bd[a] && unsigned(gj) > bi[a]));
                knn_offer<KL>(ld[a], li[a], ok, d, unsigned(gj));
            }
        }
    }

    // merge the 16 sorted lists of every row: KL times the smallest head, whose lane pops it
    const bool final_out = gridDim.y == 1;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int64_t gi = i0 + ty * 4 + a;
        for (int r = 0; r < KL; ++r) {
            float md = ld[a][0];
            unsigned mi = li[a][0];
#pragma unroll
            for (int w = 1; w < 16; w <<= 1) {
                const float od = __shfl_xor(md, w);
                const unsigned oi = unsigned(__shfl_xor(int(mi), w));
                if (knn_less(od, oi, md, mi)) {
                    md = od;
                    mi = oi;
                }
            }
            if (mi != KNN_NONE && mi == li[a][0]) {
#pragma unroll
                for (int s = 0; s + 1 < KL; ++s) {
                    ld[a][s] = ld[a][s + 1];
                    li[a][s] = li[a][s + 1];
                }
                ld[a][KL - 1] = HKM_INF;
                li[a][KL - 1] = KNN_NONE;
            }
            if (tx == 0 && gi < M) {
                if (final_out) {
                    if (r < kcount) {
                        out_i[gi * ldi + col0 + r] = mi == KNN_NONE ? int64_t(-1) : int64_t(mi);
                        if (out_d) out_d[gi * ldd + col0 + r] = sqrtf(md);
                        if (r == kcount - 1) {
                            last_d2[gi] = md;
                            last_i[gi] = mi;
                        }
                    }
                } else {
                    part_d[(int64_t(blockIdx.y) * M + gi) * KL + r] = md;
                    part_i[(int64_t(blockIdx.y) * M + gi) * KL + r] = mi;
                }
            }
        }
    }
}

// ---- shared by the two matrix-core kernels -------------------------------------------------------
// The distance a list must beat: the kcount-th entry, the smaller one of the two lanes that share a query
// row.  Pairs in the lists stem from earlier tiles, i.e. from smaller rows than any later candidate, so a
// candidate at exactly the threshold ranks after kcount of them.
template <int KL>
__device__ __forceinline__ float knn_threshold(const float (&ld)[KL], int kcount) {
    float thr = ld[KL - 1];
#pragma unroll
    for (int s = 0; s < KL - 1; ++s) thr = s == kcount - 1 ? ld[s] : thr;  // only kcount entries are asked for
    return fminf(thr, __shfl_xor(thr, 32));
}

// Candidates of one 32 x 32 block.  t holds |x|^2 - 2 q.x (the accumulators start at the squared norms of
// their reference rows and the query operand carries the factor -2): element i is reference row
// j0 + 8 (i / 4) + 4 h + i % 4, its squared distance max(t + |q|^2, 0).  The smallest of the 16 is found
// first (a tree of three-input minima, nine instructions); only if it beats the threshold in some lane of
// the wave are the 16 looked at one by one -- adding |q|^2 and clamping are monotone, so the test on the
// minimum decides exactly as the tests on the elements would.  thr is carried from tile to tile and
// recomputed only after the lists may have changed.
template <int KL>
__device__ __forceinline__ void knn_block_candidates(float (&ld)[KL], unsigned (&li)[KL], float& thr,
                                                     const floatx16& t, float qn, int64_t j0, int64_t seen, int h,
                                                     int64_t r_end, int kcount, int has_bound, float bd, unsigned bi) {
    // the last tile of a split (rows past the end) and the later passes of k > 16 (pairs ranked before the
    // bound) need every element looked at
    const bool edge = j0 + 32 > r_end || has_bound;
    // While the lists are young nearly every tile holds a candidate for some lane of the wave and the test
    // on the minimum is thirteen instructions for nothing: after `seen` rows a wave of 32 queries expects
    // 32 * 32 * kcount / seen admissions per tile, and the test pays once that is below about 1.7.
    if (!edge && seen >= int64_t(608) * kcount) {
        const float s = block_min16(t) + qn;
        const float dmin = s < 0.0f ? 0.0f : s;
        if (__builtin_amdgcn_ballot_w64(dmin < thr) == 0) return;
    }
    const unsigned gj0 = unsigned(j0) + 4 * h;
    if (!edge) {
        // The common tile.  An element is first tested without the clamp (t + |q|^2 < thr: one addition, one
        // compare); the clamp only raises negative values to 0, so whatever passes the clamped test passes this
        // one, and the few that pass it are clamped and tested again before they are offered.  A NaN fails both.
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float s = t[i] + qn;
            if (__builtin_amdgcn_ballot_w64(s < thr) != 0) {
                const float d = s < 0.0f ? 0.0f : s;
                knn_insert_in_place(ld, li, d < thr ? d : HKM_INF, gj0 + 8 * (i >> 2) + (i & 3));
            }
        }
        thr = knn_threshold<KL>(ld, kcount);
        return;
    }
    float dv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        // compare + select, not fmaxf: a NaN (a NaN row, inf - inf of overflowing norms) must stay a NaN,
        // which fails every `< thr` below and is never admitted; fmaxf would turn it into distance 0
        const float s = t[i] + qn;
        dv[i] = s < 0.0f ? 0.0f : s;
    }
    // rows past the end and pairs that do not rank after the bound become +inf here
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const unsigned gj = gj0 + 8 * (i >> 2) + (i & 3);
        bool ok = gj < unsigned(r_end);
        if (has_bound) ok = ok && (dv[i] > bd || (dv[i] == bd && gj > bi));
        dv[i] = ok ? dv[i] : HKM_INF;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) knn_offer<KL>(ld, li, dv[i] < thr, dv[i], gj0 + 8 * (i >> 2) + (i & 3));
    thr = knn_threshold<KL>(ld, kcount);
}

// The two lanes of a query row (h = 0, 1): KL times the smaller head, whose lane pops it; lane h = 0
// writes -- the final output when one split covers all rows, else the split's list for knn_merge_kernel.
template <int KL>
__device__ __forceinline__ void knn_pair_merge_write(float (&ld)[KL], unsigned (&li)[KL], int kcount, int h, bool live,
                                                     int64_t gi, int64_t M, bool final_out, float* last_d2,
                                                     unsigned* last_i, float* part_d, unsigned* part_i, int64_t* out_i,
                                                     int64_t ldi, float* out_d, int64_t ldd, int col0) {
#pragma unroll
    for (int r = 0; r < KL; ++r) {
        const float od = __shfl_xor(ld[0], 32);
        const unsigned oi = unsigned(__shfl_xor(int(li[0]), 32));
        const bool other = knn_less(od, oi, ld[0], li[0]);
        const float md = other ? od : ld[0];
        const unsigned mi = other ? oi : li[0];
        if (!other && mi != KNN_NONE) {
#pragma unroll
            for (int s = 0; s + 1 < KL; ++s) {
                ld[s] = ld[s + 1];
                li[s] = li[s + 1];
            }
            ld[KL - 1] = HKM_INF;
            li[KL - 1] = KNN_NONE;
        }
        if (h == 0 && live) {
            if (final_out) {
                if (r < kcount) {
                    out_i[gi * ldi + col0 + r] = mi == KNN_NONE ? int64_t(-1) : int64_t(mi);
                    if (out_d) out_d[gi * ldd + col0 + r] = sqrtf(md);
                    if (r == kcount - 1) {
                        last_d2[gi] = md;
                        last_i[gi] = mi;
                    }
                }
            } else {
                part_d[(int64_t(blockIdx.y) * M + gi) * KL + r] = md;
                part_i[(int64_t(blockIdx.y) * M + gi) * KL + r] = mi;
            }
        }
    }
}

// |x|^2 of every reference row: 16 lanes per row, features strided over the lanes, fixed-order tree.
__global__ __launch_bounds__(256) void knn_norms_kernel(const float* __restrict__ R, int64_t Nn, int64_t ldr, int D,
                                                        float* __restrict__ xn) {
    const int t = threadIdx.x & 15;
    const int64_t row = int64_t(blockIdx.x) * 16 + (threadIdx.x >> 4);
    float s = 0.0f;
    if (row < Nn)
        for (int d = t; d < D; d += 16) {
            const float v = R[row * ldr + d];
            s = fmaf(v, v, s);
        }
#pragma unroll
    for (int w = 1; w < 16; w <<= 1) s += __shfl_xor(s, w);
    if (t == 0 && row < Nn) xn[row] = s;
}

// H features per lane: lanes 0..31 hold features [0, H) of their row, lanes 32..63 features [H, 2H).
template <int KL, int H, bool VEC>
__global__ __launch_bounds__(256) void knn_mfma_kernel(
    const float* __restrict__ Q, int64_t M, int64_t ldq, const float* __restrict__ R, int64_t Nn, int64_t ldr,
    int D, const float* __restrict__ xn, int64_t rows_per_split, int has_bound, float* __restrict__ last_d2,
    unsigned* __restrict__ last_i, float* __restrict__ part_d, unsigned* __restrict__ part_i,
    int64_t* __restrict__ out_i, int64_t ldi, float* __restrict__ out_d, int64_t ldd, int col0, int kcount) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int64_t gi = int64_t(blockIdx.x) * 128 + wave * 32 + col;
    const bool live = gi < M;
    const int64_t r_begin = int64_t(blockIdx.y) * rows_per_split;
    const int64_t r_end = min(Nn, r_begin + rows_per_split);

    float qv[H];
    float qn = 0.0f;
    {
        const float* qrow = Q + (live ? gi : 0) * ldq;
#pragma unroll
        for (int g = 0; g < H / 4; ++g) {
            const floatx4 t = load_row4<VEC>(qrow, h * H + 4 * g, D);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float q = live ? t[e] : 0.0f;
                qv[4 * g + e] = -2.0f * q;  // exact; the accumulators then hold |x|^2 - 2 q.x
                qn = fmaf(q, q, qn);
            }
        }
        qn += __shfl_xor(qn, 32);
    }

    float ld[KL];
    unsigned li[KL];
#pragma unroll
    for (int s = 0; s < KL; ++s) {
        ld[s] = HKM_INF;
        li[s] = KNN_NONE;
    }
    float thr = HKM_INF;  // what a candidate must beat: the lists are empty
    float bd = -1.0f;
    unsigned bi = 0;
    if (has_bound && live) {
        bd = last_d2[gi];
        bi = last_i[gi];
    }

    auto load_tile = [&](int64_t j0, float (&av)[H]) {
        const int64_t gj = min(j0 + col, Nn - 1);  // rows past the end are read as the last row and never admitted
        const float* row = R + gj * ldr;
#pragma unroll
        for (int g = 0; g < H / 4; ++g) {
            const floatx4 t = load_row4<VEC>(row, h * H + 4 * g, D);
#pragma unroll
            for (int e = 0; e < 4; ++e) av[4 * g + e] = t[e];
        }
    };

    float av[H];
    load_tile(r_begin, av);
    for (int64_t j0 = r_begin; j0 < r_end; j0 += 32) {
        float an[H];
        load_tile(min(j0 + 32, r_end - 1), an);  // the next tile while this one is multiplied
        const floatx16 xnv = load_cn16(xn + j0 + 4 * h);
        floatx16 acc = MFMA32(av[0], qv[0], xnv);  // starts at the squared norms of its reference rows
#pragma unroll
        for (int s = 1; s < H; ++s) acc = MFMA32(av[s], qv[s], acc);
        knn_block_candidates<KL>(ld, li, thr, acc, qn, j0, j0 - r_begin, h, r_end, kcount, has_bound, bd, bi);
#pragma unroll
        for (int s = 0; s < H; ++s) av[s] = an[s];
    }

    knn_pair_merge_write<KL>(ld, li, kcount, h, live, gi, M, gridDim.y == 1, last_d2, last_i, part_d, part_i, out_i, ldi,
                             out_d, ldd, col0);
}

// The same kernel with the tile of reference rows staged through LDS: one coalesced read per workgroup
// (D % 4 == 0, 16-byte aligned rows) instead of one strided read per wave, double-buffered, one barrier
// per tile.  Columns from D on are zeroed once and never written.
template <int KL, int H>
__global__ __launch_bounds__(256) void knn_mfma_lds_kernel(
    const float* __restrict__ Q, int64_t M, int64_t ldq, const float* __restrict__ R, int64_t Nn, int64_t ldr,
    int D, const float* __restrict__ xn, int64_t rows_per_split, int has_bound, float* __restrict__ last_d2,
    unsigned* __restrict__ last_i, float* __restrict__ part_d, unsigned* __restrict__ part_i,
    int64_t* __restrict__ out_i, int64_t ldi, float* __restrict__ out_d, int64_t ldd, int col0, int kcount) {
    constexpr int RS = 2 * H + 4;            // floats per staged row; the pad spreads 16 rows over all banks
    constexpr int NV = H >= 16 ? H / 16 : 1;  // float4 groups a thread moves per tile
    __shared__ __attribute__((aligned(16))) float sA[2][32][RS];
    __shared__ __attribute__((aligned(16))) float sXn[2][32];  // squared norms of the staged rows
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, h = lane >> 5;
    const int64_t gi = int64_t(blockIdx.x) * 128 + wave * 32 + col;
    const bool live = gi < M;
    const int64_t r_begin = int64_t(blockIdx.y) * rows_per_split;
    const int64_t r_end = min(Nn, r_begin + rows_per_split);

    for (int i = tid; i < 2 * 32 * RS; i += 256) (&sA[0][0][0])[i] = 0.0f;

    float qv[H];
    float qn = 0.0f;
    {
        const float* qrow = Q + (live ? gi : 0) * ldq;
#pragma unroll
        for (int g = 0; g < H / 4; ++g) {
            const floatx4 t = load_row4<true>(qrow, h * H + 4 * g, D);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float q = live ? t[e] : 0.0f;
                qv[4 * g + e] = -2.0f * q;  // exact; the accumulators then hold |x|^2 - 2 q.x
                qn = fmaf(q, q, qn);
            }
        }
        qn += __shfl_xor(qn, 32);
    }

    float ld[KL];
    unsigned li[KL];
#pragma unroll
    for (int s = 0; s < KL; ++s) {
        ld[s] = HKM_INF;
        li[s] = KNN_NONE;
    }
    float thr = HKM_INF;  // what a candidate must beat: the lists are empty
    float bd = -1.0f;
    unsigned bi = 0;
    if (has_bound && live) {
        bd = last_d2[gi];
        bi = last_i[gi];
    }

    // which float4 groups of a tile this thread moves: group t + 256 j of the 32 x D/4 groups, row-major
    const int c4n = D >> 2;
    int srow[NV], scol[NV];
    bool sval[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int idx = tid + 256 * j;
        srow[j] = idx / c4n;
        scol[j] = 4 * (idx - srow[j] * c4n);
        sval[j] = idx < 32 * c4n;
    }
    floatx4 st[NV];
    floatx4 stn = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int64_t j0) {
#pragma unroll
        for (int j = 0; j < NV; ++j)
            if (sval[j]) st[j] = ld4(R + min(j0 + srow[j], Nn - 1) * ldr + scol[j]);  // rows past the end: never admitted
        // the norms ride along (eight threads): the first matrix instruction of a tile needs them, and
        // a read from global memory at that point would be waited for (the buffer is padded by 64 floats)
        if (tid < 8) stn = ld4(xn + j0 + 4 * tid);
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int j = 0; j < NV; ++j)
            if (sval[j]) *reinterpret_cast<floatx4*>(&sA[buf][srow[j]][scol[j]]) = st[j];
        if (tid < 8) *reinterpret_cast<floatx4*>(&sXn[buf][4 * tid]) = stn;
    };
    __syncthreads();
    fetch(r_begin);
    stash(0);
    __syncthreads();

    int buf = 0;
    for (int64_t j0 = r_begin; j0 < r_end; j0 += 32) {
        const bool more = j0 + 32 < r_end;
        if (more) fetch(j0 + 32);  // the next tile while this one is multiplied
        const floatx16 xnv = load_cn16(&sXn[buf][4 * h]);
        floatx16 acc;
        const float* arow = &sA[buf][col][h * H];
#pragma unroll
        for (int g = 0; g < H / 4; ++g) {
            const floatx4 a = *reinterpret_cast<const floatx4*>(arow + 4 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e)  // the accumulators start at the squared norms of their reference rows
                acc = (g == 0 && e == 0) ? MFMA32(a[e], qv[0], xnv) : MFMA32(a[e], qv[4 * g + e], acc);
        }
        knn_block_candidates<KL>(ld, li, thr, acc, qn, j0, j0 - r_begin, h, r_end, kcount, has_bound, bd, bi);
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    knn_pair_merge_write<KL>(ld, li, kcount, h, live, gi, M, gridDim.y == 1, last_d2, last_i, part_d, part_i, out_i, ldi,
                             out_d, ldd, col0);
}

// One wave per query row: kcount times the smallest (distance, row) pair after the one before among the
// nsplit * KL pairs of the row's split lists.
__global__ __launch_bounds__(256) void knn_merge_kernel(const float* __restrict__ part_d,
                                                        const unsigned* __restrict__ part_i, int nsplit, int KL,
                                                        int64_t M, float* __restrict__ last_d2,
                                                        unsigned* __restrict__ last_i, int64_t* __restrict__ out_i,
                                                        int64_t ldi, float* __restrict__ out_d, int64_t ldd, int col0,
                                                        int kcount) {
    const int lane = threadIdx.x & 63;
    const int64_t gi = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (gi >= M) return;
    const int total = nsplit * KL;
    float pd = -1.0f;  // the pair selected last; squared distances are >= 0
    unsigned pi = 0;
    for (int r = 0; r < kcount; ++r) {
        float md = HKM_INF;
        unsigned mi = KNN_NONE;
        for (int c = lane; c < total; c += 64) {
            const int s = c / KL, e = c - s * KL;
            const float d = part_d[(int64_t(s) * M + gi) * KL + e];
            const unsigned i = part_i[(int64_t(s) * M + gi) * KL + e];
            const bool after = d > pd || (d == pd && i > pi);
            if (i != KNN_NONE && after && knn_less(d, i, md, mi)) {
                md = d;
                mi = i;
            }
        }
#pragma unroll
        for (int w = 1; w < 64; w <<= 1) {
            const float od = __shfl_xor(md, w);
            const unsigned oi = unsigned(__shfl_xor(int(mi), w));
            if (knn_less(od, oi, md, mi)) {
                md = od;
                mi = oi;
            }
        }
        if (lane == 0) {
            out_i[gi * ldi + col0 + r] = mi == KNN_NONE ? int64_t(-1) : int64_t(mi);
            if (out_d) out_d[gi * ldd + col0 + r] = sqrtf(md);
            if (r == kcount - 1) {
                last_d2[gi] = md;
                last_i[gi] = mi;
            }
        }
        if (mi == KNN_NONE) {
            // nothing left (fewer finite distances than neighbours asked for): the rest stays unset
            for (int r2 = r + 1; r2 < kcount && lane == 0; ++r2) {
                out_i[gi * ldi + col0 + r2] = -1;
                if (out_d) out_d[gi * ldd + col0 + r2] = HKM_INF;
                if (r2 == kcount - 1) {
                    last_d2[gi] = HKM_INF;
                    last_i[gi] = KNN_NONE;
                }
            }
            break;
        }
        pd = md;
        pi = mi;
    }
}

// One wave per query row, lanes over the classes: votes[c] = sum over the neighbours, in their order, of
// Y[neighbour][c]; the class with the most votes, the first one on ties (torch.argmax).
__global__ __launch_bounds__(256) void knn_vote_kernel(const int64_t* __restrict__ idx, int64_t M, int k, int64_t ldi,
                                                       const float* __restrict__ Y, int64_t Nn, int C, int64_t ldy,
                                                       int64_t* __restrict__ classes) {
    const int lane = threadIdx.x & 63;
    const int64_t gi = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (gi >= M) return;
    float best = -HKM_INF;
    int bc = 0x7fffffff;
    for (int c = lane; c < C; c += 64) {
        float v = 0.0f;
        for (int j = 0; j < k; ++j) {
            const int64_t row = idx[gi * ldi + j];
            if (row >= 0 && row < Nn) v += Y[row * ldy + c];
        }
        if (v > best || bc == 0x7fffffff) {  // ascending c inside a lane: '>' keeps the first maximum
            best = v;
            bc = c;
        }
    }
#pragma unroll
    for (int w = 1; w < 64; w <<= 1) {
        const float ov = __shfl_xor(best, w);
        const int oc = __shfl_xor(bc, w);
        if (oc != 0x7fffffff && (bc == 0x7fffffff || ov > best || (ov == best && oc < bc))) {
            best = ov;
            bc = oc;
        }
    }
    if (lane == 0) classes[gi] = bc == 0x7fffffff ? 0 : bc;
}

// ------------------------------------------------------------------------------------------------
bool knn_uses_mfma(int32_t D);

// Workgroups to aim for when the reference rows are split: every workgroup pays for filling its lists
// before its threshold bites, so no more splits than it takes to fill the CUs at the kernel's occupancy
// (4 workgroups per CU up to 32 features, 3 up to 64, fewer above; measured best 1536 / 768).
int knn_target_workgroups(int32_t D) {
    if (!knn_uses_mfma(D)) return 768;
    return D <= 32 ? KNN_MAX_TARGET : (D <= 64 ? 768 : 512);
}

int knn_max_target_workgroups() { return KNN_MAX_TARGET; }

KnnPlan knn_plan(int64_t M, int64_t N, int target) {
    KnnPlan p;
    const int64_t qtiles = (M + 127) / 128;  // the larger of the two kernels' query tiles
    int64_t ns = qtiles > 0 ? (target + qtiles - 1) / qtiles : 1;
    ns = std::min<int64_t>(ns, std::max<int64_t>(1, N / 256));
    ns = std::max<int64_t>(1, std::min<int64_t>(ns, KNN_MAX_SPLITS));
    int64_t rps = ((N + ns - 1) / ns + KNN_T - 1) / KNN_T * KNN_T;
    if (rps < KNN_T) rps = KNN_T;
    p.rows_per_split = rps;
    p.nsplit = int(std::max<int64_t>(1, (N + rps - 1) / rps));
    p.part_slots = p.nsplit > 1 ? size_t(p.nsplit) * size_t(M) * 16 : 0;
    return p;
}

template <int KL>
static void knn_launch_tiles(const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx, int D,
                             const KnnPlan& p, int has_bound, float* last_d2, unsigned* last_i, float* part_d,
                             unsigned* part_i, int64_t* idx, int64_t ldi, float* dist, int64_t ldd, int col0,
                             int kcount, hipStream_t st) {
    const int64_t qtiles = (M + KNN_T - 1) / KNN_T;
    hipLaunchKernelGGL(knn_tile_kernel<KL>, dim3((unsigned)qtiles, (unsigned)p.nsplit), dim3(256), 0, st, Q, M, ldq, X,
                       N, ldx, D, p.rows_per_split, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, dist, ldd,
                       col0, kcount);
}

template <int KL, int H>
static void knn_launch_mfma(bool vec, const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx,
                            int D, const float* xn, const KnnPlan& p, int has_bound, float* last_d2, unsigned* last_i,
                            float* part_d, unsigned* part_i, int64_t* idx, int64_t ldi, float* dist, int64_t ldd,
                            int col0, int kcount, hipStream_t st) {
    const dim3 grid((unsigned)((M + 127) / 128), (unsigned)p.nsplit);
    if (vec)
        hipLaunchKernelGGL((knn_mfma_lds_kernel<KL, H>), grid, dim3(256), 0, st, Q, M, ldq, X, N, ldx, D, xn,
                           p.rows_per_split, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, dist, ldd, col0,
                           kcount);
    else
        hipLaunchKernelGGL((knn_mfma_kernel<KL, H, false>), grid, dim3(256), 0, st, Q, M, ldq, X, N, ldx, D, xn,
                           p.rows_per_split, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, dist, ldd, col0,
                           kcount);
}

bool knn_uses_mfma(int32_t D) { return D >= 16 && D <= 128; }

int launch_knn(const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx, int32_t D, int32_t k,
               int64_t* idx, int64_t ldi, float* dist, int64_t ldd, float* xn, float* last_d2, unsigned* last_i,
               float* part_d, unsigned* part_i, hipStream_t st) {
    if (M == 0) return HKM_OK;
    const KnnPlan p = knn_plan(M, N, knn_target_workgroups(D));
    const bool mfma = knn_uses_mfma(D);
    // list length: the smallest instantiated one that holds k (an insertion costs five instructions per slot)
    const int KL = mfma ? (k <= 6 ? 6 : k <= 8 ? 8 : 16) : (k <= 4 ? 4 : (k <= 8 ? 8 : 16));
    int rc;
    if (mfma) {
        hipLaunchKernelGGL(knn_norms_kernel, dim3((unsigned)((N + 15) / 16)), dim3(256), 0, st, X, N, ldx, D, xn);
        if ((rc = check_launch("knn_norms_kernel"))) return rc;
    }
    const bool vec = D % 4 == 0 && ldq % 4 == 0 && ldx % 4 == 0 &&
                     ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(X)) & 15u) == 0;
    for (int col0 = 0; col0 < k; col0 += KL) {
        const int kcount = std::min(KL, k - col0);
        const int has_bound = col0 > 0;
#define HKM_KNN_MFMA(KLV, HV)                                                                                        \
    knn_launch_mfma<KLV, HV>(vec, Q, M, ldq, X, N, ldx, D, xn, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, \
                             dist, ldd, col0, kcount, st)
        if (mfma) {
            const int H = D <= 16 ? 8 : (D <= 32 ? 16 : (D <= 64 ? 32 : 64));
            if (KL == 6) {
                if (H == 8) HKM_KNN_MFMA(6, 8);
                else if (H == 16) HKM_KNN_MFMA(6, 16);
                else if (H == 32) HKM_KNN_MFMA(6, 32);
                else HKM_KNN_MFMA(6, 64);
            } else if (KL == 8) {
                if (H == 8) HKM_KNN_MFMA(8, 8);
                else if (H == 16) HKM_KNN_MFMA(8, 16);
                else if (H == 32) HKM_KNN_MFMA(8, 32);
                else HKM_KNN_MFMA(8, 64);
            } else {
                if (H == 8) HKM_KNN_MFMA(16, 8);
                else if (H == 16) HKM_KNN_MFMA(16, 16);
                else if (H == 32) HKM_KNN_MFMA(16, 32);
                else HKM_KNN_MFMA(16, 64);
            }
            if ((rc = check_launch("knn_mfma_kernel"))) return rc;
        } else {
            if (KL == 4)
                knn_launch_tiles<4>(Q, M, ldq, X, N, ldx, D, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi,
                                    dist, ldd, col0, kcount, st);
            else if (KL == 8)
                knn_launch_tiles<8>(Q, M, ldq, X, N, ldx, D, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi,
                                    dist, ldd, col0, kcount, st);
            else
                knn_launch_tiles<16>(Q, M, ldq, X, N, ldx, D, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi,
                                     dist, ldd, col0, kcount, st);
            if ((rc = check_launch("knn_tile_kernel"))) return rc;
        }
#undef HKM_KNN_MFMA
        if (p.nsplit > 1) {
            hipLaunchKernelGGL(knn_merge_kernel, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, st, part_d, part_i,
                               p.nsplit, KL, M, last_d2, last_i, idx, ldi, dist, ldd, col0, kcount);
            if ((rc = check_launch("knn_merge_kernel"))) return rc;
        }
    }
    return HKM_OK;
}

int launch_knn_vote(const int64_t* idx, int64_t M, int32_t k, int64_t ldi, const float* Y, int64_t N, int32_t C,
                    int64_t ldy, int64_t* classes, hipStream_t st) {
    if (M == 0) return HKM_OK;
    hipLaunchKernelGGL(knn_vote_kernel, dim3((unsigned)((M + 3) / 4)), dim3(256), 0, st, idx, M, k, ldi, Y, N, C, ldy,
                       classes);
    return check_launch("knn_vote_kernel");
}

}  // namespace hkm
