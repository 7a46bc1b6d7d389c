// k nearest rows without the distance matrix: the cdist -> topk(largest=False) -> label vote chain of
// heat/classification/kneighborsclassifier.py:114-132.
//
//   * knn_tile_kernel: a workgroup owns 64 query rows and walks its share of the reference rows in
//     tiles of 64 (4 x 4 register block per lane, both tiles staged through LDS in chunks of 16
//     features, sum (q - r)^2 in fp32 -- the direct form, no cancellation).  Every lane keeps the KL
//     best (distance, row) pairs of its four query rows, sorted, in registers; a candidate is only
//     looked at when it beats the row's threshold, the smallest KL-th entry among the 16 lanes that
//     share the row (that lane alone holds KL closer rows, so nothing above it can rank).  At the end
//     the 16 lists of a row are merged with shuffles.  Reference rows can be split over several
//     workgroups (grid.y); their lists are merged by knn_merge_kernel.  More than KL neighbours are
//     found in passes: a pass only admits pairs that rank after the last pair of the pass before.
//   * order: ascending (squared distance, row index) -- the first row wins exact ties.
//   * knn_vote_kernel: sum of the label rows of the k neighbours, argmax with the first class on ties.
//
// Bound: the vector ALU, 2 operations (subtract, fused multiply-add) per (query, row, feature).
#include "hkm_common.h"

namespace hkm {

static constexpr int KNN_T = 64;
static constexpr int KNN_KC = 16;
static constexpr int KNN_MAX_SPLITS = 64;
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
            for (int w = 1; w < 16; w <<= 1) thr = fminf(thr, __shfl_xor(thr, w));
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int64_t gj = j0 + tx * 4 + b;
                const float d = acc[a][b];
                bool ok = gj < r_end && d < thr;
                if (has_bound) ok = ok && (d > bd[a] || (d == bd[a] && unsigned(gj) > bi[a]));
                if (ok) knn_insert<KL>(ld[a], li[a], d, unsigned(gj));
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
KnnPlan knn_plan(int64_t M, int64_t N) {
    KnnPlan p;
    const int64_t qtiles = (M + KNN_T - 1) / KNN_T;
    int64_t ns = qtiles > 0 ? (2048 + qtiles - 1) / qtiles : 1;
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

int launch_knn(const float* Q, int64_t M, int64_t ldq, const float* X, int64_t N, int64_t ldx, int32_t D, int32_t k,
               int64_t* idx, int64_t ldi, float* dist, int64_t ldd, float* last_d2, unsigned* last_i, float* part_d,
               unsigned* part_i, hipStream_t st) {
    if (M == 0) return HKM_OK;
    const KnnPlan p = knn_plan(M, N);
    const int KL = k <= 4 ? 4 : (k <= 8 ? 8 : 16);
    for (int col0 = 0; col0 < k; col0 += KL) {
        const int kcount = std::min(KL, k - col0);
        const int has_bound = col0 > 0;
        if (KL == 4)
            knn_launch_tiles<4>(Q, M, ldq, X, N, ldx, D, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, dist,
                                ldd, col0, kcount, st);
        else if (KL == 8)
            knn_launch_tiles<8>(Q, M, ldq, X, N, ldx, D, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, dist,
                                ldd, col0, kcount, st);
        else
            knn_launch_tiles<16>(Q, M, ldq, X, N, ldx, D, p, has_bound, last_d2, last_i, part_d, part_i, idx, ldi, dist,
                                 ldd, col0, kcount, st);
        int rc = check_launch("knn_tile_kernel");
        if (rc) return rc;
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
