// Full matrix of quadratic-expansion distances on the fp32 matrix cores, for the public cdist / rbf
// API with quadratic_expansion=True (heat/spatial/distance.py:47-64, 136-183):
//   out[i][j] = f( max(0, (|x_i|^2 + |y_j|^2) - 2 x_i.y_j) ),  f = identity, sqrt or exp(-. / 2 sigma^2).
//
// A (persistent) workgroup owns one 128 x 128 tile of the output at a time; its four waves form a 2 x 2 grid of 64 x 64
// sub-tiles (2 x 2 blocks of v_mfma_f32_32x32x2_f32).  The A operand carries rows of X, the B operand
// rows of Y: in the accumulator a lane then owns ONE column j (lane % 32) and 16 rows i, so a store
// instruction writes two runs of 32 consecutive floats -- whole 128-byte lines of the row-major
// output.  Features are consumed in chunks of 32; both operand panels of a chunk are fetched one
// chunk ahead with 16-byte loads (workgroup-uniform base + per-thread offset, no vector address
// arithmetic in the loop) and staged through double-buffered LDS (row stride 36 floats keeps the
// 16-byte operand reads conflict-free).  The squared norms are accumulated by the staging threads
// from the registers they stage.  The epilogue follows the reference's order: (|x|^2 + |y|^2) first,
// then - 2 x.y, clamp at 0 (NaN passes through), then sqrt / exp.  Every vector instruction of the
// epilogue takes issue time from the fp32 matrix pipe, so it is kept short: one compare + select for
// the clamp, and the square root in its short correctly rounded form (sqrt_rn_short) unless a wave
// holds a positive value below that form's range.
#include "hkm_common.h"

namespace hkm {

#define MFMA32(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)

static constexpr int CM_T = 128;   // tile edge
static constexpr int CM_DC = 32;   // feature chunk
static constexpr int CM_LD = CM_DC + 4;

__device__ __forceinline__ floatx4 cm_ld4(const float* p) { return *reinterpret_cast<const floatx4*>(p); }

// FULL: the tile lies inside the matrix (no guards on the stores); EPI: 0 squared distance, 1 sqrt with
// the short form above, 2 exp(-d2 * gauss), 3 sqrt by the library routine (any input)
template <bool FULL, int EPI>
__device__ __forceinline__ void cm_store_values(const floatx16 (&acc)[2][2], float* __restrict__ out_tile,
                                                int64_t ldo, int wx, int wy, int p, int h, int rows_left,
                                                int cols_left, float gauss) {
    // byte offset of this lane inside the tile, without the block / register terms (those are uniform)
    const unsigned lane_off = unsigned(((wx * 64 + 4 * h) * ldo + wy * 64 + p) * 4);
#pragma unroll
    for (int xb = 0; xb < 2; ++xb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            // rows 8g + 4h .. + 3 of the block: registers 4g .. 4g + 3
            const int r0 = wx * 64 + xb * 32 + 8 * g + 4 * h;
            float d[4][2];
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int yb = 0; yb < 2; ++yb) {
                    float t = acc[xb][yb][4 * g + q];
                    if (EPI == 2) t = expf(-t * gauss);
                    else if (EPI == 1) t = sqrt_rn_short(t);
                    else if (EPI == 3) t = sqrtf(t);
                    d[q][yb] = t;
                }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float* rowp = out_tile + int64_t(xb * 32 + 8 * g + q) * ldo;  // uniform
#pragma unroll
                for (int yb = 0; yb < 2; ++yb)
                    if (FULL || (r0 + q < rows_left && wy * 64 + yb * 32 + p < cols_left))
                        *reinterpret_cast<float*>(reinterpret_cast<char*>(rowp + yb * 32) + lane_off) = d[q][yb];
            }
        }
}

template <bool FULL, int EPI>
__device__ __forceinline__ void cm_store_tile(floatx16 (&acc)[2][2], const float* sXn, const float* sYn,
                                              float* __restrict__ out_tile, int64_t ldo, int wx, int wy, int p,
                                              int h, int rows_left, int cols_left, float gauss) {
    // squared distances in place, in the reference's order: (|x|^2 + |y|^2) first, then - 2 x.y, then
    // the clamp at 0.  A NaN passes through (NaN < 0 is false); the value is never -0 (the sum of
    // the norms is never -0), so the comparison form equals clamp(min=0) on every input.
    const float yn[2] = {sYn[wy * 64 + p], sYn[wy * 64 + 32 + p]};
#pragma unroll
    for (int xb = 0; xb < 2; ++xb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const floatx4 xn4 = cm_ld4(sXn + wx * 64 + xb * 32 + 8 * g + 4 * h);
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int yb = 0; yb < 2; ++yb) {
                    const float t = fmaf(-2.0f, acc[xb][yb][4 * g + q], xn4[q] + yn[yb]);
                    acc[xb][yb][4 * g + q] = t < 0.0f ? 0.0f : t;
                }
        }
    if (EPI == 1) {
        // the short square root covers 0 and everything from 2^-96 up; a wave whose smallest POSITIVE
        // value lies below takes the library routine for its whole sub-tile.  As unsigned integers
        // (bits - 1) orders the non-negative floats with zero moved to the top, so one integer
        // minimum tree finds the smallest positive value (a NaN sits above every finite value).
        unsigned m = 0xffffffffu;
#pragma unroll
        for (int xb = 0; xb < 2; ++xb)
#pragma unroll
            for (int yb = 0; yb < 2; ++yb)
#pragma unroll
                for (int v = 0; v < 16; v += 2)
                    m = min(m, min(sqrt_short_key(acc[xb][yb][v]), sqrt_short_key(acc[xb][yb][v + 1])));
        if (__builtin_amdgcn_ballot_w64(m < SQRT_SHORT_KEY_LIMIT) != 0) {  // some 0 < t < 2^-96 in the wave
            cm_store_values<FULL, 3>(acc, out_tile, ldo, wx, wy, p, h, rows_left, cols_left, gauss);
            return;
        }
    }
    cm_store_values<FULL, EPI>(acc, out_tile, ldo, wx, wy, p, h, rows_left, cols_left, gauss);
}

template <bool VEC, int EPI>
__global__ __launch_bounds__(256, 2) void cdist_mfma_kernel(const float* __restrict__ X, int64_t M, int64_t ldx,
                                                         const float* __restrict__ Y, int64_t Nn, int64_t ldy,
                                                         int D, float* __restrict__ out, int64_t ldo,
                                                         float gauss, int64_t tiles_n, int64_t total, int ndc) {
    __shared__ __align__(16) float sA[2][CM_T * CM_LD];  // rows of X
    __shared__ __align__(16) float sB[2][CM_T * CM_LD];  // rows of Y
    __shared__ float sXn[CM_T], sYn[CM_T];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wx = wave & 1, wy = wave >> 1;  // this wave: rows [64 wx, +64) x columns [64 wy, +64) of the tile
    const int p = lane & 31, h = lane >> 5;
    // staging: rows sr + 32 q (q = 0..3) of both panels, column group sc; rows beyond the matrix are
    // clamped to its last row (their results are never stored)
    const int sr = tid >> 3, sc = (tid & 7) * 4;
    const float* baseA = X;
    const float* baseB = Y;
    unsigned offA[4], offB[4];
    auto set_tile = [&](int64_t t) {
        const int64_t i0 = (t / tiles_n) * CM_T, j0 = (t % tiles_n) * CM_T;
        baseA = X + i0 * ldx;
        baseB = Y + j0 * ldy;
        const int64_t lastA = M - 1 - i0, lastB = Nn - 1 - j0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int r = sr + 32 * q;
            const int ra = r < lastA ? r : int(lastA);
            const int rb = r < lastB ? r : int(lastB);
            offA[q] = unsigned((int64_t(ra) * ldx + sc) * 4);
            offB[q] = unsigned((int64_t(rb) * ldy + sc) * 4);
        }
    };
    floatx4 pa[4], pb[4];
    auto issue = [&](int dc) {
        const float* a = baseA + dc * CM_DC;
        const float* b = baseB + dc * CM_DC;
        if (VEC && dc * CM_DC + CM_DC <= D) {  // whole chunk inside the rows: unconditional 16-byte loads
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                pa[q] = *reinterpret_cast<const floatx4*>(reinterpret_cast<const char*>(a) + offA[q]);
                pb[q] = *reinterpret_cast<const floatx4*>(reinterpret_cast<const char*>(b) + offB[q]);
            }
        } else {
            const int c0 = dc * CM_DC + sc;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float* ra = reinterpret_cast<const float*>(reinterpret_cast<const char*>(a) + offA[q]);
                const float* rb = reinterpret_cast<const float*>(reinterpret_cast<const char*>(b) + offB[q]);
                floatx4 va = {0.f, 0.f, 0.f, 0.f}, vb = {0.f, 0.f, 0.f, 0.f};
                if (VEC) {
                    if (c0 < D) {
                        va = cm_ld4(ra);
                        vb = cm_ld4(rb);
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (c0 + t < D) {
                            va[t] = ra[t];
                            vb[t] = rb[t];
                        }
                }
                pa[q] = va;
                pb[q] = vb;
            }
        }
    };

    // persistent workgroup: tiles blockIdx.x, + gridDim.x, ...; the loop runs over (tile, chunk) steps so
    // that the first chunk of the NEXT tile is already on its way while a tile's results are stored
    const int64_t my_tiles = int64_t(blockIdx.x) < total ? (total - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const int64_t nsteps = my_tiles * ndc;
    int64_t tile = blockIdx.x;
    int dc = 0;
    floatx16 acc[2][2];
    float xsq[4] = {0.f, 0.f, 0.f, 0.f}, ysq[4] = {0.f, 0.f, 0.f, 0.f};
    // registers of the chunk in flight -> LDS buffer `buf`, squared norms accumulated on the way
    auto stage = [&](int buf) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            *reinterpret_cast<floatx4*>(&sA[buf][(sr + 32 * q) * CM_LD + sc]) = pa[q];
            *reinterpret_cast<floatx4*>(&sB[buf][(sr + 32 * q) * CM_LD + sc]) = pb[q];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                xsq[q] = fmaf(pa[q][t], pa[q][t], xsq[q]);
                ysq[q] = fmaf(pb[q][t], pb[q][t], ysq[q]);
            }
        }
    };
    if (nsteps > 0) {
        set_tile(tile);
        issue(0);
        if (my_tiles >= 16) {
            // Stagger the start.  Workgroups launched together would run their store phases together:
            // the matrix cores idle while the whole chip stores, and the memory system idles while it
            // computes.  Sixteen start phases across one tile period (about 10 000 cycles per chunk
            // with two workgroups sharing a CU) spread the stores evenly over time; workgroups b and
            // b + 256, which tend to share a CU, start half a period apart.  Costs at most one tile
            // time of the my_tiles a workgroup processes.
            const int phase = (((blockIdx.x >> 3) & 7) + 8 * ((blockIdx.x >> 8) & 1)) & 15;
            for (int i = 0; i < phase * ndc; ++i) __builtin_amdgcn_s_sleep(10);  // 640 cycles each
        }
        stage(0);
    }
    // One barrier per step: it publishes the chunk staged at the end of the previous step and retires
    // every read of the other buffer.  The chunk of the NEXT step is requested right after it and moved
    // to LDS after this step's MFMAs -- before a tile's results are stored, so that no wait for loaded
    // data ever has those stores ahead of it in the memory queue (loads and stores share one counter).
    for (int64_t it = 0; it < nsteps; ++it) {
        const int buf = int(it & 1);
        __syncthreads();

        const int64_t cur_tile = tile;
        const int cur_dc = dc;
        const bool more = it + 1 < nsteps;
        if (++dc == ndc) {
            dc = 0;
            tile += gridDim.x;
            if (more) set_tile(tile);
        }
        if (more) issue(dc);

        if (cur_dc == 0) {
#pragma unroll
            for (int xb = 0; xb < 2; ++xb)
#pragma unroll
                for (int yb = 0; yb < 2; ++yb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[xb][yb][v] = 0.f;
        }

        // this lane-half's 16 features of the chunk, for both operands
        floatx4 b[2][4];
#pragma unroll
        for (int yb = 0; yb < 2; ++yb) {
            const float* brow = &sB[buf][(wy * 64 + yb * 32 + p) * CM_LD + h * 16];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[yb][j] = cm_ld4(brow + 4 * j);
        }
#pragma unroll
        for (int xb = 0; xb < 2; ++xb) {
            const float* arow = &sA[buf][(wx * 64 + xb * 32 + p) * CM_LD + h * 16];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const floatx4 a = cm_ld4(arow + 4 * j);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int yb = 0; yb < 2; ++yb) acc[xb][yb] = MFMA32(a[t], b[yb][j][t], acc[xb][yb]);
            }
        }

        const bool last = cur_dc == ndc - 1;
        if (last) {
            // squared norms of the tile's rows of X and Y: the eight threads that staged a row add their
            // parts (the previous tile's readers of sXn / sYn are behind this step's barrier)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float vx = xsq[q], vy = ysq[q];
                vx += __shfl_xor(vx, 1);
                vy += __shfl_xor(vy, 1);
                vx += __shfl_xor(vx, 2);
                vy += __shfl_xor(vy, 2);
                vx += __shfl_xor(vx, 4);
                vy += __shfl_xor(vy, 4);
                if ((tid & 7) == 0) {
                    sXn[sr + 32 * q] = vx;
                    sYn[sr + 32 * q] = vy;
                }
                xsq[q] = 0.f;
                ysq[q] = 0.f;
            }
        }
        if (more) stage(buf ^ 1);
        if (last) {
            __syncthreads();
            const int64_t i0 = (cur_tile / tiles_n) * CM_T, j0 = (cur_tile % tiles_n) * CM_T;
            float* out_tile = out + i0 * ldo + j0;
            const int rows_left = int(M - i0 < CM_T ? M - i0 : CM_T), cols_left = int(Nn - j0 < CM_T ? Nn - j0 : CM_T);
            if (rows_left == CM_T && cols_left == CM_T)
                cm_store_tile<true, EPI>(acc, sXn, sYn, out_tile, ldo, wx, wy, p, h, rows_left, cols_left, gauss);
            else
                cm_store_tile<false, EPI>(acc, sXn, sYn, out_tile, ldo, wx, wy, p, h, rows_left, cols_left, gauss);
        }
    }
}

// true if the matrix-core kernel takes this call (the caller falls back to the vector kernel otherwise)
bool cdist_mfma_eligible(int64_t M, int64_t Nn, int32_t D, int64_t ldx, int64_t ldy, int64_t ldo) {
    // worth it from 16 features on; per-thread offsets inside a tile are 32-bit byte offsets
    const int64_t lim = (int64_t(1) << 31) / 4 / CM_T;
    const int64_t tiles = ((M + CM_T - 1) / CM_T) * ((Nn + CM_T - 1) / CM_T);
    return D >= 16 && ldx < lim && ldy < lim && ldo < lim && tiles <= 0x7fffffffLL;
}

int launch_cdist_mfma(const float* X, int64_t M, int64_t ldx, const float* Y, int64_t Nn, int64_t ldy,
                      int32_t D, float* out, int64_t ldo, int32_t sqrt_flag, float gauss, hipStream_t st) {
    const int64_t tiles_m = (M + CM_T - 1) / CM_T, tiles_n = (Nn + CM_T - 1) / CM_T;
    const int64_t total = tiles_m * tiles_n;
    const int ndc = (D + CM_DC - 1) / CM_DC;
    const bool vec = aligned16(X) && aligned16(Y) && (ldx % 4 == 0) && (ldy % 4 == 0) && (D % 4 == 0);
    const int epi = gauss != 0.f ? 2 : (sqrt_flag ? 1 : 0);
    int64_t grid = int64_t(num_cus()) * 2;  // two workgroups per CU (LDS), persistent
    if (grid > total) grid = total;
#define HKM_GO(V, E)                                                                                      \
    hipLaunchKernelGGL((cdist_mfma_kernel<V, E>), dim3((unsigned)grid), dim3(256), 0, st, X, M, ldx, Y, Nn, \
                       ldy, D, out, ldo, gauss, tiles_n, total, ndc)
    if (vec) {
        if (epi == 2) HKM_GO(true, 2);
        else if (epi == 1) HKM_GO(true, 1);
        else HKM_GO(true, 0);
    } else {
        if (epi == 2) HKM_GO(false, 2);
        else if (epi == 1) HKM_GO(false, 1);
        else HKM_GO(false, 0);
    }
#undef HKM_GO
    return check_launch("cdist_mfma_kernel");
}

}  // namespace hkm
