// Fused distance + argmin on the fp32 matrix cores (v_mfma_f32_32x32x2_f32): the assignment alone for D >= 4
// (up to 16 features only from 32 centroids on), the one-sweep step for D >= 2 whatever K is.
//
// Operand roles: the A operand (M = 32 rows) carries CENTROIDS, the B operand (N = 32 columns)
// carries POINTS.  In the 32x32 accumulator a lane then owns one point (column lane%32) and 16
// centroid rows (8*(v/4) + 4*(lane/32) + v%4 for register v), so the min/argmin over centroids is a
// scan over the lane's own registers, followed by ONE exchange between lane and lane^32.
//
// The contraction index is permuted: lane-half h feeds k = h*DP/2 + 4j + t at step (j, t), which
// lets both operands be fetched as 16-byte vectors.  A and B use the same permutation, so every k
// is consumed exactly once.
//
// Arithmetic mirrors heat/spatial/distance.py:59-64: d2 = (|x|^2 + |c|^2) - 2*(x.c), clamped at 0;
// first index wins ties (torch.min, heat/core/statistics.py:177).
#include <pthread.h>
#include <time.h>

#include "hkm_common.h"
#include "hkm_mfma_util.h"

namespace hkm {

// ------------------------------------------------------------------------------------------------
// Resident variant: the whole centroid matrix and its squared norms live in LDS for the lifetime of
// a persistent workgroup; each wave streams its own 32*PB points from global memory straight into
// B-operand registers.  No barrier inside the tile loop.
//
// On this hardware every VALU instruction takes issue time away from the fp32 MFMA pipe (there is no
// co-execution), so the epilogue is kept short (about 1.3 VALU instructions per distance):
//   * LDS row k holds -2*c_k (zero-padded to DP; scaling by -2 is exact) and a separate LDS array the
//     squared norms |c_k|^2; the accumulators of a block START at the norms of their centroid rows
//     (the C operand of the first MFMA, four 16-byte LDS reads, no vector instruction), so they end
//     as |c|^2 - 2 x.c.  |x|^2 is the same for every centroid: it is added to the minimum only;
//   * the clamp at 0 is applied lazily: only if some running minimum went negative (a point that
//     coincides with a centroid up to rounding) the tile is rescanned with the clamp on every value;
//   * per block of 16 values a tree of three-input minima; if that improves the running minimum the
//     block is only remembered (its number and a copy of the 16 values: ten instructions), and the
//     position of the minimum is looked up by equality once per point, in the copy that survived the
//     last block (block_min_keep / kept_argmin).  The lane-half term of the index is added once per
//     tile.
// ------------------------------------------------------------------------------------------------
// One centroid block (32 rows) against the wave's PB point blocks: DP/2 MFMAs per point block.  The
// accumulators start at the squared norms of the lane's 16 centroid rows (cn16 points at the norm of
// row 4*h of the block; rows 8g + 4h .. 8g + 4h + 3 belong to accumulator elements 4g .. 4g + 3), so
// they end as |c|^2 - 2 x.c: the distance without the term |x|^2, which is the same for every centroid.
template <int DP, int PB>
__device__ __forceinline__ void resident_block(const float* arow, const floatx16& c0, int h,
                                               const floatx4 (&b)[PB][DP / 8], floatx16 (&acc)[PB]) {
    constexpr int NJ = DP / 8;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const floatx4 a = ld4(arow + h * (DP / 2) + 4 * j);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb)
                acc[pb] = (j == 0 && t == 0) ? MFMA32(a[t], b[pb][j][t], c0) : MFMA32(a[t], b[pb][j][t], acc[pb]);
    }
}

// The same with the block's A fragments already in registers (the centroids never change during a launch, so
// a wave with registers to spare keeps its first blocks' fragments for good instead of reading them from LDS
// for every tile).
template <int DP, int PB>
__device__ __forceinline__ void resident_block_regs(const floatx4 (&a)[DP / 8], const floatx16& c0,
                                                    const floatx4 (&b)[PB][DP / 8], floatx16 (&acc)[PB]) {
    constexpr int NJ = DP / 8;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb)
                acc[pb] = (j == 0 && t == 0) ? MFMA32(a[j][t], b[pb][j][t], c0) : MFMA32(a[j][t], b[pb][j][t], acc[pb]);
}

// Two centroid blocks at once against one point block: two independent accumulator chains share the
// point registers, so a wave always has a matrix instruction that does not wait for the one before it,
// and the first block's minimum tree finds its results complete while the second chain ends.
template <int DP>
__device__ __forceinline__ void resident_block_pair(const float* arow0, const float* arow1, const floatx16& c0,
                                                    const floatx16& c1, int h, const floatx4 (&b)[DP / 8],
                                                    floatx16& acc0, floatx16& acc1) {
    constexpr int NJ = DP / 8;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const floatx4 a0 = ld4(arow0 + h * (DP / 2) + 4 * j);
        const floatx4 a1 = ld4(arow1 + h * (DP / 2) + 4 * j);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            acc0 = (j == 0 && t == 0) ? MFMA32(a0[t], b[j][t], c0) : MFMA32(a0[t], b[j][t], acc0);
            acc1 = (j == 0 && t == 0) ? MFMA32(a1[t], b[j][t], c1) : MFMA32(a1[t], b[j][t], acc1);
        }
    }
}

// Scan of all centroid blocks.  CLAMP applies max(. + |x|^2, 0) to every value (the rescan of a tile
// whose lazy minimum came out negative).  Two blocks per trip: the squared norms of both are requested
// at the top of the trip into the registers that then serve, in place, as their accumulators (norms
// carried over the loop's back edge instead were copied into place, eight moves per block).
// RB > 0 (even; two point blocks only): the A fragments of blocks 0 .. RB - 1 come from `ares` instead of LDS.
template <int DP, int PB, bool CLAMP, int RB = 0>
__device__ __forceinline__ void resident_scan(const float* sC, const float* sCn, int ncb, int p, int h,
                                              const floatx4 (&b)[PB][DP / 8],
                                              const float (&xn)[PB], float (&m)[PB],
                                              int (&mi)[PB],
                                              const floatx4 (*ares)[DP / 8] = nullptr) {
    constexpr int LDC = DP + 4;
    int blk[PB];
    floatx16 keep[PB];
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) {
        m[pb] = HKM_INF;
        blk[pb] = 0;
        keep_undefined(keep[pb]);
    }
    auto one_block = [&](int cb, const floatx16& c0) {
        floatx16 acc[PB];
        resident_block<DP, PB>(sC + (cb * 32 + p) * LDC, c0, h, b, acc);
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            if (CLAMP) {
                // the full distance (|x|^2 + (|c|^2 - 2 x.c)) clamped at 0, as the reference orders them
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[pb][v] = fmaxf(acc[pb][v] + xn[pb], 0.0f);
            }
            block_min_keep(acc[pb], cb, m[pb], blk[pb], keep[pb]);
        }
    };
    if (PB == 1) {
        int cb = 0;
        for (; cb + 1 < ncb; cb += 2) {
            const floatx16 c0 = load_cn16(sCn + cb * 32 + 4 * h);
            const floatx16 c1 = load_cn16(sCn + (cb + 1) * 32 + 4 * h);
            floatx16 acc0, acc1;
            resident_block_pair<DP>(sC + (cb * 32 + p) * LDC, sC + ((cb + 1) * 32 + p) * LDC, c0, c1, h, b[0], acc0, acc1);
            if (CLAMP) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc0[v] = fmaxf(acc0[v] + xn[0], 0.0f);
                    acc1[v] = fmaxf(acc1[v] + xn[0], 0.0f);
                }
            }
            block_min_keep(acc0, cb, m[0], blk[0], keep[0]);
            block_min_keep(acc1, cb + 1, m[0], blk[0], keep[0]);
        }
        if (cb < ncb) one_block(cb, load_cn16(sCn + cb * 32 + 4 * h));
    } else {
        int cb = 0;
        if constexpr (RB > 0) {
#pragma unroll
            for (int r = 0; r < RB; r += 2) {
                if (r < ncb) {
                    const floatx16 ca = load_cn16(sCn + r * 32 + 4 * h);
                    const floatx16 cb1 = load_cn16(sCn + (r + 1 < ncb ? r + 1 : r) * 32 + 4 * h);
                    floatx16 acc[PB];
                    resident_block_regs<DP, PB>(ares[r], ca, b, acc);
#pragma unroll
                    for (int pb = 0; pb < PB; ++pb) block_min_keep(acc[pb], r, m[pb], blk[pb], keep[pb]);
                    if (r + 1 < ncb) {
                        resident_block_regs<DP, PB>(ares[r + 1], cb1, b, acc);
#pragma unroll
                        for (int pb = 0; pb < PB; ++pb) block_min_keep(acc[pb], r + 1, m[pb], blk[pb], keep[pb]);
                    }
                }
            }
            cb = RB;
        }
        for (; cb < ncb; cb += 2) {
            const floatx16 ca = load_cn16(sCn + cb * 32 + 4 * h);
            const floatx16 cb1 = load_cn16(sCn + (cb + 1 < ncb ? cb + 1 : cb) * 32 + 4 * h);
            one_block(cb, ca);
            if (cb + 1 < ncb) one_block(cb + 1, cb1);
        }
    }
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) {
        mi[pb] = kept_argmin(keep[pb], m[pb], blk[pb]);
        // without CLAMP the minimum still lacks |x|^2
        if (!CLAMP) m[pb] += xn[pb];
    }
}

// The rows of one tile for a wave: PB blocks of 32 rows starting at row0 (wave-uniform), a lane takes the
// DP/2 columns of its half of row p of each block.  Whole tiles of whole, aligned rows (`fast`, decided
// once per kernel) are addressed as a wave-uniform base plus a 32-bit lane offset, so a tile costs no
// vector address arithmetic; the ragged last tile and narrow or unaligned rows take the general path
// (row index clamped to N - 1, columns beyond D read as zero).
template <int DP, int PB, bool VEC>
__device__ __forceinline__ void fetch_rows(const float* __restrict__ X, int64_t N, int D, int64_t ldx, int64_t row0,
                                           int p, int h, bool fast, unsigned lane_off,
                                           floatx4 (&dst)[PB][DP / 8]) {
    constexpr int NJ = DP / 8;
    if (fast && row0 + PB * 32 <= N) {
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            const char* base = reinterpret_cast<const char*>(X + (row0 + pb * 32) * ldx);
#pragma unroll
            for (int j = 0; j < NJ; ++j) dst[pb][j] = *reinterpret_cast<const floatx4*>(base + lane_off + 16 * j);
        }
    } else {
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            int64_t r = row0 + pb * 32 + p;
            r = r < N ? r : N - 1;
            const float* xr = X + r * ldx;
#pragma unroll
            for (int j = 0; j < NJ; ++j) dst[pb][j] = load_row4<VEC>(xr, h * (DP / 2) + 4 * j, D);
        }
    }
}

template <int DP, int PB, bool VEC>
__global__ __launch_bounds__(256) void assign_mfma_resident_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, int32_t* __restrict__ labels, float* __restrict__ min_d2, int64_t ntiles) {
    extern __shared__ __align__(16) float lds[];
    constexpr int LDC = DP + 4;  // row: DP scaled coordinates, |c|^2, 1, 2 pad; also keeps 16-B reads conflict-free
    constexpr int NJ = DP / 8;   // 16-byte groups per lane-half
    const int KP = (K + 31) & ~31;
    float* sC = lds;              // [KP][LDC]
    float* sCn = lds + KP * LDC;  // [KP] squared norms
    const int tid = threadIdx.x;

    for (int i = tid; i < KP * DP; i += 256) {
        const int r = i / DP, c = i - r * DP;
        sC[r * LDC + c] = (r < K && c < D) ? -2.0f * C[int64_t(r) * ldc + c] : 0.f;
    }
    for (int r = tid; r < KP; r += 256) {
        float s = HKM_INF;  // padding rows can never win
        if (r < K) {
            s = 0.f;
            const float* c = C + int64_t(r) * ldc;
            for (int d = 0; d < D; ++d) s = fmaf(c[d], c[d], s);
        }
        sCn[r] = s;
    }
    __syncthreads();

    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int p = lane & 31, h = lane >> 5;
    const int ncb = KP >> 5;
    const bool fast = VEC && D == DP && ldx < (int64_t(1) << 24);
    const unsigned lane_off = unsigned((int64_t(p) * ldx + h * (DP / 2)) * 4);

    // One tile: the rows of the next one are requested (into the other of two register sets, which swap
    // roles from tile to tile) before this one is scanned.
    auto step = [&](int64_t tile, const floatx4 (&b)[PB][NJ], floatx4 (&bnext)[PB][NJ]) {
        const int64_t row0 = tile * (4 * PB * 32) + wave * (PB * 32);
        float xn[PB], m[PB];
        int mi[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) s = fmaf(b[pb][j][t], b[pb][j][t], s);
            xn[pb] = s + __shfl_xor(s, 32);
        }
        if (tile + gridDim.x < ntiles)
            fetch_rows<DP, PB, VEC>(X, N, D, ldx, row0 + int64_t(gridDim.x) * (4 * PB * 32), p, h, fast, lane_off, bnext);

        resident_scan<DP, PB, false>(sC, sCn, ncb, p, h, b, xn, m, mi);
        bool neg = false;
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) neg |= m[pb] < 0.f;
        if (__any(neg)) resident_scan<DP, PB, true>(sC, sCn, ncb, p, h, b, xn, m, mi);

#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            mi[pb] += 4 * h;
            merge_halves(m[pb], mi[pb]);
            const int64_t rb = row0 + pb * 32;  // wave-uniform: the stores take it as their scalar base
            if (h == 0 && rb + p < N) {
                labels[rb + p] = mi[pb];
                if (min_d2) min_d2[rb + p] = m[pb];
            }
        }
    };

    floatx4 b0[PB][NJ], b1[PB][NJ];
    if (int64_t(blockIdx.x) < ntiles)
        fetch_rows<DP, PB, VEC>(X, N, D, ldx, int64_t(blockIdx.x) * (4 * PB * 32) + wave * (PB * 32), p, h, fast,
                                lane_off, b0);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += 2 * int64_t(gridDim.x)) {
        step(tile, b0, b1);
        if (tile + gridDim.x < ntiles) step(tile + gridDim.x, b1, b0);
    }
}

// ------------------------------------------------------------------------------------------------
// One-sweep Lloyd step for the resident shapes: the same persistent kernel, and once the labels of a
// wave's points are final the point rows -- still in the B-operand registers -- are added to
// per-workgroup fp64 accumulators in LDS with ds_add_f64.  X is read from HBM once per iteration.
//
// Atomic additions arrive in any order, so the sums are made ORDER-INDEPENDENT instead: every row is
// first rounded to a multiple of q_i = 2^(E_i - 28), where 2^E_i bounds the row's largest
// coordinate (taken from |x_i|^2, which the distance needs anyway), by (v + B_i) - B_i with
// B_i = 1.5 * 2^52 * q_i.  All addends of a workgroup are then multiples of 2^(Emin - 28) and every
// partial sum is below n_wg * 2^Emax, so as long as Emax - Emin <= 53 - 28 - ceil(log2 n_wg) every
// addition is exact in fp64 and the result does not depend on the order.  The rounding keeps 28 bits
// below the row's largest coordinate (error <= 2^-29 of it per addend) -- or below a floor derived from the
// centroid norms, for rows far smaller than the centroids (see e_floor in the kernel).  A workgroup whose rows
// violate the range condition, or hold a row whose |x|^2 is inf or NaN (coordinates above 1.8e19 or
// non-finite ones: the bound 2^E is then meaningless), raises its flag; the step then falls back to
// the two-pass update, whose kernels start by looking at the flags.
// ------------------------------------------------------------------------------------------------
static constexpr int FUSED_QBITS = 28;
#ifndef HKM_RESIDENT_A_BLOCKS
#define HKM_RESIDENT_A_BLOCKS 4
#endif
// Point blocks per wave of the resident kernels.  Up to 32 padded features there is a choice: TWO point
// blocks against every centroid row a wave reads from LDS (eight waves per CU in the one-sweep kernel), or ONE
// with sixteen waves.  Two halve the LDS reads per matrix instruction, and that decides on chips that lower
// their clock under these kernels.  Measured on the 10M x 32 x 256 workload over a dozen chips of the same
// model: on those that hold 2.39 GHz one point block is 3 % faster (one-sweep kernel 1.326 against 1.366 ms);
// on those that do not it runs at 2.1-2.2 GHz and two point blocks at 2.3 GHz (1.45 against 1.39 ms).  Both
// geometries cut the rows into the same tiles of 512 and hand them to the same workgroups, so every output
// of a step is bit for bit the same whichever runs.  Which one: HKM_POINT_BLOCKS (1 or 2) if set; else what
// the trial below found on this device; else two.  Wider rows leave registers for one point block only
// (twelve waves).
__host__ __device__ constexpr int fused_threads(int pb, int dp) {
    return pb == 2 ? 512 : (dp <= 32 ? 1024 : dp <= 64 ? 768 : 512);  // beyond 64 features a wave needs 256 registers
}

int env_point_blocks() {
    const char* e = getenv("HKM_POINT_BLOCKS");
    if (e && (e[0] == '1' || e[0] == '2') && e[1] == 0) return e[0] - '0';
    return 0;
}

// ---- the trial: which geometry this chip runs faster, found on the caller's own steps ----------------
// Nothing extra is launched and nothing waits.  While a device has no verdict, the one-sweep steps of large
// fits (a million rows or more) that follow each other closely on one stream are taken in three windows of
// consecutive calls -- two point blocks, one, two again -- each long enough (about 30 ms of device time by
// the step's flop count) for the clock to settle under its geometry: a device coming out of idle needs some
// 30 ms of load to reach its clock, and a chip that lowers its clock under one geometry has done so 20 ms
// into it.  The last third of every window lies between two events on the stream.  Later calls look at the
// last event without waiting; once it has completed, one point block is kept if it beat the SECOND
// two-block window by at least 1 % (repeated timings differ by half a percent), else two.  A pause between
// two calls (the device may have gone idle), another shape or another stream starts the windows again, so a
// process that only ever runs short fits far apart keeps the default, where the choice is worth nothing
// anyway.  Both geometries write the same bits, so no result depends on any of this.  State: per device,
// process-wide, behind a mutex.
static const int TRIAL_MAX_DEVICES = 64;
static const int64_t TRIAL_MIN_ROWS = int64_t(1) << 20;
struct GeomTrial {
    pthread_mutex_t mu = PTHREAD_MUTEX_INITIALIZER;
    int decided = 0;        // 0: no verdict yet, else 1 or 2
    int window = 0;         // 0: two point blocks, 1: one, 2: two again; 3: all recorded, verdict pending
    int calls = 0;          // calls made in the current window
    int window_calls = 0;   // length of a window for the shape under trial
    int64_t n = 0;          // the shape and the stream under trial
    int d = 0, k = 0;
    hipStream_t stream = nullptr;
    double last_call = 0.;  // host clock at the previous call, seconds
    double gap = 0.;        // a longer pause than this between two calls starts over
    hipEvent_t ev[3][2] = {};
    bool have_events = false;
    float window_ms[3] = {0.f, 0.f, 0.f};  // per step, for the query
};
static GeomTrial g_trial[TRIAL_MAX_DEVICES];

static double host_seconds() {
    timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return double(ts.tv_sec) + 1e-9 * double(ts.tv_nsec);
}

static GeomTrial* trial_of_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TRIAL_MAX_DEVICES) return nullptr;
    return &g_trial[dev];
}

int tuned_point_blocks() {
    GeomTrial* t = trial_of_device();
    if (!t) return 0;
    pthread_mutex_lock(&t->mu);
    const int v = t->decided;
    pthread_mutex_unlock(&t->mu);
    return v;
}

int trial_report(float* ms_two, float* ms_one) {
    GeomTrial* t = trial_of_device();
    if (!t) return 0;
    pthread_mutex_lock(&t->mu);
    const int v = t->decided;
    if (ms_two) *ms_two = t->window_ms[2];
    if (ms_one) *ms_one = t->window_ms[1];
    pthread_mutex_unlock(&t->mu);
    return v;
}

int resident_point_blocks(int dp) {
    if (dp > 32) return 1;
    if (const int e = env_point_blocks()) return e;
    if (const int t = tuned_point_blocks()) return t;
    return 2;
}

// What the one-sweep launcher asks before and tells after its launch.  `end` is the event to record behind
// the launch (the last call of a window), or null.
struct TrialTicket {
    int pb = 2;
    hipEvent_t end = nullptr;
};

static void trial_restart(GeomTrial& t, int64_t N, int32_t D, int32_t K, hipStream_t st) {
    t.window = 0;
    t.calls = 0;
    t.n = N;
    t.d = D;
    t.k = K;
    t.stream = st;
    // the step's time from its flop count at about two thirds of the matrix peak: only sizes the windows
    const double kp = double((K + 31) / 32 * 32);
    const double est_ms = 2.0 * double(N) * kp * resident_dp(D) / 1.0e11;
    int c = int(30.0 / (est_ms > 1e-3 ? est_ms : 1e-3)) + 1;
    t.window_calls = c < 6 ? 6 : c > 600 ? 600 : c;
    t.gap = 1e-3 * (est_ms * 4.0 > 10.0 ? est_ms * 4.0 : 10.0);
}

static TrialTicket trial_begin(int64_t N, int32_t D, int32_t K, hipStream_t st) {
    TrialTicket tk;
    const int dp = resident_dp(D);
    if (dp > 32) {
        tk.pb = 1;
        return tk;
    }
    if (const int e = env_point_blocks()) {
        tk.pb = e;
        return tk;
    }
    GeomTrial* tp = trial_of_device();
    if (!tp) return tk;
    GeomTrial& t = *tp;
    pthread_mutex_lock(&t.mu);
    if (t.decided) {
        tk.pb = t.decided;
    } else if (N >= TRIAL_MIN_ROWS) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        const bool capturing = hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone;
        if (t.window == 3) {
            // every window is recorded: a look at the last event, no wait
            if (hipEventQuery(t.ev[2][1]) == hipSuccess) {
                bool ok = true;
                for (int w = 0; w < 3; ++w) {
                    float ms = 0.f;
                    ok = ok && hipEventElapsedTime(&ms, t.ev[w][0], t.ev[w][1]) == hipSuccess;
                    const int timed = t.window_calls / 3 > 2 ? t.window_calls / 3 : 2;
                    t.window_ms[w] = ms / float(timed);
                }
                if (ok && t.window_ms[1] > 0.f && t.window_ms[2] > 0.f) {
                    t.decided = t.window_ms[1] < 0.99f * t.window_ms[2] ? 1 : 2;
                    for (auto& pair : t.ev)
                        for (auto& e : pair) (void)hipEventDestroy(e);
                    t.have_events = false;
                    tk.pb = t.decided;
                } else {
                    t.window = 0;  // unusable timings: start over
                    t.calls = 0;
                }
            } else {
                (void)hipGetLastError();  // hipErrorNotReady is no error of this call
            }
        } else if (!capturing) {
            const double now = host_seconds();
            const bool other = t.n != N || t.d != D || t.k != K || t.stream != st;
            if (other || t.window_calls == 0 || (t.calls + t.window > 0 && now - t.last_call > t.gap))
                trial_restart(t, N, D, K, st);
            t.last_call = now;
            if (!t.have_events) {
                bool ok = true;
                for (auto& pair : t.ev)
                    for (auto& e : pair) ok = ok && hipEventCreate(&e) == hipSuccess;
                t.have_events = ok;
                if (!ok) (void)hipGetLastError();
            }
            if (t.have_events) {
                tk.pb = t.window == 1 ? 1 : 2;
                const int timed = t.window_calls / 3 > 2 ? t.window_calls / 3 : 2;
                if (t.calls == t.window_calls - timed) (void)hipEventRecord(t.ev[t.window][0], st);
                if (++t.calls == t.window_calls) {
                    tk.end = t.ev[t.window][1];
                    t.calls = 0;
                    ++t.window;
                }
            }
        }
    }
    pthread_mutex_unlock(&t.mu);
    return tk;
}

static void trial_end(const TrialTicket& tk, hipStream_t st) {
    if (tk.end) (void)hipEventRecord(tk.end, st);
}

template <int DP, int PB, bool VEC>
__global__ __launch_bounds__(fused_threads(PB, DP)) void lloyd_mfma_resident_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, int32_t* __restrict__ labels, float* __restrict__ min_d2, int64_t ntiles,
    double* __restrict__ fsum, int32_t* __restrict__ fcnt, int32_t* __restrict__ flags,
    int range_bits, int nrep) {
    extern __shared__ __align__(16) float lds[];
    constexpr int LDC = DP + 4;
    constexpr int LDA = DP + 1;  // odd row stride (in doubles): rows of different clusters spread over the banks
    constexpr int NJ = DP / 8;
    const int KP = (K + 31) & ~31;
    float* sC = lds;                                              // [KP][LDC]
    float* sCn = lds + KP * LDC;                                  // [KP] squared norms
    // With few clusters many lanes of an atomic instruction meet at one address and are served one after the
    // other, so the accumulators come in nrep copies (a power of two; a lane uses copy p mod nrep), an odd
    // number of doubles apart so that the copies of a row start in different banks.
    const size_t rstride = size_t(K) * LDA + 1;
    double* sA = reinterpret_cast<double*>(sCn + KP);             // [nrep][K][LDA] (+ 1 pad per copy)
    int* sN = reinterpret_cast<int*>(sA + nrep * rstride);        // [nrep][K] counts, then Emin, Emax, non-finite,
                                                                  // largest / smallest non-zero centroid norm
    int* sMeta = sN + nrep * K;
    const int tid = threadIdx.x, nthr = blockDim.x;

    for (int i = tid; i < KP * DP; i += nthr) {
        const int r = i / DP, c = i - r * DP;
        sC[r * LDC + c] = (r < K && c < D) ? -2.0f * C[int64_t(r) * ldc + c] : 0.f;
    }
    for (int r = tid; r < KP; r += nthr) {
        float s = HKM_INF;
        if (r < K) {
            s = 0.f;
            const float* c = C + int64_t(r) * ldc;
            for (int d = 0; d < D; ++d) s = fmaf(c[d], c[d], s);
        }
        sCn[r] = s;
    }
    for (int i = tid; i < int(nrep * rstride); i += nthr) sA[i] = 0.0;
    for (int i = tid; i < nrep * K; i += nthr) sN[i] = 0;
    if (tid == 0) {
        sMeta[0] = 0x7fffffff;
        sMeta[1] = -0x7fffffff;
        sMeta[2] = 0;
        sMeta[3] = 0;
        sMeta[4] = 0x7fffffff;
    }
    __syncthreads();
    // The squared centroid norms (bits of non-negative floats order like integers) give the rows' expected
    // magnitude, the same for every workgroup: a row at the largest centroid would get the exponent e_ref
    // below.  Rows up to 2^head times larger still fit the exact range; rows whose own exponent lies below
    // e_floor = e_ref + head - range_bits are rounded to the quantum of e_floor instead of their own, so that
    // a few rows near the origin -- the rule in two or three dimensions -- no longer cost the exact path.
    // The floor never rises more than 4 above the exponent of the SMALLEST non-zero centroid norm: the sums
    // of that cluster, too, keep 24 bits below its centroid's magnitude (centroids whose norms span more than
    // the exact range leave the rows of the large ones outside it, and the step falls back as before).
    for (int r = tid; r < K; r += nthr) {
        const int b = __float_as_int(sCn[r]) & 0x7fffffff;
        atomicMax(&sMeta[3], b);
        if (b != 0) atomicMin(&sMeta[4], b);
    }
    __syncthreads();
    int e_floor = -0x3fffffff;  // no usable centroid norm (all zero, inf, NaN): every row keeps its own quantum
    {
        const int cexp = (sMeta[3] >> 23) & 0xff, cexp_min = (sMeta[4] >> 23) & 0xff;
        if (cexp != 0 && cexp != 255) {
            const int e_ref = ((cexp - 127) >> 1) + 2, e_min = ((cexp_min - 127) >> 1) + 2;
            const int head = range_bits < 4 ? (range_bits < 0 ? 0 : range_bits) : 4;
            e_floor = min(e_ref + head - range_bits, e_min + 4);
        }
    }

    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), nw = nthr >> 6;
    const int p = lane & 31, h = lane >> 5;
    const int ncb = KP >> 5;
    const int64_t tile_rows = int64_t(nw) * PB * 32;
    const bool fast = VEC && D == DP && ldx < (int64_t(1) << 24);
    const unsigned lane_off = unsigned((int64_t(p) * ldx + h * (DP / 2)) * 4);
    double* sA_lane = sA + (p & (nrep - 1)) * rstride;
    int* sN_lane = sN + (p & (nrep - 1)) * K;
    // with two point blocks per wave (eight waves, 256 registers each) the first blocks' A fragments stay in
    // registers: a quarter of the centroid reads from LDS at K = 256
    constexpr int RB = PB == 2 ? HKM_RESIDENT_A_BLOCKS : 0;
    floatx4 ares[RB > 0 ? RB : 1][NJ];
    if constexpr (RB > 0) {
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                ares[r][j] = ld4(sC + ((r < ncb ? r : 0) * 32 + p) * LDC + h * (DP / 2) + 4 * j);
    }
    int emin = 0x7fffffff, emax = -0x7fffffff;
    int nonfinite = 0;  // a row whose |x|^2 is inf or NaN: its bound 2^E says nothing about its coordinates

    // One tile: the rows of the next one are requested (into the other of two register sets, which swap
    // roles from tile to tile) before this one is scanned.
    auto step = [&](int64_t tile, const floatx4 (&b)[PB][NJ], floatx4 (&bnext)[PB][NJ]) {
        const int64_t row0 = tile * tile_rows + wave * (PB * 32);
        float xnr[PB], m[PB];
        int mi[PB];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) s = fmaf(b[pb][j][t], b[pb][j][t], s);
            xnr[pb] = s + __shfl_xor(s, 32);
        }
        if (tile + gridDim.x < ntiles)
            fetch_rows<DP, PB, VEC>(X, N, D, ldx, row0 + int64_t(gridDim.x) * tile_rows, p, h, fast, lane_off, bnext);

        resident_scan<DP, PB, false, RB>(sC, sCn, ncb, p, h, b, xnr, m, mi, ares);
        bool neg = false;
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) neg |= m[pb] < 0.f;
        if (__any(neg)) resident_scan<DP, PB, true>(sC, sCn, ncb, p, h, b, xnr, m, mi);

#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            mi[pb] += 4 * h;
            merge_halves(m[pb], mi[pb]);
            const int64_t rb = row0 + pb * 32;  // wave-uniform: the stores take it as their scalar base
            const bool valid = rb + p < N;
            if (h == 0 && valid) {
                labels[rb + p] = mi[pb];
                if (min_d2) min_d2[rb + p] = m[pb];
                atomicAdd(&sN_lane[mi[pb]], 1);
            }
            if (valid && xnr[pb] != 0.f) {  // an all-zero row adds nothing
                // |x_d| < 2^E: |x|^2 < 2^(e2+1) up to rounding, one more bit of slack
                const int e2 = (__float_as_int(xnr[pb]) >> 23) - 127;
                nonfinite |= int((e2 & 0xff) == 128);  // exponent field 255 (the sign bit of |x|^2 is clear or NaN)
                const int E = max((e2 >> 1) + 2, e_floor);
                emin = min(emin, E);
                emax = max(emax, E);
                const double B = __hiloint2double(((1023 + 52 - FUSED_QBITS + E) << 20) | 0x80000, 0);
                double* row = sA_lane + size_t(mi[pb]) * LDA + h * (DP / 2);
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const double v = (double(b[pb][j][t]) + B) - B;
                        __hip_atomic_fetch_add(row + 4 * j + t, v, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
            }
        }
    };

    floatx4 b0[PB][NJ], b1[PB][NJ];
    if (int64_t(blockIdx.x) < ntiles)
        fetch_rows<DP, PB, VEC>(X, N, D, ldx, int64_t(blockIdx.x) * tile_rows + wave * (PB * 32), p, h, fast, lane_off,
                                b0);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += 2 * int64_t(gridDim.x)) {
        step(tile, b0, b1);
        if (tile + gridDim.x < ntiles) step(tile + gridDim.x, b1, b0);
    }

    atomicMin(&sMeta[0], emin);
    atomicMax(&sMeta[1], emax);
    if (nonfinite) atomicOr(&sMeta[2], 1);
    __syncthreads();
    double* gs = fsum + size_t(blockIdx.x) * K * D;
    for (int i = tid; i < K * D; i += nthr) {
        const int k = i / D, d = i - k * D;
        double v = 0.0;  // exact whatever the order (or the flag is up and the value unused)
        for (int r = 0; r < nrep; ++r) v += sA[r * rstride + size_t(k) * LDA + d];
        gs[i] = v;
    }
    for (int i = tid; i < K; i += nthr) {
        int c = 0;
        for (int r = 0; r < nrep; ++r) c += sN[r * K + i];
        fcnt[size_t(blockIdx.x) * K + i] = c;
    }
    if (tid == 0) {
        const int lo = sMeta[0], hi = sMeta[1];
        flags[blockIdx.x] = ((hi >= lo && hi - lo > range_bits) || sMeta[2]) ? 1 : 0;
    }
}

// ------------------------------------------------------------------------------------------------
// Tiled variant for 16 < D <= 64 when the centroids do not fit in LDS: same wave-level scheme as the
// resident kernel (a wave keeps its 32*PB points in B-operand registers for the whole feature range
// and scans centroid blocks), but the centroids pass through LDS in tiles of 128 rows, double
// buffered; all 256 threads fetch the next tile while the current one is scanned, one barrier per
// tile (every 4*(DP/2)*PB MFMAs per wave).  The running (min, argmin) is carried across tiles and the
// clamp at 0 is applied to the final minimum: where several centroids coincide with a point up to
// rounding (several negative values) the most negative one wins instead of the first -- a tie at the
// resolution of the formula.  Squared centroid norms come from global memory.
// ------------------------------------------------------------------------------------------------
template <int DP, int PB, bool VEC>
__global__ __launch_bounds__(256) void assign_mfma_tiled_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, const float* __restrict__ cn, int32_t* __restrict__ labels,
    float* __restrict__ min_d2, int64_t ntiles) {
    extern __shared__ __align__(16) float lds[];
    constexpr int LDC = DP + 4;
    constexpr int NJ = DP / 8;
    constexpr int TC = 128;                 // centroid rows per LDS tile
    constexpr int GPR = DP / 4;             // 16-byte groups per row
    constexpr int NQ = TC * GPR / 256;      // groups per thread and tile
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int p = lane & 31, h = lane >> 5;
    const int nct = (K + TC - 1) / TC;
    const int64_t my_tiles = (ntiles - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const int64_t nsteps = my_tiles * nct;

    floatx4 pc[NQ];
    float pcn = 0.f;  // squared norm of row `tid` of the tile (threads 0..127)
    auto issue = [&](int ct) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int g = tid + 256 * q;
            const int r = ct * TC + g / GPR, c = (g % GPR) * 4;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (r < K) v = load_row4<VEC>(C + int64_t(r) * ldc, c, D);
            pc[q] = v;
        }
        if (tid < TC) pcn = cn[ct * TC + tid];  // padded with +inf beyond K
    };

    int64_t tile = blockIdx.x;
    int ct = 0;
    if (nsteps > 0) issue(0);

    floatx4 b[PB][NJ];
    float xn[PB], m[PB];
    int blk[PB];
    floatx16 keep[PB];

    for (int64_t it = 0; it < nsteps; ++it) {
        float* sC = lds + (it & 1) * (TC * LDC + TC);
        float* sCn = sC + TC * LDC;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int g = tid + 256 * q;
            *reinterpret_cast<floatx4*>(sC + (g / GPR) * LDC + (g % GPR) * 4) = -2.0f * pc[q];
        }
        if (tid < TC) sCn[tid] = pcn;
        __syncthreads();

        const int64_t cur_tile = tile;
        const int cur_ct = ct;
        if (++ct == nct) {
            ct = 0;
            tile += gridDim.x;
        }
        if (it + 1 < nsteps) issue(ct);

        const int64_t row0 = cur_tile * (4 * PB * 32) + wave * (PB * 32);
        if (cur_ct == 0) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                int64_t r = row0 + pb * 32 + p;
                r = r < N ? r : N - 1;
                const float* xr = X + r * ldx;
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    b[pb][j] = load_row4<VEC>(xr, h * (DP / 2) + 4 * j, D);
#pragma unroll
                    for (int t = 0; t < 4; ++t) s = fmaf(b[pb][j][t], b[pb][j][t], s);
                }
                xn[pb] = s + __shfl_xor(s, 32);
                m[pb] = HKM_INF;
                blk[pb] = 0;
                keep_undefined(keep[pb]);
            }
        }

#pragma unroll 1
        for (int cb = 0; cb < TC / 32; ++cb) {
            floatx16 acc[PB];
            const floatx16 c0 = load_cn16(sCn + cb * 32 + 4 * h);
            resident_block<DP, PB>(sC + (cb * 32 + p) * LDC, c0, h, b, acc);
#pragma unroll
            for (int pb = 0; pb < PB; ++pb)
                block_min_keep(acc[pb], cur_ct * (TC / 32) + cb, m[pb], blk[pb], keep[pb]);
        }

        if (cur_ct == nct - 1) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                // the distance gets its |x|^2 and the clamp at 0 here, once per point
                float mm = fmaxf(m[pb] + xn[pb], 0.0f);
                int ii = kept_argmin(keep[pb], m[pb], blk[pb]) + 4 * h;
                merge_halves(mm, ii);
                const int64_t r = row0 + pb * 32 + p;
                if (h == 0 && r < N) {
                    labels[r] = ii;
                    if (min_d2) min_d2[r] = mm;
                }
            }
        }
    }
}

// The tiled kernel with the cross term from three-way split bf16 operands on the bf16 matrix cores
// (opt-in, arithmetic as in hkm_assign_split.hip).  The threads that stage a centroid tile split the
// fp32 values they fetched into three bf16 planes (one LDS buffer, two barriers per tile; two
// workgroups per CU overlap); a wave splits its points once per point tile and keeps the parts in
// registers.  DP is a multiple of 16 here (whole k-steps of the bf16 MFMA).
template <int DP, bool VEC>
__global__ __launch_bounds__(256) void assign_split_tiled_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, const float* __restrict__ cn, int32_t* __restrict__ labels,
    float* __restrict__ min_d2, int64_t ntiles) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int PB = 2;
    constexpr int LDB = DP + 8;             // row stride of a plane in bf16 elements
    constexpr int NJ = DP / 8;
    constexpr int NS = DP / 16;             // k-steps
    constexpr int TC = 128;                 // centroid rows per LDS tile
    constexpr int GPR = DP / 4;             // 16-byte groups of fp32 per row
    constexpr int NQ = TC * GPR / 256;      // groups per thread and tile
    constexpr int PLANE = TC * LDB;         // bf16 elements per plane
    __bf16* planes = reinterpret_cast<__bf16*>(lds_raw);                       // [3][TC][LDB]
    float* sCn = reinterpret_cast<float*>(lds_raw + size_t(3) * PLANE * 2);    // [TC]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int p = lane & 31, h = lane >> 5;
    const int nct = (K + TC - 1) / TC;
    const int64_t my_tiles = (ntiles - blockIdx.x + gridDim.x - 1) / gridDim.x;
    const int64_t nsteps = my_tiles * nct;

    floatx4 pc[NQ];
    float pcn = 0.f;
    auto issue = [&](int ct) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int g = tid + 256 * q;
            const int r = ct * TC + g / GPR, c = (g % GPR) * 4;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (r < K) v = load_row4<VEC>(C + int64_t(r) * ldc, c, D);
            pc[q] = v;
        }
        if (tid < TC) pcn = cn[ct * TC + tid];  // padded with +inf beyond K
    };

    int64_t tile = blockIdx.x;
    int ct = 0;
    if (nsteps > 0) issue(0);

    uintx4 xs[PB][3][NS];
    float xn[PB], m[PB];
    int mi[PB];

    for (int64_t it = 0; it < nsteps; ++it) {
        if (it > 0) __syncthreads();  // the previous tile's operands have been read
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int g = tid + 256 * q;
            unsigned a1[2], a2[2], a3[2];
#pragma unroll
            for (int e = 0; e < 2; ++e)
                split_pair(-2.0f * pc[q][2 * e], -2.0f * pc[q][2 * e + 1], a1[e], a2[e], a3[e]);
            const int o = (g / GPR) * LDB + (g % GPR) * 4;
            *reinterpret_cast<uint2*>(planes + o) = make_uint2(a1[0], a1[1]);
            *reinterpret_cast<uint2*>(planes + PLANE + o) = make_uint2(a2[0], a2[1]);
            *reinterpret_cast<uint2*>(planes + 2 * PLANE + o) = make_uint2(a3[0], a3[1]);
        }
        if (tid < TC) sCn[tid] = pcn;
        __syncthreads();

        const int64_t cur_tile = tile;
        const int cur_ct = ct;
        if (++ct == nct) {
            ct = 0;
            tile += gridDim.x;
        }
        if (it + 1 < nsteps) issue(ct);

        const int64_t row0 = cur_tile * (4 * PB * 32) + wave * (PB * 32);
        if (cur_ct == 0) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                int64_t r = row0 + pb * 32 + p;
                r = r < N ? r : N - 1;
                const float* xr = X + r * ldx;
                float s = 0.f;
                floatx4 b[NJ];
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    b[j] = load_row4<VEC>(xr, h * (DP / 2) + 4 * j, D);
#pragma unroll
                    for (int t = 0; t < 4; ++t) s = fmaf(b[j][t], b[j][t], s);
                }
                xn[pb] = s + __shfl_xor(s, 32);
#pragma unroll
                for (int st = 0; st < NS; ++st)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const floatx4 g = b[2 * st + (q >> 1)];
                        unsigned p1, p2, p3;
                        split_pair(g[2 * (q & 1)], g[2 * (q & 1) + 1], p1, p2, p3);
                        xs[pb][0][st][q] = p1;
                        xs[pb][1][st][q] = p2;
                        xs[pb][2][st][q] = p3;
                    }
                m[pb] = HKM_INF;
                mi[pb] = 0;
            }
        }

        constexpr int XP[6] = {2, 0, 1, 1, 0, 0};
        constexpr int CP[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll 1
        for (int cb = 0; cb < TC / 32; ++cb) {
            const floatx16 c0 = load_cn16(sCn + cb * 32 + 4 * h);
            uintx4 cs[3][NS];
#pragma unroll
            for (int part = 0; part < 3; ++part)
#pragma unroll
                for (int st = 0; st < NS; ++st)
                    cs[part][st] = *reinterpret_cast<const uintx4*>(planes + part * PLANE + (cb * 32 + p) * LDB +
                                                                   h * (DP / 2) + 8 * st);
            floatx16 acc[PB];
#pragma unroll
            for (int t = 0; t < 6; ++t)
#pragma unroll
                for (int st = 0; st < NS; ++st)
#pragma unroll
                    for (int pb = 0; pb < PB; ++pb)
                        acc[pb] = (t == 0 && st == 0)
                                      ? MFMA_BF16(as_bf16x8(cs[CP[t]][st]), as_bf16x8(xs[pb][XP[t]][st]), c0)
                                      : MFMA_BF16(as_bf16x8(cs[CP[t]][st]), as_bf16x8(xs[pb][XP[t]][st]), acc[pb]);
            const int kb = cur_ct * TC + cb * 32;
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) block_argmin(acc[pb], kb, m[pb], mi[pb]);
        }

        if (cur_ct == nct - 1) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                float mm = fmaxf(m[pb] + xn[pb], 0.0f);
                int ii = mi[pb] + 4 * h;
                merge_halves(mm, ii);
                const int64_t r = row0 + pb * 32 + p;
                if (h == 0 && r < N) {
                    labels[r] = ii;
                    if (min_d2) min_d2[r] = mm;
                }
            }
        }
    }
}

template <int DP, bool VEC>
static int launch_split_tiled_t(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                                int32_t K, int64_t ldc, const float* cn, int32_t* labels, float* min_d2,
                                hipStream_t st) {
    constexpr int PB = 2;
    const int64_t ntiles = (N + 4 * PB * 32 - 1) / (4 * PB * 32);
    const size_t lds = size_t(3) * 128 * (DP + 8) * 2 + 128 * sizeof(float);
    auto kern = assign_split_tiled_kernel<DP, VEC>;
    int64_t grid = int64_t(num_cus()) * 2;
    if (grid > ntiles) grid = ntiles;
    prof_begin(st);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, st, X, N, D, ldx, C, K, ldc, cn, labels,
                       min_d2, ntiles);
    prof_end(st);
    return check_launch("assign_split_tiled_kernel");
}

template <int DP, bool VEC>
static int launch_tiled_t(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                          int32_t K, int64_t ldc, const float* cn, int32_t* labels, float* min_d2,
                          hipStream_t st) {
    constexpr int PB = 2;
    const int64_t ntiles = (N + 4 * PB * 32 - 1) / (4 * PB * 32);
    const size_t lds = size_t(2) * 128 * (DP + 5) * sizeof(float);
    auto kern = assign_mfma_tiled_kernel<DP, PB, VEC>;
    int64_t grid = int64_t(num_cus()) * 2;
    if (grid > ntiles) grid = ntiles;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return fail(HKM_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    prof_begin(st);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, st, X, N, D, ldx, C, K, ldc, cn,
                       labels, min_d2, ntiles);
    prof_end(st);
    return check_launch("assign_mfma_tiled_kernel");
}

int launch_assign_mfma_tiled(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                             int32_t K, int64_t ldc, const float* cn, int32_t* labels,
                             float* min_d2, bool split, hipStream_t st) {
    const bool vec = aligned16(X) && aligned16(C) && (ldx % 4 == 0) && (ldc % 4 == 0) && (D % 4 == 0);
    if (split) {
        const int sdp = D <= 32 ? 32 : D <= 48 ? 48 : 64;  // whole k-steps of 16
#define HKM_SCASE(d)                                                                                    \
    case d:                                                                                             \
        return vec ? launch_split_tiled_t<d, true>(X, N, D, ldx, C, K, ldc, cn, labels, min_d2, st)     \
                   : launch_split_tiled_t<d, false>(X, N, D, ldx, C, K, ldc, cn, labels, min_d2, st);
        switch (sdp) { HKM_SCASE(32) HKM_SCASE(48) HKM_SCASE(64) }
#undef HKM_SCASE
    }
    const int dp = resident_dp(D);
#define HKM_CASE(d)                                                                              \
    case d:                                                                                      \
        return vec ? launch_tiled_t<d, true>(X, N, D, ldx, C, K, ldc, cn, labels, min_d2, st)    \
                   : launch_tiled_t<d, false>(X, N, D, ldx, C, K, ldc, cn, labels, min_d2, st);
    switch (dp) {
        HKM_CASE(8) HKM_CASE(16) HKM_CASE(24) HKM_CASE(32) HKM_CASE(48) HKM_CASE(64)
        default:
            return fail(HKM_EUNSUPPORTED, "assign_mfma_tiled: D=%d", D);
    }
#undef HKM_CASE
}

template <int DP, int PB, bool VEC>
static int launch_resident_t(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                             int32_t K, int64_t ldc, int32_t* labels, float* min_d2,
                             hipStream_t st) {
    const int64_t ntiles = (N + 4 * PB * 32 - 1) / (4 * PB * 32);
    const size_t lds = resident_lds_bytes(D, K);
    auto kern = assign_mfma_resident_kernel<DP, PB, VEC>;
    // persistent grid: as many workgroups as are resident at once (registers and the centroids' LDS
    // footprint decide: two per CU with two point blocks per wave, up to four with one)
    int per_cu = 0;
    hipError_t oe = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), 256, lds);
    if (oe != hipSuccess) return fail(HKM_EHIP, "hipOccupancyMaxActiveBlocksPerMultiprocessor: %s", hipGetErrorString(oe));
    per_cu = per_cu < 1 ? 1 : per_cu > 4 ? 4 : per_cu;
    int64_t grid = int64_t(num_cus()) * per_cu;
    if (grid > ntiles) grid = ntiles;
    prof_begin(st);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, st, X, N, D, ldx, C, K, ldc,
                       labels, min_d2, ntiles);
    prof_end(st);
    return check_launch("assign_mfma_resident_kernel");
}

static size_t fused_lds_bytes_with(int32_t D, int32_t K, int nrep) {
    const size_t kp = (size_t(K) + 31) / 32 * 32;
    const int dp = resident_dp(D);
    return kp * (dp + 5) * sizeof(float) + size_t(nrep) * (size_t(K) * (dp + 1) + 1) * sizeof(double) +
           (size_t(nrep) * K + 8) * sizeof(int);
}

// Copies of the fp64 accumulators in the one-sweep kernel: up to 64 clusters, as many as bring the lanes
// that meet at one address down to a few.  One workgroup per CU runs this kernel, so the copies may take most of
// the LDS: with the 48 KB they were held to before, 10M x 64, K = 8 ran on 8 copies in 0.652 ms (16: 0.605 ms),
// 10M x 32, K = 32 on 4 in 0.360 ms (16: 0.345 ms); more than 16 copies gain nothing (10M x 32, K = 8: 0.3215 /
// 0.3194 / 0.3166 ms with 16 / 32 / 64).  The sums are exact, so the number of copies does not change a bit.
int fused_replicas(int32_t D, int32_t K) {
    int r = K <= 32 ? 16 : K <= 64 ? 4 : 1;
    const size_t cap = 128 * 1024;
    while (r > 1 && fused_lds_bytes_with(D, K, r) > cap) r >>= 1;
    return r;
}

size_t fused_lds_bytes(int32_t D, int32_t K) { return fused_lds_bytes_with(D, K, fused_replicas(D, K)); }

int fused_grid(int64_t N, int32_t D) {
    const int dp = resident_dp(D);
    const int pb = dp > 32 ? 1 : 2;  // up to 32 features both geometries cut the rows into the same tiles
    const int64_t tile_rows = int64_t(fused_threads(pb, dp) / 64) * pb * 32;
    const int64_t ntiles = (N + tile_rows - 1) / tile_rows;
    int64_t grid = num_cus();
    if (grid > FUSED_MAX_GRID) grid = FUSED_MAX_GRID;
    if (grid > ntiles) grid = ntiles;
    return int(grid < 1 ? 1 : grid);
}

template <int DP, int PB, bool VEC>
static int launch_fused_t(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C, int32_t K,
                          int64_t ldc, int32_t* labels, float* min_d2, double* fsum, int32_t* fcnt,
                          int32_t* flags, hipStream_t st) {
    constexpr int THREADS = fused_threads(PB, DP);
    const int64_t tile_rows = int64_t(THREADS / 64) * PB * 32;
    const int64_t ntiles = (N + tile_rows - 1) / tile_rows;
    const int grid = fused_grid(N, D);
    const size_t lds = fused_lds_bytes(D, K);
    auto kern = lloyd_mfma_resident_kernel<DP, PB, VEC>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return fail(HKM_EHIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    // rows one workgroup adds up, as a power of two
    const int64_t per_wg = (ntiles + grid - 1) / grid * tile_rows;
    int lg = 0;
    while ((int64_t(1) << lg) < per_wg) ++lg;
    const int range_bits = 53 - FUSED_QBITS - lg;
    prof_begin(st);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(THREADS), lds, st, X, N, D, ldx, C, K, ldc,
                       labels, min_d2, ntiles, fsum, fcnt, flags, range_bits, fused_replicas(D, K));
    prof_end(st);
    return check_launch("lloyd_mfma_resident_kernel");
}

int launch_lloyd_mfma_resident(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                               int32_t K, int64_t ldc, int32_t* labels, float* min_d2, double* fsum,
                               int32_t* fcnt, int32_t* flags, hipStream_t st) {
    const bool vec = aligned16(X) && (ldx % 4 == 0) && (D % 4 == 0);
    const int dp = resident_dp(D);
    const TrialTicket tk = trial_begin(N, D, K, st);
    const int pb = tk.pb;
    int rc = HKM_EUNSUPPORTED;
    bool found = false;
#define HKM_CASE(d, b)                                                                                           \
    if (!found && dp == d && pb == b) {                                                                          \
        found = true;                                                                                            \
        rc = vec ? launch_fused_t<d, b, true>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, st)    \
                 : launch_fused_t<d, b, false>(X, N, D, ldx, C, K, ldc, labels, min_d2, fsum, fcnt, flags, st);  \
    }
    HKM_CASE(8, 2) HKM_CASE(8, 1) HKM_CASE(16, 2) HKM_CASE(16, 1) HKM_CASE(24, 2) HKM_CASE(24, 1) HKM_CASE(32, 2)
    HKM_CASE(32, 1) HKM_CASE(48, 1) HKM_CASE(64, 1) HKM_CASE(96, 1) HKM_CASE(128, 1)
#undef HKM_CASE
    trial_end(tk, st);
    if (!found) return fail(HKM_EUNSUPPORTED, "lloyd_mfma_resident: D=%d", D);
    return rc;
}

int launch_assign_mfma_resident(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                                int32_t K, int64_t ldc, int32_t* labels, float* min_d2,
                                hipStream_t st) {
    const bool vec = aligned16(X) && (ldx % 4 == 0) && (D % 4 == 0);
    const int dp = resident_dp(D);
    const int pb = resident_point_blocks(dp);
#define HKM_CASE(d, b)                                                                         \
    if (dp == d && pb == b)                                                                    \
        return vec ? launch_resident_t<d, b, true>(X, N, D, ldx, C, K, ldc, labels, min_d2, st) \
                   : launch_resident_t<d, b, false>(X, N, D, ldx, C, K, ldc, labels, min_d2, st);
    HKM_CASE(8, 2) HKM_CASE(8, 1) HKM_CASE(16, 2) HKM_CASE(16, 1) HKM_CASE(24, 2) HKM_CASE(24, 1) HKM_CASE(32, 2)
    HKM_CASE(32, 1) HKM_CASE(48, 1) HKM_CASE(64, 1) HKM_CASE(96, 1) HKM_CASE(128, 1)
#undef HKM_CASE
    return fail(HKM_EUNSUPPORTED, "assign_mfma_resident: D=%d", D);
}

// ------------------------------------------------------------------------------------------------
// Streaming variant for any K and D, 2-D decomposition.  A work item is (tile of 128 points) x (tile
// of 128 centroids) over all features in chunks of 32; the four waves of a workgroup form a 2 x 2 grid,
// each computing 64 points x 64 centroids per chunk (2 x 2 MFMA blocks, 64 MFMAs).  Both operand
// panels of a chunk (128 x 32 floats each) are fetched with fully coalesced 16-byte loads by all 256
// threads one chunk ahead and staged through double-buffered LDS (row stride 36 floats keeps the
// 16-byte operand reads conflict-free).  After the last chunk one more MFMA adds
// (-|c|^2/2) * 1 + 1 * (-|x|^2/2), so the accumulator is minus half the squared distance (squared
// centroid norms come from global memory, padded with +inf; |x|^2 is accumulated by the staging
// threads from the registers they stage and combined once per tile).
//
// Work items are laid out so that the workgroups of one XCD (workgroup b runs on XCD b % 8) work on
// the SAME few point tiles at the same time, one centroid tile each: a point tile is then read from
// HBM once and served to the other workgroups from that XCD's L2, instead of once per centroid tile.
// The per-item (min, argmin) of a point are merged across centroid tiles with a 64-bit unsigned
// atomic min on the key (bits of the clamped d2) << 32 | index: for non-negative floats the bit
// pattern orders like the value, so the smallest distance wins and, among equal distances, the
// smallest index -- an order-independent, hence deterministic, merge.
// ------------------------------------------------------------------------------------------------
struct StreamPlan {
    int nct, ndc, W, PG;  // centroid tiles, feature chunks, workgroups per XCD, point tiles in flight per XCD
    int grid;
};
static StreamPlan stream_plan(int64_t N, int32_t D, int32_t K) {
    StreamPlan pl;
    pl.nct = (K + 127) / 128;
    pl.ndc = (D + 31) / 32;
    const int w_max = num_cus() * 2 / 8;  // two workgroups per CU
    if (pl.nct <= w_max) {
        pl.PG = w_max / pl.nct;
        const int64_t per_xcd = ((N + 127) / 128 + 7) / 8;  // point tiles per XCD
        if (pl.PG > per_xcd) pl.PG = int(per_xcd < 1 ? 1 : per_xcd);
        pl.W = pl.PG * pl.nct;
    } else {
        pl.PG = 1;
        pl.W = w_max;
    }
    pl.grid = pl.W * 8;
    return pl;
}

__global__ void fill_keys_kernel(unsigned long long* __restrict__ keys, int64_t n) {
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += int64_t(gridDim.x) * blockDim.x)
        keys[i] = ~0ull;
}

__global__ void unpack_keys_kernel(const unsigned long long* __restrict__ keys, int64_t n,
                                   int32_t* __restrict__ labels, float* __restrict__ min_d2) {
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += int64_t(gridDim.x) * blockDim.x) {
        const unsigned long long k = keys[i];
        const unsigned hi = unsigned(k >> 32);
        // a row whose distances were all NaN never lowered its key: label 0 like the reference's
        // torch.min on an all-NaN row
        labels[i] = hi == 0xffffffffu ? 0 : int32_t(unsigned(k));
        if (min_d2) min_d2[i] = __uint_as_float(hi);
    }
}

template <bool VEC>
__global__ __launch_bounds__(256) void assign_mfma_stream_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, const float* __restrict__ cn, unsigned long long* __restrict__ keys, int64_t ntiles,
    int nct, int ndc, int W, int PG) {
    constexpr int PB = 2, CB = 2, TP = 128, TC = 128, DC = 32, LDS_LD = DC + 4;
    __shared__ __align__(16) float sA[2][TC * LDS_LD];
    __shared__ __align__(16) float sB[2][TP * LDS_LD];
    __shared__ float sM[2][TP];
    __shared__ int sI[2][TP];
    __shared__ float sXn[TP];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wp = wave & 1, wc = wave >> 1;  // this wave: points [64 wp, +64), centroids [64 wc, +64)
    const int p = lane & 31, h = lane >> 5;

    // items of this workgroup: item q = (point tile xt0 + 8 PG (q / cpw), centroid tile ct0 + W (q % cpw))
    const int xcd = blockIdx.x & 7, l = blockIdx.x >> 3;
    const bool spread = nct <= W;  // one centroid tile per workgroup, PG point tiles in flight
    const int ct0 = spread ? l % nct : l;
    const int64_t xt0 = xcd + 8 * int64_t(spread ? l / nct : 0);
    const int cpw = spread ? 1 : (nct - l + W - 1) / W;
    const int64_t xstep = 8 * int64_t(PG);
    const int64_t nx = xt0 < ntiles ? (ntiles - xt0 + xstep - 1) / xstep : 0;
    const int64_t nsteps = nx * cpw * ndc;

    const int sr = tid >> 3;         // staging: rows sr + 32 q (q = 0..3) of both panels
    const int sc = (tid & 7) * 4;    // column group

    // Addresses of a chunk's loads are (workgroup-uniform panel base, advanced by scalar arithmetic)
    // + (a per-thread byte offset that only changes with the tile): no vector instruction per chunk.
    // Rows beyond K or N are clamped to the last valid row (a padding centroid has |c|^2 = +inf and
    // never wins; a padding point is never stored).
    const float* baseA = C;
    const float* baseB = X;
    unsigned offA[4], offB[4];
    auto set_tile = [&](int64_t xt, int ct) {
        baseA = C + int64_t(ct) * TC * ldc;
        baseB = X + xt * TP * ldx;
        const int lastA = K - 1 - ct * TC;
        const int64_t lastB = N - 1 - xt * TP;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int r = sr + 32 * q;
            const int ra = r < lastA ? r : lastA;
            const int rb = r < lastB ? r : int(lastB);
            offA[q] = unsigned((int64_t(ra) * ldc + sc) * 4);
            offB[q] = unsigned((int64_t(rb) * ldx + sc) * 4);
        }
    };
    floatx4 pa[4], pb_[4];
    auto issue = [&](int dc) {
        const float* a = baseA + dc * DC;
        const float* bq = baseB + dc * DC;
        if (VEC && dc * DC + DC <= D) {  // whole chunk inside the rows: unconditional 16-byte loads
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                pa[q] = *reinterpret_cast<const floatx4*>(reinterpret_cast<const char*>(a) + offA[q]);
                pb_[q] = *reinterpret_cast<const floatx4*>(reinterpret_cast<const char*>(bq) + offB[q]);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // offsets hold the column group; load_row4 wants the row start and the column
                pa[q] = load_row4<VEC>(reinterpret_cast<const float*>(reinterpret_cast<const char*>(a) + offA[q]) - sc - dc * DC,
                                       dc * DC + sc, D);
                pb_[q] = load_row4<VEC>(reinterpret_cast<const float*>(reinterpret_cast<const char*>(bq) + offB[q]) - sc - dc * DC,
                                        dc * DC + sc, D);
            }
        }
    };

    int64_t xi = 0;  // index of the point tile within this workgroup's sequence
    int ci = 0, dc = 0;
    if (nsteps > 0) {
        set_tile(xt0, ct0);
        issue(0);
    }

    floatx16 acc[PB][CB];
    float xsq[4] = {0.f, 0.f, 0.f, 0.f};  // |x|^2 of staging rows sr + 32 q over this thread's column group

    for (int64_t it = 0; it < nsteps; ++it) {
        const int buf = int(it & 1);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            *reinterpret_cast<floatx4*>(&sA[buf][(sr + 32 * q) * LDS_LD + sc]) = pa[q];
            *reinterpret_cast<floatx4*>(&sB[buf][(sr + 32 * q) * LDS_LD + sc]) = pb_[q];
#pragma unroll
            for (int t = 0; t < 4; ++t) xsq[q] = fmaf(pb_[q][t], pb_[q][t], xsq[q]);
        }
        __syncthreads();

        const int64_t cur_xt = xt0 + xi * xstep;
        const int cur_ct = ct0 + ci * W, cur_dc = dc;
        if (++dc == ndc) {
            dc = 0;
            if (++ci == cpw) {
                ci = 0;
                ++xi;
            }
            if (it + 1 < nsteps) set_tile(xt0 + xi * xstep, ct0 + ci * W);
        }
        if (it + 1 < nsteps) issue(dc);

        if (cur_dc == 0) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[pb][cb][v] = 0.f;
            }
        }

        // this lane-half's 16 features of the chunk, for both operands
        floatx4 b[PB][4];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) {
            const float* brow = &sB[buf][(wp * 64 + pb * 32 + p) * LDS_LD + h * 16];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[pb][j] = ld4(brow + 4 * j);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const float* arow = &sA[buf][(wc * 64 + cb * 32 + p) * LDS_LD + h * 16];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const floatx4 a = ld4(arow + 4 * j);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int pb = 0; pb < PB; ++pb)
                        acc[pb][cb] = MFMA32(a[t], b[pb][j][t], acc[pb][cb]);
            }
        }

        if (cur_dc == ndc - 1) {
            // squared norms of the tile's points: the eight threads that staged a row add their parts
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v = xsq[q];
                v += __shfl_xor(v, 1);
                v += __shfl_xor(v, 2);
                v += __shfl_xor(v, 4);
                if ((tid & 7) == 0) sXn[sr + 32 * q] = v;
                xsq[q] = 0.f;
            }
            __syncthreads();
            float m[PB];
            int mi[PB];
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                const float xn = sXn[wp * 64 + pb * 32 + p];
                const float baug = h ? -0.5f * xn : 1.0f;
                m[pb] = -HKM_INF;
                mi[pb] = 0;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const int kb = cur_ct * TC + wc * 64 + cb * 32;
                    const float aaug = h ? 1.0f : -0.5f * cn[kb + p];
                    // g = x.c - |c|^2/2 - |x|^2/2 = -d2/2 (halving is exact): the nearest centroid has
                    // the LARGEST g; the clamp of d2 at 0 is a clamp of g at 0 from above
                    const floatx16 g16 = MFMA32(aaug, baug, acc[pb][cb]);
                    float bm = fminf(g16[0], 0.0f);
                    int bi = 0;
#pragma unroll
                    for (int v = 1; v < 16; ++v) {
                        const float g = fminf(g16[v], 0.0f);
                        const bool gt = g > bm;
                        bi = gt ? 8 * (v >> 2) + (v & 3) : bi;
                        bm = gt ? g : bm;
                    }
                    const bool gt = bm > m[pb];
                    mi[pb] = gt ? kb + bi : mi[pb];
                    m[pb] = gt ? bm : m[pb];
                }
                // merge lane halves, then the two waves that cover the same points
                mi[pb] += 4 * h;
                // back to the squared distance (+inf if every g was NaN or -inf); the "+ 0" turns a
                // -0.0 into +0.0, whose bit pattern is the smallest key
                m[pb] = -2.0f * m[pb] + 0.0f;
                merge_halves(m[pb], mi[pb]);
                if (h == 0) {
                    sM[wc][wp * 64 + pb * 32 + p] = m[pb];
                    sI[wc][wp * 64 + pb * 32 + p] = mi[pb];
                }
            }
            __syncthreads();
            if (tid < TP) {
                float m0 = sM[0][tid];
                int i0 = sI[0][tid];
                const float m1 = sM[1][tid];
                const int i1 = sI[1][tid];
                if (m1 < m0 || (m1 == m0 && i1 < i0)) {
                    m0 = m1;
                    i0 = i1;
                }
                const int64_t r = cur_xt * TP + tid;
                if (r < N && m0 < HKM_INF) {
                    const unsigned long long key =
                        (static_cast<unsigned long long>(__float_as_uint(m0)) << 32) | unsigned(i0);
                    atomicMin(keys + r, key);
                }
            }
        }
    }
}

// The same kernel with the cross term evaluated from three-way split bf16 operands on the bf16 matrix
// cores (opt-in, see hkm_assign_split.hip for the arithmetic): the staging threads split the fp32
// values they fetched and store three bf16 planes per panel.
template <bool VEC>
__global__ __launch_bounds__(256) void assign_split_stream_kernel(
    const float* __restrict__ X, int64_t N, int D, int64_t ldx, const float* __restrict__ C, int K,
    int64_t ldc, const float* __restrict__ cn, unsigned long long* __restrict__ keys, int64_t ntiles,
    int nct, int ndc, int W, int PG) {
    constexpr int PB = 2, CB = 2, TP = 128, TC = 128, DC = 32, LDB = DC + 8;
    // three bf16 planes per panel, one buffer (two barriers per chunk; two workgroups per CU overlap)
    __shared__ __align__(16) __bf16 sA[3][TC * LDB];
    __shared__ __align__(16) __bf16 sB[3][TP * LDB];
    __shared__ float sM[2][TP];
    __shared__ int sI[2][TP];
    __shared__ float sXn[TP];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wp = wave & 1, wc = wave >> 1;  // this wave: points [64 wp, +64), centroids [64 wc, +64)
    const int p = lane & 31, h = lane >> 5;

    // items of this workgroup: item q = (point tile xt0 + 8 PG (q / cpw), centroid tile ct0 + W (q % cpw))
    const int xcd = blockIdx.x & 7, l = blockIdx.x >> 3;
    const bool spread = nct <= W;  // one centroid tile per workgroup, PG point tiles in flight
    const int ct0 = spread ? l % nct : l;
    const int64_t xt0 = xcd + 8 * int64_t(spread ? l / nct : 0);
    const int cpw = spread ? 1 : (nct - l + W - 1) / W;
    const int64_t xstep = 8 * int64_t(PG);
    const int64_t nx = xt0 < ntiles ? (ntiles - xt0 + xstep - 1) / xstep : 0;
    const int64_t nsteps = nx * cpw * ndc;

    const int sr = tid >> 3;         // staging: rows sr + 32 q (q = 0..3) of both panels
    const int sc = (tid & 7) * 4;    // column group

    // Addresses of a chunk's loads are (workgroup-uniform panel base, advanced by scalar arithmetic)
    // + (a per-thread byte offset that only changes with the tile): no vector instruction per chunk.
    // Rows beyond K or N are clamped to the last valid row (a padding centroid has |c|^2 = +inf and
    // never wins; a padding point is never stored).
    const float* baseA = C;
    const float* baseB = X;
    unsigned offA[4], offB[4];
    auto set_tile = [&](int64_t xt, int ct) {
        baseA = C + int64_t(ct) * TC * ldc;
        baseB = X + xt * TP * ldx;
        const int lastA = K - 1 - ct * TC;
        const int64_t lastB = N - 1 - xt * TP;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int r = sr + 32 * q;
            const int ra = r < lastA ? r : lastA;
            const int rb = r < lastB ? r : int(lastB);
            offA[q] = unsigned((int64_t(ra) * ldc + sc) * 4);
            offB[q] = unsigned((int64_t(rb) * ldx + sc) * 4);
        }
    };
    floatx4 pa[4], pb_[4];
    auto issue = [&](int dc) {
        const float* a = baseA + dc * DC;
        const float* bq = baseB + dc * DC;
        if (VEC && dc * DC + DC <= D) {  // whole chunk inside the rows: unconditional 16-byte loads
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                pa[q] = *reinterpret_cast<const floatx4*>(reinterpret_cast<const char*>(a) + offA[q]);
                pb_[q] = *reinterpret_cast<const floatx4*>(reinterpret_cast<const char*>(bq) + offB[q]);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // offsets hold the column group; load_row4 wants the row start and the column
                pa[q] = load_row4<VEC>(reinterpret_cast<const float*>(reinterpret_cast<const char*>(a) + offA[q]) - sc - dc * DC,
                                       dc * DC + sc, D);
                pb_[q] = load_row4<VEC>(reinterpret_cast<const float*>(reinterpret_cast<const char*>(bq) + offB[q]) - sc - dc * DC,
                                        dc * DC + sc, D);
            }
        }
    };

    int64_t xi = 0;  // index of the point tile within this workgroup's sequence
    int ci = 0, dc = 0;
    if (nsteps > 0) {
        set_tile(xt0, ct0);
        issue(0);
    }

    floatx16 acc[PB][CB];
    float xsq[4] = {0.f, 0.f, 0.f, 0.f};  // |x|^2 of staging rows sr + 32 q over this thread's column group

    for (int64_t it = 0; it < nsteps; ++it) {
        if (it > 0) __syncthreads();  // the previous chunk's operands have been read
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            unsigned a1[2], a2[2], a3[2], b1[2], b2[2], b3[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                split_pair(pa[q][2 * e], pa[q][2 * e + 1], a1[e], a2[e], a3[e]);
                split_pair(pb_[q][2 * e], pb_[q][2 * e + 1], b1[e], b2[e], b3[e]);
            }
            const int o = (sr + 32 * q) * LDB + sc;
            *reinterpret_cast<uint2*>(&sA[0][o]) = make_uint2(a1[0], a1[1]);
            *reinterpret_cast<uint2*>(&sA[1][o]) = make_uint2(a2[0], a2[1]);
            *reinterpret_cast<uint2*>(&sA[2][o]) = make_uint2(a3[0], a3[1]);
            *reinterpret_cast<uint2*>(&sB[0][o]) = make_uint2(b1[0], b1[1]);
            *reinterpret_cast<uint2*>(&sB[1][o]) = make_uint2(b2[0], b2[1]);
            *reinterpret_cast<uint2*>(&sB[2][o]) = make_uint2(b3[0], b3[1]);
#pragma unroll
            for (int t = 0; t < 4; ++t) xsq[q] = fmaf(pb_[q][t], pb_[q][t], xsq[q]);
        }
        __syncthreads();

        const int64_t cur_xt = xt0 + xi * xstep;
        const int cur_ct = ct0 + ci * W, cur_dc = dc;
        if (++dc == ndc) {
            dc = 0;
            if (++ci == cpw) {
                ci = 0;
                ++xi;
            }
            if (it + 1 < nsteps) set_tile(xt0 + xi * xstep, ct0 + ci * W);
        }
        if (it + 1 < nsteps) issue(dc);

        if (cur_dc == 0) {
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[pb][cb][v] = 0.f;
            }
        }

        // k-step s of the bf16 MFMA covers features 16 s .. 16 s + 15 of the chunk, 8 per lane-half;
        // the six partial products per (centroid block, point block), smallest first
        uintx4 xb[PB][3][2];
#pragma unroll
        for (int pb = 0; pb < PB; ++pb)
#pragma unroll
            for (int part = 0; part < 3; ++part)
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2)
                    xb[pb][part][s2] = *reinterpret_cast<const uintx4*>(
                        &sB[part][(wp * 64 + pb * 32 + p) * LDB + 16 * s2 + 8 * h]);
        constexpr int XP[6] = {2, 0, 1, 1, 0, 0};
        constexpr int CP[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            uintx4 ca[3][2];
#pragma unroll
            for (int part = 0; part < 3; ++part)
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2)
                    ca[part][s2] = *reinterpret_cast<const uintx4*>(
                        &sA[part][(wc * 64 + cb * 32 + p) * LDB + 16 * s2 + 8 * h]);
#pragma unroll
            for (int t = 0; t < 6; ++t)
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                    for (int pb = 0; pb < PB; ++pb)
                        acc[pb][cb] = MFMA_BF16(as_bf16x8(ca[CP[t]][s2]), as_bf16x8(xb[pb][XP[t]][s2]), acc[pb][cb]);
        }

        if (cur_dc == ndc - 1) {
            // squared norms of the tile's points: the eight threads that staged a row add their parts
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v = xsq[q];
                v += __shfl_xor(v, 1);
                v += __shfl_xor(v, 2);
                v += __shfl_xor(v, 4);
                if ((tid & 7) == 0) sXn[sr + 32 * q] = v;
                xsq[q] = 0.f;
            }
            __syncthreads();
            float m[PB];
            int mi[PB];
#pragma unroll
            for (int pb = 0; pb < PB; ++pb) {
                const float xn = sXn[wp * 64 + pb * 32 + p];
                const float baug = h ? -0.5f * xn : 1.0f;
                m[pb] = -HKM_INF;
                mi[pb] = 0;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const int kb = cur_ct * TC + wc * 64 + cb * 32;
                    const float aaug = h ? 1.0f : -0.5f * cn[kb + p];
                    // g = x.c - |c|^2/2 - |x|^2/2 = -d2/2 (halving is exact): the nearest centroid has
                    // the LARGEST g; the clamp of d2 at 0 is a clamp of g at 0 from above
                    const floatx16 g16 = MFMA32(aaug, baug, acc[pb][cb]);
                    float bm = fminf(g16[0], 0.0f);
                    int bi = 0;
#pragma unroll
                    for (int v = 1; v < 16; ++v) {
                        const float g = fminf(g16[v], 0.0f);
                        const bool gt = g > bm;
                        bi = gt ? 8 * (v >> 2) + (v & 3) : bi;
                        bm = gt ? g : bm;
                    }
                    const bool gt = bm > m[pb];
                    mi[pb] = gt ? kb + bi : mi[pb];
                    m[pb] = gt ? bm : m[pb];
                }
                // merge lane halves, then the two waves that cover the same points
                mi[pb] += 4 * h;
                // back to the squared distance (+inf if every g was NaN or -inf); the "+ 0" turns a
                // -0.0 into +0.0, whose bit pattern is the smallest key
                m[pb] = -2.0f * m[pb] + 0.0f;
                merge_halves(m[pb], mi[pb]);
                if (h == 0) {
                    sM[wc][wp * 64 + pb * 32 + p] = m[pb];
                    sI[wc][wp * 64 + pb * 32 + p] = mi[pb];
                }
            }
            __syncthreads();
            if (tid < TP) {
                float m0 = sM[0][tid];
                int i0 = sI[0][tid];
                const float m1 = sM[1][tid];
                const int i1 = sI[1][tid];
                if (m1 < m0 || (m1 == m0 && i1 < i0)) {
                    m0 = m1;
                    i0 = i1;
                }
                const int64_t r = cur_xt * TP + tid;
                if (r < N && m0 < HKM_INF) {
                    const unsigned long long key =
                        (static_cast<unsigned long long>(__float_as_uint(m0)) << 32) | unsigned(i0);
                    atomicMin(keys + r, key);
                }
            }
        }
    }
}

int launch_assign_mfma_stream(const float* X, int64_t N, int32_t D, int64_t ldx, const float* C,
                              int32_t K, int64_t ldc, const float* cn, unsigned long long* keys,
                              int32_t* labels, float* min_d2, bool split, hipStream_t st) {
    const bool vec = aligned16(X) && aligned16(C) && (ldx % 4 == 0) && (ldc % 4 == 0) && (D % 4 == 0);
    // per-thread offsets inside a 128-row tile are 32-bit byte offsets
    if (ldx >= (int64_t(1) << 22) || ldc >= (int64_t(1) << 22))
        return fail(HKM_EUNSUPPORTED, "assign_mfma_stream: leading dimension of 2^22 elements or more");
    const int64_t ntiles = (N + 127) / 128;
    const StreamPlan pl = stream_plan(N, D, K);
    int64_t fgrid = (N + 255) / 256;
    const int64_t fcap = int64_t(num_cus()) * 8;
    if (fgrid > fcap) fgrid = fcap;
    hipLaunchKernelGGL(fill_keys_kernel, dim3((unsigned)fgrid), dim3(256), 0, st, keys, N);
    int rc = check_launch("fill_keys_kernel");
    if (rc) return rc;
    prof_begin(st);
    if (split && vec)
        hipLaunchKernelGGL(assign_split_stream_kernel<true>, dim3(pl.grid), dim3(256), 0, st, X, N, D, ldx,
                           C, K, ldc, cn, keys, ntiles, pl.nct, pl.ndc, pl.W, pl.PG);
    else if (split)
        hipLaunchKernelGGL(assign_split_stream_kernel<false>, dim3(pl.grid), dim3(256), 0, st, X, N, D, ldx,
                           C, K, ldc, cn, keys, ntiles, pl.nct, pl.ndc, pl.W, pl.PG);
    else if (vec)
        hipLaunchKernelGGL(assign_mfma_stream_kernel<true>, dim3(pl.grid), dim3(256), 0, st, X, N, D, ldx,
                           C, K, ldc, cn, keys, ntiles, pl.nct, pl.ndc, pl.W, pl.PG);
    else
        hipLaunchKernelGGL(assign_mfma_stream_kernel<false>, dim3(pl.grid), dim3(256), 0, st, X, N, D,
                           ldx, C, K, ldc, cn, keys, ntiles, pl.nct, pl.ndc, pl.W, pl.PG);
    prof_end(st);
    if ((rc = check_launch("assign_mfma_stream_kernel"))) return rc;
    hipLaunchKernelGGL(unpack_keys_kernel, dim3((unsigned)fgrid), dim3(256), 0, st, keys, N, labels, min_d2);
    return check_launch("unpack_keys_kernel");
}

}  // namespace hkm
