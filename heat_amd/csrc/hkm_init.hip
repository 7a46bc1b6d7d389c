// Device side of the k-means|| centroid initialisation (heat/cluster/_kcluster.py:146-247,283-350):
// the distance work is the assign kernel with its min d^2 output; what is left are an ordered
// Bernoulli selection of candidate rows, a histogram of labels and the k-means++ seeding of the
// candidates.  The first two are integer work and reproducible: the selection is a count / scan /
// write compaction in row order, the histogram uses integer atomics only; the seeding runs in one
// workgroup with a fixed order of every sum.
#include "hkm_common.h"

namespace hkm {

// row i is selected iff u[i] <= (oversampling * sqrt(min_d2[i])) / max(cost, 1e-12), evaluated in
// fp32 in that order (_kcluster.py:314-322)
__device__ __forceinline__ bool selected(float d2, float u, float os, float denom) {
    const float p = (os * sqrtf(d2)) / denom;
    return u <= p;
}

__global__ __launch_bounds__(256) void select_count_kernel(const float* __restrict__ d2,
                                                           const float* __restrict__ u, int64_t n,
                                                           int64_t per_block,
                                                           const float* __restrict__ cost, float os,
                                                           long long* __restrict__ block_cnt, bool vec) {
    __shared__ int sh[256];
    const float denom = fmaxf(*cost, 1e-12f);
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    int c = 0;
    int64_t i0 = b0;
    if (vec) {  // both arrays 16-byte aligned, per_block a multiple of 1024: whole 16-byte groups
        for (; i0 + 1024 <= b1; i0 += 1024) {
            const float4 a = *reinterpret_cast<const float4*>(d2 + i0 + threadIdx.x * 4);
            const float4 b = *reinterpret_cast<const float4*>(u + i0 + threadIdx.x * 4);
            c += (selected(a.x, b.x, os, denom) ? 1 : 0) + (selected(a.y, b.y, os, denom) ? 1 : 0) +
                 (selected(a.z, b.z, os, denom) ? 1 : 0) + (selected(a.w, b.w, os, denom) ? 1 : 0);
        }
    }
    for (int64_t i = i0 + threadIdx.x; i < b1; i += 256) c += selected(d2[i], u[i], os, denom) ? 1 : 0;
    sh[threadIdx.x] = c;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if (threadIdx.x < w) sh[threadIdx.x] += sh[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) block_cnt[blockIdx.x] = sh[0];
}

// exclusive scan of the block counts in place (nb <= RED_SLOTS), total to *count
__global__ __launch_bounds__(256) void select_scan_kernel(long long* __restrict__ block_cnt, int nb,
                                                          long long* __restrict__ count) {
    __shared__ long long sh[256];
    const int per = (nb + 255) / 256;
    const int i0 = threadIdx.x * per, i1 = min(nb, i0 + per);
    long long s = 0;
    for (int i = i0; i < i1; ++i) s += block_cnt[i];
    sh[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        long long run = 0;
        for (int t = 0; t < 256; ++t) {
            const long long v = sh[t];
            sh[t] = run;
            run += v;
        }
        *count = run;
    }
    __syncthreads();
    long long run = sh[threadIdx.x];
    for (int i = i0; i < i1; ++i) {
        const long long v = block_cnt[i];
        block_cnt[i] = run;
        run += v;
    }
}

__global__ __launch_bounds__(256) void select_write_kernel(const float* __restrict__ d2,
                                                           const float* __restrict__ u, int64_t n,
                                                           int64_t per_block,
                                                           const float* __restrict__ cost, float os,
                                                           const long long* __restrict__ block_off,
                                                           const long long* __restrict__ count, int nb,
                                                           int64_t* __restrict__ idx, int64_t cap) {
    __shared__ int wave_cnt[4];
    // a block without a selected row (nearly all of them: a round selects a handful of rows) is done
    const long long mine = (int(blockIdx.x) + 1 < nb ? block_off[blockIdx.x + 1] : *count) - block_off[blockIdx.x];
    if (mine == 0) return;
    const float denom = fmaxf(*cost, 1e-12f);
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    long long run = block_off[blockIdx.x];
    for (int64_t base = b0; base < b1; base += 256) {
        const int64_t i = base + threadIdx.x;
        const bool f = i < b1 && selected(d2[i], u[i], os, denom);
        const unsigned long long m = __ballot(f);
        const int before = __popcll(m & ((1ull << lane) - 1ull));
        if (lane == 0) wave_cnt[wave] = __popcll(m);
        __syncthreads();
        int off = 0, tot = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int c = wave_cnt[w];
            if (w < wave) off += c;
            tot += c;
        }
        if (f) {
            const long long pos = run + off + before;
            if (pos < cap) idx[pos] = i;
        }
        run += tot;
        __syncthreads();
    }
}

int launch_select(const float* d2, const float* u, int64_t N, const float* cost, float os,
                  int64_t* idx, int64_t cap, int64_t* count, double* red, hipStream_t st) {
    // short blocks: the few blocks that hold a selected row walk their range in dependent steps of 256
    // rows in the write pass and set its duration
    int nb = int((N + 2047) / 2048);
    if (nb < 1) nb = 1;
    if (nb > RED_SLOTS) nb = RED_SLOTS;
    int64_t per_block = N > 0 ? (N + nb - 1) / nb : 1;
    per_block = (per_block + 1023) / 1024 * 1024;
    nb = int((N + per_block - 1) / per_block);
    if (nb < 1) nb = 1;
    long long* bc = reinterpret_cast<long long*>(red);
    const bool vec = aligned16(d2) && aligned16(u);
    hipLaunchKernelGGL(select_count_kernel, dim3(nb), dim3(256), 0, st, d2, u, N, per_block, cost, os, bc, vec);
    int rc = check_launch("select_count_kernel");
    if (rc) return rc;
    hipLaunchKernelGGL(select_scan_kernel, dim3(1), dim3(256), 0, st, bc, nb,
                       reinterpret_cast<long long*>(count));
    if ((rc = check_launch("select_scan_kernel"))) return rc;
    hipLaunchKernelGGL(select_write_kernel, dim3(nb), dim3(256), 0, st, d2, u, N, per_block, cost, os,
                       bc, reinterpret_cast<const long long*>(count), nb, idx, cap);
    return check_launch("select_write_kernel");
}

// ---- histogram of labels ---------------------------------------------------------------------
static constexpr int HIST_LDS = 4096;

__global__ __launch_bounds__(256) void zero_i64_kernel(long long* __restrict__ p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

__global__ __launch_bounds__(256) void label_hist_kernel(const int32_t* __restrict__ labels,
                                                         int64_t n, int64_t per_block, int K,
                                                         unsigned long long* __restrict__ counts) {
    __shared__ unsigned int sh[HIST_LDS];
    const bool lds = K <= HIST_LDS;
    if (lds) {
        for (int k = threadIdx.x; k < K; k += 256) sh[k] = 0;
        __syncthreads();
    }
    const int64_t b0 = int64_t(blockIdx.x) * per_block;
    const int64_t b1 = min(n, b0 + per_block);
    for (int64_t i = b0 + threadIdx.x; i < b1; i += 256) {
        const int l = labels[i];
        if (l < 0 || l >= K) continue;
        if (lds) atomicAdd(&sh[l], 1u);
        else atomicAdd(&counts[l], 1ull);
    }
    if (lds) {
        __syncthreads();
        for (int k = threadIdx.x; k < K; k += 256) {
            const unsigned int c = sh[k];
            if (c) atomicAdd(&counts[k], (unsigned long long)c);
        }
    }
}

int launch_label_counts(const int32_t* labels, int64_t N, int32_t K, int64_t* counts,
                        hipStream_t st) {
    hipLaunchKernelGGL(zero_i64_kernel, dim3((K + 255) / 256), dim3(256), 0, st,
                       reinterpret_cast<long long*>(counts), K);
    int rc = check_launch("zero_i64_kernel");
    if (rc || N == 0) return rc;
    int64_t nb = (N + 65535) / 65536;
    const int64_t cap = int64_t(num_cus()) * 8;
    if (nb > cap) nb = cap;
    const int64_t per_block = (N + nb - 1) / nb;
    hipLaunchKernelGGL(label_hist_kernel, dim3((unsigned)nb), dim3(256), 0, st, labels, N, per_block, K,
                       reinterpret_cast<unsigned long long*>(counts));
    return check_launch("label_hist_kernel");
}

// ---- k-means++ seeding of a small row set in one launch ------------------------------------------
// heat/cluster/batchparallelclustering.py:22-46 on the candidates of k-means|| (a few hundred to a few
// thousand rows): K - 1 sequential categorical draws with probability proportional to
// weight * (distance to the closest centre chosen so far).  Issued from the host, every draw is a
// dozen launches of a few hundred threads; here one workgroup keeps the running distances in
// registers and does a draw in a few microseconds:
//   * thread t owns the rows [t R, (t + 1) R), R = ceil(M / 1024) <= SEED_RPT, so thread order is row order;
//   * the distance of a row to the newest centre is the direct form, summed in feature order and
//     followed by the correctly rounded square root (p = 2) or sum |x - c| (p = 1): the same numbers
//     hkm_pairwise_f32 returns for that column;
//   * weight * distance is formed in fp32, as the host code would, and scanned in fp64 in row order
//     (sequential inside a thread, shuffle scan across a wave, wave totals through LDS);
//   * draw k picks the first row whose inclusive prefix exceeds u[k - 1] * total (inverse CDF).  A row
//     with weight * distance = 0 -- in particular every centre already chosen -- cannot be picked.
// total <= 0 (every row coincides with a chosen centre, or all weights are zero) has no valid
// distribution: the remaining entries of idx are set to -1.
static constexpr int SEED_THREADS = 1024;
static constexpr int SEED_RPT = HKM_SEED_MAX_ROWS / SEED_THREADS;

template <int P>
__device__ __forceinline__ float seed_row_dist(const float* __restrict__ x, const float* __restrict__ c, int D) {
    float acc = 0.f;
    for (int f = 0; f < D; ++f) {
        const float df = x[f] - c[f];
        acc = P == 1 ? acc + fabsf(df) : fmaf(df, df, acc);
    }
    return P == 1 ? acc : sqrtf(acc);
}

template <int P>
__global__ __launch_bounds__(SEED_THREADS) void seed_plus_plus_kernel(const float* __restrict__ X, int M, int D,
                                                                      int64_t ldx, const float* __restrict__ w,
                                                                      int first, const float* __restrict__ u, int K,
                                                                      long long* __restrict__ idx) {
    __shared__ double s_wave[SEED_THREADS / 64];
    __shared__ int s_pick, s_last;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int R = (M + SEED_THREADS - 1) / SEED_THREADS;
    const int r0 = tid * R;
    float dist[SEED_RPT], wt[SEED_RPT];
#pragma unroll
    for (int r = 0; r < SEED_RPT; ++r) {
        dist[r] = 0.f;
        wt[r] = (r < R && r0 + r < M) ? (w ? w[r0 + r] : 1.0f) : 0.f;
    }
    int cur = first;
    if (tid == 0) idx[0] = first;
    for (int k = 1; k < K; ++k) {
        // running distance to the closest chosen centre, and this thread's share of the mass
        const float* c = X + int64_t(cur) * ldx;
        double mine = 0.0;
#pragma unroll
        for (int r = 0; r < SEED_RPT; ++r)
            if (r < R && r0 + r < M) {
                const float d = seed_row_dist<P>(X + int64_t(r0 + r) * ldx, c, D);
                dist[r] = k == 1 ? d : fminf(dist[r], d);
                mine += double(wt[r] * dist[r]);
            }
        // inclusive scan over the threads, in thread (= row) order
        double incl = mine;
#pragma unroll
        for (int s = 1; s < 64; s <<= 1) {
            const double o = __shfl_up(incl, s);
            if (lane >= s) incl += o;
        }
        if (tid == 0) {
            s_pick = 0x7fffffff;
            s_last = -1;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        double before = 0.0, total = 0.0;
#pragma unroll
        for (int v = 0; v < SEED_THREADS / 64; ++v) {
            if (v < wave) before += s_wave[v];
            total += s_wave[v];
        }
        if (!(total > 0.0)) {  // uniform: every thread sees the same total
            for (int j = k + tid; j < K; j += SEED_THREADS) idx[j] = -1;
            return;
        }
        const double target = double(u[k - 1]) * total;
        double run = before + (incl - mine);
        int pick = 0x7fffffff, last = -1;
#pragma unroll
        for (int r = 0; r < SEED_RPT; ++r)
            if (r < R && r0 + r < M) {
                const float wd = wt[r] * dist[r];
                run += double(wd);
                if (wd > 0.f) {
                    last = r0 + r;
                    if (run > target && pick == 0x7fffffff) pick = r0 + r;
                }
            }
        if (pick != 0x7fffffff) atomicMin(&s_pick, pick);
        if (last >= 0) atomicMax(&s_last, last);
        __syncthreads();
        // rounding may leave the last prefix a hair below u * total: the last row with mass then
        cur = s_pick != 0x7fffffff ? s_pick : s_last;
        if (tid == 0) idx[k] = cur;
        __syncthreads();  // s_pick / s_last are reset at the top of the next draw
    }
}

// ---- k-means++ seeding of a large row set: two launches per draw, no host round trip --------------
// The same draws as seed_plus_plus_kernel for up to 2^24 rows (BatchParallelKMeans seeds its local rows
// this way, heat/cluster/batchparallelclustering.py:22-46,270-276).  Per draw:
//   seed_rows_dist_kernel  one read of X: distance of every row to the newest centre (eight lanes per
//                          row, 16-byte loads, four rows in flight per lane group), running minimum
//                          in `dist`, and the fp64 sum of weight * distance of every block of rows;
//   seed_rows_pick_kernel  one workgroup: scans the block sums in block order, finds the block that
//                          holds u * total, then scans that block's rows in row order.
// The newest centre is read from idx[k - 1] on the device, so the K - 1 draws are enqueued back to back.
// A draw that finds no mass writes -1; every later launch sees it and passes it on.
__global__ void seed_rows_first_kernel(long long* __restrict__ idx, long long first) { idx[0] = first; }

static constexpr int SEEDR_THREADS = 256;
static constexpr int SEEDR_LPR = 8;     // lanes per row
static constexpr int SEEDR_PICK_T = 1024;
static constexpr int SEEDR_MAX_PER_BLOCK = 8192;  // rows of one block: 8 per thread of the pick kernel

template <int P, bool VEC>
__global__ __launch_bounds__(SEEDR_THREADS) void seed_rows_dist_kernel(
    const float* __restrict__ X, int64_t M, int D, int64_t ldx, const float* __restrict__ w,
    const long long* __restrict__ idx, int k, int64_t per_block, float* __restrict__ dist,
    double* __restrict__ block_sum) {
    __shared__ double sh[SEEDR_THREADS];
    const long long cur = idx[k - 1];
    if (cur < 0) return;  // an earlier draw found no mass
    const float* c = X + cur * ldx;
    const int tid = threadIdx.x, sub = tid & (SEEDR_LPR - 1), grp = tid / SEEDR_LPR;
    constexpr int GROUPS = SEEDR_THREADS / SEEDR_LPR;  // rows per pass of the workgroup
    constexpr int UF = 4;
    const int64_t b0 = int64_t(blockIdx.x) * per_block, b1 = min(M, b0 + per_block);
    double mass = 0.0;
    for (int64_t r0 = b0 + grp; r0 < b1; r0 += int64_t(GROUPS) * UF) {
        float acc[UF];
#pragma unroll
        for (int t = 0; t < UF; ++t) acc[t] = 0.f;
        if (VEC) {
            for (int f = 4 * sub; f < D; f += 4 * SEEDR_LPR) {
                const float4 cv = *reinterpret_cast<const float4*>(c + f);
                float4 xv[UF];
#pragma unroll
                for (int t = 0; t < UF; ++t) {
                    const int64_t r = r0 + int64_t(t) * GROUPS;
                    xv[t] = *reinterpret_cast<const float4*>(X + (r < b1 ? r : b0) * ldx + f);
                }
#pragma unroll
                for (int t = 0; t < UF; ++t) {
                    const float d0 = xv[t].x - cv.x, d1 = xv[t].y - cv.y, d2 = xv[t].z - cv.z, d3 = xv[t].w - cv.w;
                    if (P == 1) acc[t] += (fabsf(d0) + fabsf(d1)) + (fabsf(d2) + fabsf(d3));
                    else acc[t] = fmaf(d3, d3, fmaf(d2, d2, fmaf(d1, d1, fmaf(d0, d0, acc[t]))));
                }
            }
        } else {
            for (int f = sub; f < D; f += SEEDR_LPR) {
                const float cv = c[f];
#pragma unroll
                for (int t = 0; t < UF; ++t) {
                    const int64_t r = r0 + int64_t(t) * GROUPS;
                    const float df = X[(r < b1 ? r : b0) * ldx + f] - cv;
                    acc[t] = P == 1 ? acc[t] + fabsf(df) : fmaf(df, df, acc[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < UF; ++t) {
            float a = acc[t];
            a += __shfl_xor(a, 1);
            a += __shfl_xor(a, 2);
            a += __shfl_xor(a, 4);
            const int64_t r = r0 + int64_t(t) * GROUPS;
            if (sub == 0 && r < b1) {
                float d = P == 1 ? a : sqrtf(a);
                if (r == cur) d = 0.f;  // exactly zero for the row itself, whatever the summation order
                if (k > 1) d = fminf(dist[r], d);
                dist[r] = d;
                mass += double((w ? w[r] : 1.0f) * d);
            }
        }
    }
    const double t = block_sum_fixed(mass, sh);
    if (tid == 0) block_sum[blockIdx.x] = t;
}

// inclusive scan of one value per thread in thread order; *total receives the sum (all threads)
__device__ __forceinline__ double seed_block_scan(double v, double* s_wave, double& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    double incl = v;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const double o = __shfl_up(incl, s);
        if (lane >= s) incl += o;
    }
    __syncthreads();  // s_wave may still be read from the previous scan
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    double before = 0.0;
    total = 0.0;
    for (int q = 0; q < SEEDR_PICK_T / 64; ++q) {
        if (q < wave) before += s_wave[q];
        total += s_wave[q];
    }
    return before + incl;
}

__global__ __launch_bounds__(SEEDR_PICK_T) void seed_rows_pick_kernel(
    int64_t M, const float* __restrict__ w, const float* __restrict__ u, int k, int K, int64_t per_block,
    int nb, const float* __restrict__ dist, const double* __restrict__ block_sum, long long* __restrict__ idx) {
    __shared__ double s_wave[SEEDR_PICK_T / 64];
    __shared__ int s_pick, s_last;
    __shared__ double s_before;
    const int tid = threadIdx.x;
    if (idx[k - 1] < 0) {
        if (tid == 0) idx[k] = -1;
        return;
    }
    // 1. the block that holds u * total
    const int bper = (nb + SEEDR_PICK_T - 1) / SEEDR_PICK_T;
    double mine = 0.0;
    for (int q = 0; q < bper; ++q) {
        const int b = tid * bper + q;
        if (b < nb) mine += block_sum[b];
    }
    if (tid == 0) {
        s_pick = 0x7fffffff;
        s_last = -1;
    }
    double total;
    const double incl = seed_block_scan(mine, s_wave, total);
    if (!(total > 0.0)) {
        if (tid == 0) idx[k] = -1;
        return;
    }
    const double target = double(u[k - 1]) * total;
    {
        double run = incl - mine;
        int pick = 0x7fffffff, last = -1;
        double before_pick = 0.0;
        for (int q = 0; q < bper; ++q) {
            const int b = tid * bper + q;
            if (b < nb) {
                const double v = block_sum[b];
                if (v > 0.0) {
                    last = b;
                    if (run + v > target && pick == 0x7fffffff) {
                        pick = b;
                        before_pick = run;
                    }
                }
                run += v;
            }
        }
        if (pick != 0x7fffffff) atomicMin(&s_pick, pick);
        if (last >= 0) atomicMax(&s_last, last);
        __syncthreads();
        const int chosen = s_pick != 0x7fffffff ? s_pick : s_last;
        // the mass in front of the chosen block, from the thread that owns it
        if (chosen >= tid * bper && chosen < (tid + 1) * bper) {
            double r2 = incl - mine;
            for (int b = tid * bper; b < chosen; ++b) r2 += block_sum[b];
            s_before = r2;
        }
        __syncthreads();
        (void)before_pick;
    }
    const int blk = s_pick != 0x7fffffff ? s_pick : s_last;
    const double tin = target - s_before;  // target inside the block
    __syncthreads();
    if (tid == 0) {
        s_pick = 0x7fffffff;
        s_last = -1;
    }
    // 2. the row inside the block, rows in row order: thread t owns R consecutive rows
    const int64_t b0 = int64_t(blk) * per_block, b1 = min(M, b0 + per_block);
    const int R = int((per_block + SEEDR_PICK_T - 1) / SEEDR_PICK_T);
    float wd[SEEDR_MAX_PER_BLOCK / SEEDR_PICK_T];
    double rows = 0.0;
#pragma unroll
    for (int q = 0; q < SEEDR_MAX_PER_BLOCK / SEEDR_PICK_T; ++q) {
        const int64_t r = b0 + int64_t(tid) * R + q;
        wd[q] = (q < R && r < b1) ? (w ? w[r] : 1.0f) * dist[r] : 0.f;
        rows += double(wd[q]);
    }
    double tot2;
    const double incl2 = seed_block_scan(rows, s_wave, tot2);
    double run = incl2 - rows;
    int pick = 0x7fffffff, last = -1;
#pragma unroll
    for (int q = 0; q < SEEDR_MAX_PER_BLOCK / SEEDR_PICK_T; ++q) {
        run += double(wd[q]);
        if (wd[q] > 0.f) {
            last = tid * R + q;
            if (run > tin && pick == 0x7fffffff) pick = tid * R + q;
        }
    }
    if (pick != 0x7fffffff) atomicMin(&s_pick, pick);
    if (last >= 0) atomicMax(&s_last, last);
    __syncthreads();
    if (tid == 0) {
        const int off = s_pick != 0x7fffffff ? s_pick : s_last;  // the chosen block has mass, so off >= 0
        idx[k] = off >= 0 ? b0 + off : -1;
    }
}

int launch_seed_plus_plus_rows(const float* X, int64_t M, int32_t D, int64_t ldx, const float* w, int64_t first,
                               const float* u, int32_t K, int32_t p, int64_t* idx, float* dist, double* red,
                               hipStream_t st) {
    long long* idx_ll = reinterpret_cast<long long*>(idx);
    hipLaunchKernelGGL(seed_rows_first_kernel, dim3(1), dim3(1), 0, st, idx_ll, (long long)first);
    int rc = check_launch("seed_rows_first_kernel");
    if (rc) return rc;
    int nb = int((M + 4095) / 4096);
    if (nb < 1) nb = 1;
    if (nb > RED_SLOTS) nb = RED_SLOTS;
    int64_t per_block = ((M + nb - 1) / nb + 31) / 32 * 32;
    nb = int((M + per_block - 1) / per_block);
    const bool vec = aligned16(X) && ldx % 4 == 0 && D % 4 == 0;
    for (int k = 1; k < K; ++k) {
#define HKM_GO(PP, V)                                                                                          \
    hipLaunchKernelGGL((seed_rows_dist_kernel<PP, V>), dim3(nb), dim3(SEEDR_THREADS), 0, st, X, M, D, ldx, w, \
                       idx_ll, k, per_block, dist, red)
        if (p == 1) {
            if (vec) HKM_GO(1, true);
            else HKM_GO(1, false);
        } else {
            if (vec) HKM_GO(2, true);
            else HKM_GO(2, false);
        }
#undef HKM_GO
        if ((rc = check_launch("seed_rows_dist_kernel"))) return rc;
        hipLaunchKernelGGL(seed_rows_pick_kernel, dim3(1), dim3(SEEDR_PICK_T), 0, st, M, w, u, k, K, per_block, nb,
                           dist, red, idx_ll);
        if ((rc = check_launch("seed_rows_pick_kernel"))) return rc;
    }
    return HKM_OK;
}

int launch_seed_plus_plus(const float* X, int32_t M, int32_t D, int64_t ldx, const float* w, int32_t first,
                          const float* u, int32_t K, int32_t p, int64_t* idx, hipStream_t st) {
    if (p == 1)
        hipLaunchKernelGGL(seed_plus_plus_kernel<1>, dim3(1), dim3(SEED_THREADS), 0, st, X, M, D, ldx, w, first, u, K,
                           reinterpret_cast<long long*>(idx));
    else
        hipLaunchKernelGGL(seed_plus_plus_kernel<2>, dim3(1), dim3(SEED_THREADS), 0, st, X, M, D, ldx, w, first, u, K,
                           reinterpret_cast<long long*>(idx));
    return check_launch("seed_plus_plus_kernel");
}

}  // namespace hkm
