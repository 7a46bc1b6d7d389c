// Device helpers shared by the matrix-core kernels (fp32 and split-bf16 products).
#pragma once
#include "hkm_common.h"

namespace hkm {

#define MFMA32(a, b, c) __builtin_amdgcn_mfma_f32_32x32x2f32((a), (b), (c), 0, 0, 0)

__device__ __forceinline__ floatx4 ld4(const float* p) {
    return *reinterpret_cast<const floatx4*>(p);
}

// 16 bytes of row `p` starting at column c; columns >= D read as zero.  VEC: p + c is 16-B aligned
// and D % 4 == 0, so a group is either fully inside or fully outside the row.
template <bool VEC>
__device__ __forceinline__ floatx4 load_row4(const float* row, int c, int D) {
    floatx4 v = {0.f, 0.f, 0.f, 0.f};
    if (VEC) {
        if (c < D) v = ld4(row + c);
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (c + t < D) v[t] = row[c + t];
    }
    return v;
}

__device__ __forceinline__ void merge_halves(float& m, int& mi) {
    const float om = __shfl_xor(m, 32);
    const int oi = __shfl_xor(mi, 32);
    if (om < m || (om == m && oi < mi)) {
        m = om;
        mi = oi;
    }
}

// the squared norms of the 16 centroid rows a lane owns in a block (cn16 points at the norm of row
// 4*h of the block; rows 8g + 4h .. 8g + 4h + 3 belong to accumulator elements 4g .. 4g + 3)
__device__ __forceinline__ floatx16 load_cn16(const float* cn16) {
    floatx16 c0;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const floatx4 t = ld4(cn16 + 8 * g);
#pragma unroll
        for (int q = 0; q < 4; ++q) c0[4 * g + q] = t[q];
    }
    return c0;
}

// Minimum and first argmin over the 16 distances a lane holds of one centroid block, merged into the
// running (m, mi).  The minimum is a tree of three-input minima (8 instructions, no dependence on
// compare results); only lanes whose block minimum improves the running one look for its position,
// by equality from the last register down so that the first one wins -- independent compares, then a
// chain of selects with literal indices.  Strict '<' keeps the earlier block on ties.  NaNs never win.
__device__ __forceinline__ void block_argmin(const floatx16& d, int kb, float& m, int& mi) {
    const float t0 = fminf(fminf(d[0], d[1]), d[2]);
    const float t1 = fminf(fminf(d[3], d[4]), d[5]);
    const float t2 = fminf(fminf(d[6], d[7]), d[8]);
    const float t3 = fminf(fminf(d[9], d[10]), d[11]);
    const float t4 = fminf(fminf(d[12], d[13]), d[14]);
    const float bm = fminf(fminf(fminf(t0, t1), t2), fminf(fminf(t3, t4), d[15]));
    if (bm < m) {
        // all compares first (each into its own scalar register pair), then the selects: a select
        // right behind the compare it consumes would wait for it
        bool e[15];
#pragma unroll
        for (int v = 0; v < 15; ++v) e[v] = d[v] == bm;
        __builtin_amdgcn_sched_barrier(0);
        int bi = 8 * (15 >> 2) + (15 & 3);
#pragma unroll
        for (int v = 14; v >= 0; --v) bi = e[v] ? 8 * (v >> 2) + (v & 3) : bi;
        mi = kb + bi;
        m = bm;
    }
}

// ---- split-bf16 products: an fp32 value as the sum of three bf16 parts ----
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

#define MFMA_BF16(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16((a), (b), (c), 0, 0, 0)

// two fp32 values -> their bf16 roundings packed in one register (element 0 in the low half)
__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
    const floatx2 v = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf16_lo(unsigned u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(unsigned u) { return __uint_as_float(u & 0xffff0000u); }

// three-way split of a pair; p1, p2, p3 receive the packed parts
__device__ __forceinline__ void split_pair(float a, float b, unsigned& p1, unsigned& p2, unsigned& p3) {
    p1 = pack_bf16(a, b);
    const float ra = a - bf16_lo(p1), rb = b - bf16_hi(p1);
    p2 = pack_bf16(ra, rb);
    p3 = pack_bf16(ra - bf16_lo(p2), rb - bf16_hi(p2));
}

__device__ __forceinline__ bf16x8 as_bf16x8(const uintx4& u) { return __builtin_bit_cast(bf16x8, u); }

}  // namespace hkm
