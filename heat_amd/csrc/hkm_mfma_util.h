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
// running (m, mi).  The minimum is a tree of three-input minima (9 instructions, no dependence on
// compare results); only lanes whose block minimum improves the running one look for its position,
// by equality from the last register down so that the first one wins.  Strict '<' keeps the earlier
// block on ties.  NaNs never win.
//
// Both halves are written out as instructions: the compiler's own form of the tree spends more
// instructions on canonicalising operands that are matrix-core results, and it places every compare of
// the lookup directly in front of the select that consumes it, which on this chip costs two idle cycles
// per pair (a vector instruction must not read a scalar register pair written by the instruction before
// it).  Here the compares run two ahead of the selects through three scalar register pairs, so no pair
// is read within two instructions of being written and nothing idles.
__device__ __forceinline__ float block_min16(const floatx16& d) {
    // The first read of the block is left to the compiler (a canonicalisation: one instruction that
    // returns its operand): it knows how many idle cycles a read of fresh matrix-core results needs,
    // which an instruction sequence it cannot see into would not get.
    const float t0 = __builtin_canonicalizef(d[0]);
    float a, b, c, e;
    asm("v_min3_f32 %[a], %[t0], %[d1], %[d2]\n\t"
        "v_min3_f32 %[b], %[d3], %[d4], %[d5]\n\t"
        "v_min3_f32 %[c], %[d6], %[d7], %[d8]\n\t"
        "v_min3_f32 %[e], %[d9], %[d10], %[d11]\n\t"
        "v_min3_f32 %[a], %[a], %[b], %[c]\n\t"
        "v_min3_f32 %[b], %[d12], %[d13], %[d14]\n\t"
        "v_min3_f32 %[a], %[a], %[e], %[b]\n\t"
        "v_min_f32 %[a], %[a], %[d15]"
        : [a] "=&v"(a), [b] "=&v"(b), [c] "=&v"(c), [e] "=&v"(e)
        : [t0] "v"(t0), [d1] "v"(d[1]), [d2] "v"(d[2]), [d3] "v"(d[3]), [d4] "v"(d[4]), [d5] "v"(d[5]), [d6] "v"(d[6]),
          [d7] "v"(d[7]), [d8] "v"(d[8]), [d9] "v"(d[9]), [d10] "v"(d[10]), [d11] "v"(d[11]), [d12] "v"(d[12]),
          [d13] "v"(d[13]), [d14] "v"(d[14]), [d15] "v"(d[15]));
    return a;
}

// position (8 * (v / 4) + v % 4 for register v: the centroid row inside the block, without the
// lane-half term) of the first of the 16 distances that equals bm
__device__ __forceinline__ int block_pos16(const floatx16& d, float bm) {
    int bi;
    unsigned long long s0, s1, s2;
    asm("v_cmp_eq_f32_e64 %[s0], %[d14], %[bm]\n\t"
        "v_cmp_eq_f32_e64 %[s1], %[d13], %[bm]\n\t"
        "v_cmp_eq_f32_e64 %[s2], %[d12], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], 27, 26, %[s0]\n\t"
        "v_cmp_eq_f32_e64 %[s0], %[d11], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 25, %[s1]\n\t"
        "v_cmp_eq_f32_e64 %[s1], %[d10], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 24, %[s2]\n\t"
        "v_cmp_eq_f32_e64 %[s2], %[d9], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 19, %[s0]\n\t"
        "v_cmp_eq_f32_e64 %[s0], %[d8], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 18, %[s1]\n\t"
        "v_cmp_eq_f32_e64 %[s1], %[d7], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 17, %[s2]\n\t"
        "v_cmp_eq_f32_e64 %[s2], %[d6], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 16, %[s0]\n\t"
        "v_cmp_eq_f32_e64 %[s0], %[d5], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 11, %[s1]\n\t"
        "v_cmp_eq_f32_e64 %[s1], %[d4], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 10, %[s2]\n\t"
        "v_cmp_eq_f32_e64 %[s2], %[d3], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 9, %[s0]\n\t"
        "v_cmp_eq_f32_e64 %[s0], %[d2], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 8, %[s1]\n\t"
        "v_cmp_eq_f32_e64 %[s1], %[d1], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 3, %[s2]\n\t"
        "v_cmp_eq_f32_e64 %[s2], %[d0], %[bm]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 2, %[s0]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 1, %[s1]\n\t"
        "v_cndmask_b32_e64 %[bi], %[bi], 0, %[s2]"
        : [bi] "=&v"(bi), [s0] "=&s"(s0), [s1] "=&s"(s1), [s2] "=&s"(s2)
        : [d0] "v"(d[0]), [d1] "v"(d[1]), [d2] "v"(d[2]), [d3] "v"(d[3]), [d4] "v"(d[4]), [d5] "v"(d[5]),
          [d6] "v"(d[6]), [d7] "v"(d[7]), [d8] "v"(d[8]), [d9] "v"(d[9]), [d10] "v"(d[10]), [d11] "v"(d[11]),
          [d12] "v"(d[12]), [d13] "v"(d[13]), [d14] "v"(d[14]), [bm] "v"(bm));
    return bi;
}

__device__ __forceinline__ void block_argmin(const floatx16& d, int kb, float& m, int& mi) {
    const float bm = block_min16(d);
    if (bm < m) {
        mi = kb + block_pos16(d, bm);
        m = bm;
    }
}

// The same running argmin with the lookup deferred: a block whose minimum improves the running one is
// only remembered -- its number and a copy of its 16 distances (eight 64-bit moves) -- and the position
// is looked up once, after the last block, in the copy that survived (kept_argmin).  Same result as
// block_argmin bit for bit: strict '<' keeps the earliest block that reaches the final minimum, the
// lookup its first position.  15 instead of 33 vector instructions per improving block.
__device__ __forceinline__ void block_min_keep(const floatx16& d, int cb, float& m, int& blk, floatx16& keep) {
    const float bm = block_min16(d);
    if (bm < m) {
        // written out so that the two values are updated where they live (the compiler's own form pairs the
        // minima of two point blocks into 64-bit moves and shuffles them into place first)
        asm("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3" : "+v"(m), "+v"(blk) : "v"(bm), "s"(cb));
        keep = d;
    }
}

// The copy starts out without a value: it is only read after a block improved on +inf (kept_argmin
// ignores it otherwise).  Declaring it written by an empty instruction sequence costs nothing, where
// sixteen zeros would cost sixteen moves per point block.
__device__ __forceinline__ void keep_undefined(floatx16& keep) { asm volatile("" : "=v"(keep)); }

// index (without the lane-half term) of the minimum that block_min_keep tracked; 0 if no block ever
// improved on +inf (all distances +inf or NaN), as block_argmin leaves it
__device__ __forceinline__ int kept_argmin(const floatx16& keep, float m, int blk) {
    const int pos = block_pos16(keep, m);
    return m < HKM_INF ? blk * 32 + pos : 0;
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
