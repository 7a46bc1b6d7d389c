// Microbenchmarks behind the hardware figures the kernel design rests on (bench.py --probe):
//   hkm_probe_mfma_f32  a chain of fp32 matrix instructions, alone or with NOPS instructions of one other kind
//                       issued after each of them: what the matrix pipe delivers and what other work costs it;
//   hkm_probe_stream    copy / read / fill of a large buffer: what the memory system delivers.
// They launch one kernel each on the given stream and are timed by the caller.  This file is a library of
// its own (libhkm_bench.so, declared in include/hkm_bench.h): only the benchmark loads it, the product library
// holds none of it.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "hkm_bench.h"

namespace hkm_bench {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

static thread_local char g_err[256] = "";

static int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HKM_BENCH_EHIP, "%s: %s", what, hipGetErrorString(e));
    return 0;
}

static int num_cus() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return 256;
    return n;
}

enum { PROBE_NONE = 0, PROBE_FMA = 1, PROBE_CNDMASK = 2, PROBE_MIN3 = 3, PROBE_SALU = 4, PROBE_CMP = 5, PROBE_MOV64 = 6 };

template <int OP, int NOPS>
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* out, int iters, float a0, float b0) {
    floatx16 acc[2];
    for (int i = 0; i < 2; ++i)
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    float a = a0 + threadIdx.x, b = b0;
    float r0 = a0, r1 = b0, r2 = 3.f;
    int s0 = iters;
    double q0 = a0, q1 = b0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
#pragma unroll
                for (int w = 0; w < NOPS; ++w) {
                    if (OP == PROBE_FMA) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(r0) : "v"(r1), "v"(r2));
                    if (OP == PROBE_CNDMASK) asm volatile("v_cndmask_b32 %0, %1, %2, vcc" : "+v"(r0) : "v"(r1), "v"(r2));
                    if (OP == PROBE_MIN3) asm volatile("v_min3_f32 %0, %0, %1, %2" : "+v"(r0) : "v"(r1), "v"(r2));
                    if (OP == PROBE_SALU) asm volatile("s_add_u32 %0, %0, 1" : "+s"(s0) : : "scc");
                    if (OP == PROBE_CMP) asm volatile("v_cmp_lt_f32 vcc, %0, %1" : : "v"(r0), "v"(r1) : "vcc");
                    if (OP == PROBE_MOV64) asm volatile("v_mov_b64 %0, %1" : "=v"(q0) : "v"(q1));
                }
            }
        }
    }
    float s = r0 + r1 + r2 + float(s0) + float(q0);
    for (int i = 0; i < 2; ++i)
        for (int v = 0; v < 16; ++v) s += acc[i][v];
    out[size_t(blockIdx.x) * blockDim.x + threadIdx.x] = s;
}

template <int MODE>  // 0 copy, 1 read, 2 read with non-temporal loads, 3 fill
__global__ __launch_bounds__(256) void probe_stream_kernel(const floatx4* __restrict__ src, floatx4* __restrict__ dst,
                                                           size_t n4, float* sink) {
    constexpr int U = 4;
    size_t i = size_t(blockIdx.x) * 256 * U + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * 256 * U;
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
    for (; i + 256 * (U - 1) < n4; i += stride) {
        floatx4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (MODE == 3) v[u] = floatx4{1.f, 2.f, 3.f, 4.f};
            else v[u] = MODE == 2 ? __builtin_nontemporal_load(src + i + 256 * u) : src[i + 256 * u];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (MODE == 0 || MODE == 3) dst[i + 256 * u] = v[u];
            else s += v[u];
        }
    }
    const float t = s[0] + s[1] + s[2] + s[3];
    if (t == 123.456f) sink[0] = t;  // keeps the reads
}

static int launch_probe_mfma(int32_t op, int32_t nops, int32_t iters, int32_t grid, float* out, hipStream_t st) {
#define HKM_P(O, N)                                                                                        \
    if (op == O && nops == N) {                                                                            \
        hipLaunchKernelGGL((probe_mfma_kernel<O, N>), dim3(grid), dim3(256), 0, st, out, iters, 1.f, 2.f); \
        return check_launch("probe_mfma_kernel");                                                          \
    }
    HKM_P(PROBE_NONE, 0)
    HKM_P(PROBE_FMA, 4) HKM_P(PROBE_FMA, 8) HKM_P(PROBE_CNDMASK, 4) HKM_P(PROBE_CNDMASK, 8)
    HKM_P(PROBE_MIN3, 4) HKM_P(PROBE_MIN3, 8) HKM_P(PROBE_SALU, 4) HKM_P(PROBE_SALU, 8)
    HKM_P(PROBE_CMP, 4) HKM_P(PROBE_CMP, 8) HKM_P(PROBE_MOV64, 4) HKM_P(PROBE_MOV64, 8)
#undef HKM_P
    return fail(HKM_BENCH_EINVAL, "hkm_probe_mfma_f32: no kernel for op = %d with %d instructions per matrix instruction", op, nops);
}

static int launch_probe_stream(const void* src, void* dst, size_t bytes, int32_t mode, float* sink, hipStream_t st) {
    const size_t n4 = bytes / 16;
    const int grid = num_cus() * 8;
    const floatx4* s = static_cast<const floatx4*>(src);
    floatx4* d = static_cast<floatx4*>(dst);
    switch (mode) {
        case 0: hipLaunchKernelGGL(probe_stream_kernel<0>, dim3(grid), dim3(256), 0, st, s, d, n4, sink); break;
        case 1: hipLaunchKernelGGL(probe_stream_kernel<1>, dim3(grid), dim3(256), 0, st, s, d, n4, sink); break;
        case 2: hipLaunchKernelGGL(probe_stream_kernel<2>, dim3(grid), dim3(256), 0, st, s, d, n4, sink); break;
        case 3: hipLaunchKernelGGL(probe_stream_kernel<3>, dim3(grid), dim3(256), 0, st, s, d, n4, sink); break;
        default: return fail(HKM_BENCH_EINVAL, "hkm_probe_stream: mode = %d must be 0 (copy), 1 (read), 2 (streaming read) or 3 (fill)", mode);
    }
    return check_launch("probe_stream_kernel");
}

}  // namespace hkm_bench

using namespace hkm_bench;

extern "C" {

const char* hkm_bench_last_error(void) { return g_err; }

int hkm_probe_mfma_f32(int32_t op, int32_t nops, int32_t iters, int32_t grid, float* out, void* hip_stream) {
    g_err[0] = 0;
    if (iters < 1 || grid < 1 || !out)
        return fail(HKM_BENCH_EINVAL, "hkm_probe_mfma_f32: iters and grid must be >= 1 and out not NULL");
    return launch_probe_mfma(op, nops, iters, grid, out, static_cast<hipStream_t>(hip_stream));
}

int hkm_probe_stream(const void* src, void* dst, size_t bytes, int32_t mode, float* sink, void* hip_stream) {
    g_err[0] = 0;
    if (bytes < 16 || !sink || (mode != 3 && !src) || ((mode == 0 || mode == 3) && !dst))
        return fail(HKM_BENCH_EINVAL, "hkm_probe_stream: NULL buffer or fewer than 16 bytes");
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u)
        return fail(HKM_BENCH_EINVAL, "hkm_probe_stream: buffers must be 16-byte aligned");
    return launch_probe_stream(src, dst, bytes, mode, sink, static_cast<hipStream_t>(hip_stream));
}

}  // extern "C"
