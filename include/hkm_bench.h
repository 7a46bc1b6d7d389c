/*
 * hkm_bench.h -- measuring hooks and microbenchmarks around libhkm.  Nothing here replaces a line of the
 * reference (helmholtz-analytics/heat has no counterpart to any of it) and no caller of the library needs
 * it: only the benchmark binds these symbols.
 *
 *   - hkm_profile_enable / hkm_profile_collect / hkm_point_blocks / hkm_point_blocks_trial are exported by
 *     libhkm.so itself, because they report on launches the product library makes;
 *   - hkm_probe_mfma_f32 / hkm_probe_stream / hkm_bench_last_error live in a library of their own,
 *     libhkm_bench.so (heat_amd/csrc/hkm_probe.hip), which the product never loads.
 */
#ifndef HKM_BENCH_H
#define HKM_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HKM_BENCH_EINVAL (-1) /* bad argument */
#define HKM_BENCH_EHIP (-3)   /* a HIP runtime call failed */

/* ---- exported by libhkm.so ----------------------------------------------------------------------- */

/*
 * Timing of the dominant kernel.  After hkm_profile_enable(1) on the calling thread, every
 * hkm_assign_f32 / hkm_assign_static_f32 / hkm_lloyd_step_f32 / hkm_lloyd_fit_f32 call of that thread records
 * one pair of events on its stream, right before and right after the launch of its distance kernel (the one
 * hkm_assign_kernel_name / hkm_lloyd_kernel_name names: the fused distance + argmin kernel, or the one-sweep
 * kernel that also forms the per-cluster sums) and of nothing else.  hkm_profile_collect waits for the
 * recorded pairs, writes their durations in milliseconds to ms (HOST pointer, at most cap of them, in call
 * order), the number recorded to *count, and starts over.  At most 512 pairs are kept between two collects.
 * hkm_profile_enable(0) switches it off.  While off -- the default -- nothing is recorded and no event
 * exists.  hkm_profile_collect is the one call that waits for the device.
 */
int hkm_profile_enable(int32_t on);
int hkm_profile_collect(float* ms, int32_t cap, int32_t* count);

/*
 * The resident matrix-core kernels (up to 32 features) come in two launch geometries -- two point blocks per
 * wave, or one with twice the waves -- that produce the same bits and differ in speed by a few percent either
 * way, depending on the clock the individual chip holds under them.  The library finds out on the caller's own
 * steps: while a device has no verdict, consecutive hkm_lloyd_step_f32 calls of a large fit on one stream run
 * in three windows (two point blocks, one, two again; about 30 ms of device time each, the last third between
 * two events); once the last event has completed -- looked at, never waited for -- the faster geometry is
 * kept for the device until the process ends.  No extra launch, no wait; HKM_POINT_BLOCKS=1|2 in the
 * environment overrides it.
 * hkm_point_blocks: the point blocks per wave a call with D features would use now (0: D has no resident
 *   kernel); *tuned (if not NULL) tells whether that is the verdict of such a trial on the current device.
 * hkm_point_blocks_trial: the verdict for the current device (0 while there is none) and the time per step,
 *   in milliseconds, of the last window with two point blocks and of the window with one (HOST pointers,
 *   either may be NULL; 0 before the verdict).
 */
int hkm_point_blocks(int32_t D, int32_t* tuned);
int hkm_point_blocks_trial(float* ms_two, float* ms_one);

/* ---- exported by libhkm_bench.so ----------------------------------------------------------------- */

/* Message of the last error a probe raised on the calling thread ("" if none). */
const char* hkm_bench_last_error(void);

/*
 * Microbenchmarks behind the hardware figures the kernels are designed around (bench.py --probe times
 * them).  Each call enqueues ONE kernel; returns 0 or a negative HKM_BENCH_E* code.
 * hkm_probe_mfma_f32: every wave issues iters * 16 fp32 matrix instructions (v_mfma_f32_32x32x2_f32, two
 *   independent accumulators), each followed by `nops` instructions of kind `op`: 0 none (nops = 0),
 *   1 v_fma_f32, 2 v_cndmask_b32, 3 v_min3_f32, 4 s_add_u32 (scalar unit), 5 v_cmp_lt_f32, 6 v_mov_b64;
 *   nops 4 or 8.
 *   grid workgroups of 256 threads; out receives grid * 256 floats.  flops = grid * 4 * iters * 16 * 4096.
 * hkm_probe_stream: mode 0 copies bytes from src to dst, 1 reads src, 2 reads src with non-temporal loads,
 *   3 fills dst; 16-byte vectors, four in flight per thread; sink is one device float.
 */
int hkm_probe_mfma_f32(int32_t op, int32_t nops, int32_t iters, int32_t grid, float* out, void* hip_stream);
int hkm_probe_stream(const void* src, void* dst, size_t bytes, int32_t mode, float* sink, void* hip_stream);

#ifdef __cplusplus
}
#endif

#endif /* HKM_BENCH_H */
