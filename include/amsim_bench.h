/*
 * amsim_bench.h -- measurement and tuning helpers of libamsim.so.
 *
 * Not part of the drop-in boundary: nothing here replaces a functor or kernel of the reference
 * and no op kernel calls it.  The benchmark driver, the profiler runs and a few tests use these
 * entry points to measure the machine rates the GEMM kernels are priced against and to look at
 * the planner's decisions.  The product ABI is include/amsim.h.
 */
#ifndef AMSIM_BENCH_H_
#define AMSIM_BENCH_H_

#include "amsim.h"

#ifdef __cplusplus
extern "C" {
#endif

/* How a GEMM of this shape would be run when reductions may be split (contiguous, aligned
 * operands assumed): info = {outputs per lane, row tiles per workgroup, splits of the main part's
 * reduction, chunks (of 32) per split, rows in the main part, splits of the tail rows' reduction
 * (0 = no tail), chunks per tail split, chunks in all}.  For tests and tuning. */
int amsim_gemm_plan_info(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t batch, int64_t info[8]);
/* Test hook.  The LDS-table GEMM gathers table bytes into the upper half of a register whose lower
 * half must read as zero; whether a 16-bit LDS load keeps or clears the half it does not write
 * differs between devices and is probed once per device when a handle is created.  Where it is
 * kept, the kernel zeroes those registers once per reduction chunk.  on = 1 makes calls through
 * this handle take that branch whatever the probe said (results must not change), on = 0 restores
 * the probe's answer; *probed (may be NULL) receives the probe's answer: 1 = kept, 0 = cleared. */
int amsim_lut_force_gather_zeroing(amsim_lut_t lut, int on, int *probed);
/* Micro-kernels that measure, on the current device, the VALU issue rate
 * (kind 0 / 10: independent FP32 FMAs; 11..13: v_add_u32, v_lshl_add_u32,
 * v_mul_f32; 14: a 4-op mix; 15: the GEMM inner loop's earlier mix, 5 instructions per two MACs;
 * 16: the row-staged GEMM's pair per product, a 16-bit multiply-add that forms the factor + an FMA;
 * 17: the GEMM inner loop's mix, 4 instructions per two MACs: two 64-bit adds of a scalar pair, two FMAs) and
 * the LDS gather rate (kinds 1..6: u8 / u16 / b32 reads, lanes inside one
 * 128-element row or scattered, with 64 KB of LDS per workgroup; kinds 21 / 22: the u8 pair
 * again at the GEMM kernel's own LDS footprint and occupancy, reads software-pipelined).
 * Kinds 10..17 also leave two 64-bit counts at sink[512..515]: the shader-clock ticks of one
 * workgroup's loop and the same interval in 100 MHz ticks (their ratio is the clock).  Launches
 * `reps` times on `stream`, timed with HIP events; `sink` is any device buffer
 * of >= 256 floats. */
int amsim_microbench(int kind, int blocks, int iters, int reps, void *stream, float *sink,
                     double *ms_per_launch, double *ops_per_launch);
/* The rates that bound products through tables too wide for the LDS (mantissa widths 8..11,
 * rows of 4 KB in device memory): kind 0 = one 2-byte global gather per product, all lanes of a
 * wavefront inside one random row; 1 = whole random rows pulled into LDS by direct
 * global-to-LDS loads (bytes); 2 = 16-bit LDS gathers with the lanes scattered over 4 KB rows;
 * 3 = 1 and 2 overlapped (64 KB of rows per 65536 products: the shape of a row-staged GEMM that
 * keeps the rows apart in LDS); 4 = 16-byte LDS reads with the lanes scattered over a 32 KB
 * half of interleaved rows, 8 products per read (the row-staged GEMM's gathers); 5 = whole random
 * rows pulled into registers by coalesced 4-byte loads (bytes; the GEMM's own fetches).  `table`
 * is a device buffer of table_bytes >= 8 KB, 16-byte aligned; workgroups have 1024 threads;
 * ops_per_launch counts products (bytes for kinds 1 and 5). */
int amsim_microbench_wide(int kind, int blocks, int iters, int reps, void *stream, const void *table,
                          size_t table_bytes, float *sink, double *ms_per_launch, double *ops_per_launch);

/* Plain copy kernel of known size (reads 4n bytes, writes 4n bytes; n % 4 == 0,
 * 16-byte aligned buffers): the reference point that hardware traffic counters
 * (FETCH_SIZE / WRITE_SIZE) are scaled against. */
int amsim_calibration_copy(const float *src, float *dst, size_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* AMSIM_BENCH_H_ */
