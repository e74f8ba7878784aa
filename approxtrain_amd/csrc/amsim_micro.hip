// Micro-kernels that measure the two machine rates the LUT-multiply GEMM is
// bounded by, on the device they run on:
//   * VALU issue rate  (independent FP32 FMA chains, lane-ops per second);
//   * LDS gather rate  (one data-dependent LDS read per lane, gathers per
//     second) for the access shapes the kernel could use.
// They are what the roofline of the bench is priced against.
#include "amsim_internal.h"

namespace amsim {

constexpr int MICRO_THREADS = 256;
constexpr int MICRO_UNROLL = 16;

// VMODE 0: v_fma_f32   1: v_add_u32   2: v_lshl_add_u32   3: v_mul_f32
//       4: a 4-op mix (add, mul, lshl_add, fma)
//       5: the GEMM's mix per pair of MACs: one v_lshl_add_u64 (VGPR pair + SGPR pair, two LUT
//          addresses), two v_lshl_add_u32 (VGPR << 16 + SGPR), two v_fma_f32 -- 5 ops per two slots
template <int VMODE>
__global__ __launch_bounds__(MICRO_THREADS) void micro_valu_kernel(int iters, float *sink, long long *clk)
{
    float a[MICRO_UNROLL];
#pragma unroll
    for (int j = 0; j < MICRO_UNROLL; ++j) a[j] = (float)(threadIdx.x + j) * 1e-3f;
    float c1 = 0.999f + 1e-6f * threadIdx.x, c2 = 1e-3f;
    const uint64_t pair = ((uint64_t)threadIdx.x << 32) | threadIdx.x;
    const uint64_t spair = ((uint64_t)(uint32_t)iters << 32) | (uint32_t)iters;
    const long long t0 = clock64();
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int j = 0; j < MICRO_UNROLL; ++j) {
            if (VMODE == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(a[j]) : "v"(c1), "v"(c2));
            else if (VMODE == 1) asm volatile("v_add_u32 %0, %0, %1" : "+v"(a[j]) : "v"(c1));
            else if (VMODE == 2) asm volatile("v_lshl_add_u32 %0, %0, 16, %1" : "+v"(a[j]) : "v"(c1));
            else if (VMODE == 3) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(a[j]) : "v"(c1));
            else if (VMODE == 5) {
                if (j & 1) continue;  // slots are handled in pairs
                uint64_t t2;
                uint32_t t0, t1;
                asm volatile("v_lshl_add_u64 %0, %1, 0, %2" : "=v"(t2) : "v"(pair), "s"(spair));
                asm volatile("v_lshl_add_u32 %0, %1, 16, %2" : "=v"(t0) : "v"((uint32_t)t2), "s"(iters));
                asm volatile("v_lshl_add_u32 %0, %1, 16, %2" : "=v"(t1) : "v"((uint32_t)(t2 >> 32)), "s"(iters));
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[j]) : "v"(c2), "v"(t0));
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[j + 1]) : "v"(c2), "v"(t1));
            } else {
                float t, f;
                asm volatile("v_add_u32 %0, %1, %2" : "=v"(t) : "v"(a[j]), "v"(c1));
                asm volatile("v_mul_f32 %0, %1, %2" : "=v"(f) : "v"(c2), "v"(c1));
                asm volatile("v_lshl_add_u32 %0, %1, 16, 1.0" : "=v"(t) : "v"(t));
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[j]) : "v"(t), "v"(f));
            }
        }
    }
    const long long t1 = clock64();
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < MICRO_UNROLL; ++j) s += a[j];
    if (s == 123.456f) sink[threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0 && clk) *clk = t1 - t0;
}

// mode 0: ds_read_u8,  every lane inside one 128-byte row (row differs per read)
// mode 1: ds_read_u8,  lanes scattered over 16 KB
// mode 2: ds_read_u16, every lane inside one 256-byte row
// mode 3: ds_read_u16, lanes scattered over 32 KB
// mode 4: ds_read_b32, every lane inside one 512-byte row
// mode 5: ds_read_b32, lanes scattered over 64 KB
template <int MODE>
__global__ __launch_bounds__(MICRO_THREADS) void micro_lds_kernel(int iters, float *sink)
{
    __shared__ __align__(16) uint32_t lds[16384];  // 64 KB
    for (int i = threadIdx.x; i < 16384; i += MICRO_THREADS) lds[i] = i * 2654435761u;
    __syncthreads();
    constexpr int ESZ = MODE < 2 ? 1 : MODE < 4 ? 2 : 4;
    constexpr bool ROW = (MODE % 2) == 0;
    // per-lane pseudo-random element index
    uint32_t h = (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u);
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    uint32_t addr[MICRO_UNROLL];
#pragma unroll
    for (int j = 0; j < MICRO_UNROLL; ++j) {
        uint32_t r = h * (2 * j + 1) + j * 97u;
        r ^= r >> 11;
        if (ROW) addr[j] = ((r & 127u) + (uint32_t)j * 128u) * ESZ;      // row j, element r%128
        else addr[j] = (r & 16383u) * ESZ;                                // anywhere
    }
    uint32_t acc = 0;
    for (int i = 0; i < iters; ++i) {
        uint32_t v[MICRO_UNROLL];
#pragma unroll
        for (int j = 0; j < MICRO_UNROLL; ++j) {
            if (ESZ == 1) asm volatile("ds_read_u8 %0, %1" : "=v"(v[j]) : "v"(addr[j]));
            else if (ESZ == 2) asm volatile("ds_read_u16 %0, %1" : "=v"(v[j]) : "v"(addr[j]));
            else asm volatile("ds_read_b32 %0, %1" : "=v"(v[j]) : "v"(addr[j]));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        acc ^= v[0] ^ v[MICRO_UNROLL - 1];
    }
    if (acc == 0x12345u) sink[threadIdx.x] = (float)acc;
}

// plain streaming copy: the known-size kernel that hardware traffic counters are scaled against
__global__ __launch_bounds__(MICRO_THREADS) void calibration_copy_kernel(const float4 *src, float4 *dst, size_t n4)
{
    size_t i = (size_t)blockIdx.x * MICRO_THREADS + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * MICRO_THREADS;
    for (; i < n4; i += stride) dst[i] = src[i];
}

}  // namespace amsim

using namespace amsim;

extern "C" {

// Copies n floats (n a multiple of 4, 16-byte aligned buffers) with a plain
// kernel: reads 4n bytes, writes 4n bytes.
int amsim_calibration_copy(const float *src, float *dst, size_t n, void *stream)
{
    if (!src || !dst || (n & 3) || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
        return fail(AMSIM_ERR_INVALID, "calibration copy needs 16-byte aligned buffers and n % 4 == 0");
    if (n == 0) return AMSIM_OK;
    calibration_copy_kernel<<<2048, MICRO_THREADS, 0, static_cast<hipStream_t>(stream)>>>(
        reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst), n / 4);
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

// Runs micro-kernel `kind` (0 = VALU FMA, 1..6 = LDS gather modes 0..5,
// 10..15 = VALU modes 0..5 with `sink[512..]` receiving the shader-clock ticks
// of one workgroup's loop) with
// `blocks` workgroups of 256 threads, `iters` loop trips of 16 operations per
// lane, `reps` launches; returns the mean milliseconds per launch measured
// with HIP events on `stream`, and the operation count of one launch.
int amsim_microbench(int kind, int blocks, int iters, int reps, void *stream_, float *sink, double *ms_per_launch,
                     double *ops_per_launch)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (kind < 0 || (kind > 6 && kind < 10) || kind > 15 || blocks < 1 || iters < 1 || reps < 1 || !sink || !ms_per_launch || !ops_per_launch)
        return fail(AMSIM_ERR_INVALID, "bad microbench arguments");
    hipEvent_t e0, e1;
    AMSIM_HIP_CHECK(hipEventCreate(&e0));
    AMSIM_HIP_CHECK(hipEventCreate(&e1));
    auto launch = [&]() {
        switch (kind) {
        case 0: micro_valu_kernel<0><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, nullptr); break;
        case 10: micro_valu_kernel<0><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 11: micro_valu_kernel<1><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 12: micro_valu_kernel<2><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 13: micro_valu_kernel<3><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 14: micro_valu_kernel<4><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 15: micro_valu_kernel<5><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 1: micro_lds_kernel<0><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        case 2: micro_lds_kernel<1><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        case 3: micro_lds_kernel<2><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        case 4: micro_lds_kernel<3><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        case 5: micro_lds_kernel<4><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        default: micro_lds_kernel<5><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        }
    };
    launch();  // warm-up
    AMSIM_HIP_CHECK(hipEventRecord(e0, stream));
    for (int r = 0; r < reps; ++r) launch();
    AMSIM_HIP_CHECK(hipEventRecord(e1, stream));
    AMSIM_HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    AMSIM_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    AMSIM_HIP_CHECK(hipEventDestroy(e0));
    AMSIM_HIP_CHECK(hipEventDestroy(e1));
    AMSIM_HIP_CHECK(hipGetLastError());
    *ms_per_launch = (double)ms / reps;
    *ops_per_launch = (double)blocks * MICRO_THREADS * (double)iters * MICRO_UNROLL * (kind == 14 ? 4.0 : kind == 15 ? 2.5 : 1.0);
    return AMSIM_OK;
}

}  // extern "C"
