// Micro-kernels that measure the two machine rates the LUT-multiply GEMM is
// bounded by, on the device they run on:
//   * VALU issue rate  (independent FP32 FMA chains, lane-ops per second);
//   * LDS gather rate  (one data-dependent LDS read per lane, gathers per
//     second) for the access shapes the kernel could use.
// They are what the roofline of the bench is priced against.
#include "amsim_internal.h"
#include "amsim_bench.h"

#include <algorithm>

namespace amsim {

constexpr int MICRO_THREADS = 256;
constexpr int MICRO_UNROLL = 16;

// VMODE 0: v_fma_f32   1: v_add_u32   2: v_lshl_add_u32   3: v_mul_f32
//       4: a 4-op mix (add, mul, lshl_add, fma)
//       5: the GEMM's mix per pair of MACs: one v_lshl_add_u64 (VGPR pair + SGPR pair, two LUT
//          addresses), two v_lshl_add_u32 (VGPR << 16 + SGPR), two v_fma_f32 -- 5 ops per two slots
//       6: the row-staged GEMM's pair per product: v_mad_u32_u16 (16-bit half * 256 + SGPR) feeding a
//          v_fma_f32 two instructions later -- 2 ops per slot
//       7: the GEMM's mix per pair of MACs when the gathers deliver the byte already shifted: two
//          v_lshl_add_u64 (VGPR pair + SGPR pair: two LUT addresses, two product factors), two
//          v_fma_f32, alternating -- 2 ops per slot
template <int VMODE>
__global__ __launch_bounds__(MICRO_THREADS) void micro_valu_kernel(int iters, float *sink, long long *clk)
{
    float a[MICRO_UNROLL];
#pragma unroll
    for (int j = 0; j < MICRO_UNROLL; ++j) a[j] = (float)(threadIdx.x + j) * 1e-3f;
    float c1 = 0.999f + 1e-6f * threadIdx.x, c2 = 1e-3f;
    const uint64_t pair = ((uint64_t)threadIdx.x << 32) | threadIdx.x;
    const uint64_t spair = ((uint64_t)(uint32_t)iters << 32) | (uint32_t)iters;
    const long long w0 = wall_clock64();
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
            } else if (VMODE == 7) {
                if (j & 1) continue;
                uint64_t t2, u2;
                asm volatile("v_lshl_add_u64 %0, %1, 0, %2" : "=v"(t2) : "v"(pair), "s"(spair));
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[j]) : "v"(c2), "v"((uint32_t)t2));
                asm volatile("v_lshl_add_u64 %0, %1, 0, %2" : "=v"(u2) : "v"(t2), "s"(spair));
                asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(a[j + 1]) : "v"(c2), "v"((uint32_t)(u2 >> 32)));
            } else if (VMODE == 6) {
                if (j & 1) continue;
                uint32_t t0, t1;
                asm volatile("v_mad_u32_u16 %0, %2, %3, %4\n\t"
                             "v_mad_u32_u16 %1, %2, %3, %4 op_sel:[1,0,0,0]"
                             : "=&v"(t0), "=&v"(t1) : "v"((uint32_t)pair), "v"(c1), "s"(iters));
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
    const long long w1 = wall_clock64();
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < MICRO_UNROLL; ++j) s += a[j];
    if (s == 123.456f) sink[threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0 && clk) {
        clk[0] = t1 - t0;    // shader-clock ticks of the loop (s_memtime)
        clk[1] = w1 - w0;    // the same interval on the constant-rate 100 MHz counter (s_memrealtime)
    }
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

// The same gathers with the LUT GEMM's own footprint: 16.5 KB of LDS per workgroup, six
// wavefronts per SIMD, and the reads software-pipelined in two halves so that eight stay in
// flight while the other eight are consumed (the loop never drains the LDS queue).
//   mode 0: ds_read_u8, lanes inside one 128-byte row     mode 1: ds_read_u8, lanes scattered over 16 KB
template <int MODE>
__global__ __launch_bounds__(MICRO_THREADS, 6) void micro_lds_fit_kernel(int iters, float *sink)
{
    __shared__ __align__(16) uint32_t lds[16384 / 4 + 32];
    for (int i = threadIdx.x; i < 16384 / 4 + 32; i += MICRO_THREADS) lds[i] = i * 2654435761u;
    __syncthreads();
    uint32_t h = (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u);
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    uint32_t addr[MICRO_UNROLL];
#pragma unroll
    for (int j = 0; j < MICRO_UNROLL; ++j) {
        uint32_t r = h * (2 * j + 1) + j * 97u;
        r ^= r >> 11;
        addr[j] = MODE == 0 ? (r & 127u) + (uint32_t)j * 128u * 8u : (r & 16383u);
    }
    constexpr int H = MICRO_UNROLL / 2;
    uint32_t acc = 0, va[H], vb[H];
#pragma unroll
    for (int j = 0; j < H; ++j) asm volatile("ds_read_u8 %0, %1" : "=v"(vb[j]) : "v"(addr[H + j]));
    for (int i = 0; i < iters; ++i) {
#pragma unroll
        for (int j = 0; j < H; ++j) asm volatile("ds_read_u8 %0, %1" : "=v"(va[j]) : "v"(addr[j]));
        asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");  // the older half has landed
        acc ^= vb[0] ^ vb[H - 1];
#pragma unroll
        for (int j = 0; j < H; ++j) asm volatile("ds_read_u8 %0, %1" : "=v"(vb[j]) : "v"(addr[H + j]));
        asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
        acc ^= va[0] ^ va[H - 1];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    acc ^= vb[0];
    if (acc == 0x12345u) sink[threadIdx.x] = (float)acc;
}

// ---------------------------------------------------------------------------
// Rates that bound the product with tables too wide for the LDS (mantissa widths 8..11:
// 2^m rows of 2^m 16-bit entries in device memory, 4 KB per row at m = 11).  In the GEMM all
// lanes of a wavefront share the row (the uniform operand's mantissa) and differ in the entry.
//   WMODE 0: one 2-byte global load per lane and product, all lanes inside one random row
//            (every product is its own gather through L1 / L2 / MALL)
//   WMODE 1: whole random rows copied into LDS by direct global-to-LDS loads, nothing else
//            (bytes per second a compute unit can pull rows in with)
//   WMODE 2: ds_read_u16 with the lanes scattered over a 4 KB row held in LDS, 16 rows
//   WMODE 3: both together, the shape of the row-staged GEMM: per stage a 1024-thread workgroup
//            pulls 16 rows (64 KB) into one half of its LDS while every thread gathers 64
//            entries from the other half and feeds them to the convert + FMA pair
//   WMODE 4: ds_read_b128 with the lanes scattered over the 2048 16-byte groups of a 32 KB half (the
//            interleaved layout: one read brings the entries of 8 rows); counts 8 products per read
//   WMODE 5: rows pulled into registers by coalesced 4-byte loads (16 per thread and stage, buffer
//            addressing), nothing else: the bytes per second the register path brings in
// ---------------------------------------------------------------------------
constexpr int WIDE_THREADS = 1024;
constexpr int WIDE_ROW_BYTES = 4096;
constexpr int WIDE_ROWS = 16;

__device__ __forceinline__ uint32_t mix32(uint32_t x)
{
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

template <int WMODE>
__global__ __launch_bounds__(WIDE_THREADS) void micro_wide_kernel(const uint8_t *table, uint32_t table_rows, int iters, float *sink)
{
    extern __shared__ __align__(16) uint8_t wl[];  // 2 x 16 rows x 4 KB
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane_off = (mix32(tid * 2654435761u + blockIdx.x) & 2047u) * 2u;  // this lane's entry inside a row
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const float ta = 1.0f + 1e-3f * lane;
    auto fill = [&](int it, int buf) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int slot = r * 4 + (wave >> 2), part = wave & 3;
            const uint32_t row = mix32((uint32_t)it * 977u + blockIdx.x * 131u + slot) % table_rows;
#if defined(__HIP_DEVICE_COMPILE__)
            __builtin_amdgcn_global_load_lds(table + (size_t)row * WIDE_ROW_BYTES + part * 1024 + lane * 16,
                                             wl + buf * (WIDE_ROWS * WIDE_ROW_BYTES) + slot * WIDE_ROW_BYTES + part * 1024, 16, 0, 0);
#endif
        }
    };
    auto gather = [&](int buf, uint32_t salt) {
        const uint8_t *base = wl + buf * (WIDE_ROWS * WIDE_ROW_BYTES);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const uint32_t off = (lane_off + rr * 74u + salt) & 4094u;
#pragma unroll
            for (int j = 0; j < WIDE_ROWS; ++j) {
                const uint32_t e = *reinterpret_cast<const uint16_t *>(base + j * WIDE_ROW_BYTES + off);
                acc[rr] = __builtin_fmaf(ta, __uint_as_float((e << 8) + 0x3f000000u), acc[rr]);
            }
        }
    };
    if (WMODE == 0) {
        for (int it = 0; it < iters; ++it) {
            uint32_t e[WIDE_ROWS];
#pragma unroll
            for (int j = 0; j < WIDE_ROWS; ++j) {
                const uint32_t row = mix32((uint32_t)it * 977u + (blockIdx.x * 16u + wave) * 131u + j) % table_rows;
                e[j] = *reinterpret_cast<const uint16_t *>(table + (size_t)row * WIDE_ROW_BYTES + lane_off);
            }
#pragma unroll
            for (int j = 0; j < WIDE_ROWS; ++j) acc[j & 3] = __builtin_fmaf(ta, __uint_as_float((e[j] << 8) + 0x3f000000u), acc[j & 3]);
        }
    } else if (WMODE == 1) {
        for (int it = 0; it < iters; ++it) {
            fill(it, it & 1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
        acc[0] = (float)wl[tid * 16];
    } else if (WMODE == 2) {
        for (int i = tid; i < 2 * WIDE_ROWS * WIDE_ROW_BYTES / 4; i += WIDE_THREADS) reinterpret_cast<uint32_t *>(wl)[i] = mix32(i) & 0x7fff7fffu;
        __syncthreads();
        for (int it = 0; it < iters; ++it) gather(it & 1, (uint32_t)it * 2u);
    } else if (WMODE == 4) {
        for (int i = tid; i < 2 * WIDE_ROWS * WIDE_ROW_BYTES / 4; i += WIDE_THREADS) reinterpret_cast<uint32_t *>(wl)[i] = mix32(i);
        __syncthreads();
        uint32_t x = 0;
        for (int it = 0; it < iters; ++it) {
            const uint8_t *base = wl + (it & 1) * 32768;
#pragma unroll
            for (int rr = 0; rr < 8; ++rr) {
                const uint32_t off = (mix32(lane_off + rr * 7919u + (uint32_t)it) & 2047u) * 16u;
                const uint4 e = *reinterpret_cast<const uint4 *>(base + off);
                x ^= e.x ^ e.y ^ e.z ^ e.w;
            }
        }
        if (x == 0x12345u) sink[tid & 255] = 1.0f;  // (an integer-valued float could never equal the sentinel below)
    } else if (WMODE == 5) {
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(table), 0, -1, 0x00020000);
        uint32_t x = 0, va[WIDE_ROWS], vb[WIDE_ROWS];
        auto pull = [&](int it, uint32_t (&v)[WIDE_ROWS]) {
#pragma unroll
            for (int j = 0; j < WIDE_ROWS; ++j) {
                const uint32_t row = mix32((uint32_t)it * 977u + blockIdx.x * 131u + j) % table_rows;
                v[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rs, tid * 4, (int)(row * WIDE_ROW_BYTES), 0);
            }
        };
        pull(0, va);
        for (int it = 0; it < iters; it += 2) {  // one stage's loads are in flight while the stage before is consumed
            pull(it + 1, vb);
#pragma unroll
            for (int j = 0; j < WIDE_ROWS; ++j) x ^= va[j];
            pull(it + 2, va);
#pragma unroll
            for (int j = 0; j < WIDE_ROWS; ++j) x ^= vb[j];
        }
        if (x == 0x12345u) sink[tid & 255] = 1.0f;  // (an integer-valued float could never equal the sentinel below)
    } else {
        fill(0, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        for (int it = 0; it < iters; ++it) {
            fill(it + 1, (it + 1) & 1);
            gather(it & 1, (uint32_t)it * 2u);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }
    const float s = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    if (s == 123.456f) sink[tid & 255] = s;
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
// 10..16 = VALU modes 0..6 with `sink[512..]` receiving, as two 64-bit counts, the
// shader-clock ticks of one workgroup's loop and the same interval in 100 MHz ticks,
// 21 / 22 = byte gathers inside a row / scattered at the LUT GEMM's own LDS footprint and
// occupancy) with
// `blocks` workgroups of 256 threads, `iters` loop trips of 16 operations per
// lane, `reps` launches; returns the mean milliseconds per launch measured
// with HIP events on `stream`, and the operation count of one launch.
int amsim_microbench(int kind, int blocks, int iters, int reps, void *stream_, float *sink, double *ms_per_launch,
                     double *ops_per_launch)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (kind < 0 || (kind > 6 && kind < 10) || (kind > 17 && kind < 21) || kind > 22 || blocks < 1 || iters < 1 || reps < 1 || !sink || !ms_per_launch || !ops_per_launch)
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
        case 16: micro_valu_kernel<6><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 17: micro_valu_kernel<7><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink, (long long *)(sink + 512)); break;
        case 21: micro_lds_fit_kernel<0><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
        case 22: micro_lds_fit_kernel<1><<<blocks, MICRO_THREADS, 0, stream>>>(iters, sink); break;
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
    *ops_per_launch = (double)blocks * MICRO_THREADS * (double)iters * MICRO_UNROLL * (kind == 14 ? 4.0 : kind == 15 ? 2.5 : (kind == 16 || kind == 17) ? 2.0 : 1.0);
    return AMSIM_OK;
}


// Micro-kernels for tables too wide for the LDS (kinds 0..5 = WMODE above).  `table` is any
// device buffer of table_bytes >= 8 KB (rows of 4 KB are read from it), `blocks` workgroups of
// 1024 threads (kind 0: 16 wavefronts each), `iters` stages of 16 rows.  ops_per_launch counts
// products (kinds 0, 2, 3, 4) or bytes pulled in (kinds 1, 5; kind 3 pulls 1 byte per product).
int amsim_microbench_wide(int kind, int blocks, int iters, int reps, void *stream_, const void *table, size_t table_bytes,
                          float *sink, double *ms_per_launch, double *ops_per_launch)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (kind < 0 || kind > 5 || blocks < 1 || iters < 1 || reps < 1 || !table || table_bytes < 2 * WIDE_ROW_BYTES ||
        ((uintptr_t)table & 15) || !sink || !ms_per_launch || !ops_per_launch)
        return fail(AMSIM_ERR_INVALID, "bad microbench arguments");
    const uint32_t rows = (uint32_t)std::min<size_t>(table_bytes / WIDE_ROW_BYTES, 1u << 20);
    const uint8_t *t = static_cast<const uint8_t *>(table);
    const size_t lds = 2 * WIDE_ROWS * WIDE_ROW_BYTES;
    AMSIM_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(micro_wide_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    AMSIM_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(micro_wide_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    AMSIM_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(micro_wide_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    AMSIM_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(micro_wide_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    AMSIM_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(micro_wide_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    auto launch = [&]() {
        switch (kind) {
        case 0: micro_wide_kernel<0><<<blocks, WIDE_THREADS, 0, stream>>>(t, rows, iters, sink); break;
        case 1: micro_wide_kernel<1><<<blocks, WIDE_THREADS, lds, stream>>>(t, rows, iters, sink); break;
        case 2: micro_wide_kernel<2><<<blocks, WIDE_THREADS, lds, stream>>>(t, rows, iters, sink); break;
        case 4: micro_wide_kernel<4><<<blocks, WIDE_THREADS, lds, stream>>>(t, rows, iters, sink); break;
        case 5: micro_wide_kernel<5><<<blocks, WIDE_THREADS, 0, stream>>>(t, rows, iters, sink); break;
        default: micro_wide_kernel<3><<<blocks, WIDE_THREADS, lds, stream>>>(t, rows, iters, sink); break;
        }
    };
    hipEvent_t e0, e1;
    AMSIM_HIP_CHECK(hipEventCreate(&e0));
    AMSIM_HIP_CHECK(hipEventCreate(&e1));
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
    const double per_stage = kind == 0   ? (double)WIDE_THREADS * WIDE_ROWS
                             : kind == 1 ? (double)WIDE_ROWS * WIDE_ROW_BYTES
                             : kind == 4 ? (double)WIDE_THREADS * 8 * 8
                             : kind == 5 ? (double)WIDE_THREADS * WIDE_ROWS * 4
                                         : (double)WIDE_THREADS * 4 * WIDE_ROWS;
    *ops_per_launch = (double)blocks * iters * per_stage;
    return AMSIM_OK;
}

}  // extern "C"
