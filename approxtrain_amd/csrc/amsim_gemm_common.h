// Pieces shared by the LUT-multiply GEMM kernels (the LDS-table engine and the row-staged engine
// for tables too wide for the LDS): tile constants, the pre-decoded uniform operand, the output
// epilogue.
#ifndef AMSIM_GEMM_COMMON_H_
#define AMSIM_GEMM_COMMON_H_

#include "amsim_internal.h"
#include "amsim_device.h"

namespace amsim {

constexpr int KC = 32;        // reduction depth of one staged chunk
constexpr int KG = 4;         // reduction rows handled per scalar-load batch
constexpr int NG = KC / KG;
constexpr int QT = 16;        // columns per tile of the pre-decoded uniform operand
constexpr int WG_THREADS = 256;
constexpr int LUT_LDS_BYTES = 16384 + 128;   // 2^(2m) entries + one all-zero row of 2^m entries (m <= 7)
constexpr int WAVES_PER_SIMD = 6;             // occupancy the 64-row kernels are compiled for
constexpr int NUM_XCD = 8;                    // accelerator dies, each with a private L2
constexpr double MACS_PER_CU_S = 15.0e12 / 256;  // planner's price of a MAC: what one compute unit sustains
constexpr double PARTIAL_BYTES_PER_S = 3.0e12;   // planner's price of writing + re-reading partial sums
constexpr double WORKGROUP_START_S = 3.5e-6;     // planner's price of a round of workgroup starts (LUT staging, first loads)


typedef const __attribute__((address_space(4))) uint32_t *cq1_t;
typedef const __attribute__((address_space(4))) uint64_t *cq2_t;


// Output epilogue shared by the main kernel and the split reduction: bias add, then
// the activation.  ReLU keeps NaN and the sign of a negative zero (x < 0 ? 0 : x).
struct Epilogue {
    const float *bias_j, *bias_r;
    int act;
    OutMap omap;
};
// element offset of output row r (before the column term)
__device__ __forceinline__ int64_t out_row_offset(const OutMap &m, int64_t r, int64_t so_r)
{
    if (!m.enabled) return r * so_r;
    // (mapped outputs have fewer than 2^31 rows: 32-bit divisions)
    const uint32_t r32 = (uint32_t)r;
    const int x = (int)(r32 % (uint32_t)m.GW);
    const uint32_t t = r32 / (uint32_t)m.GW;
    const int y = (int)(t % (uint32_t)m.GH);
    const int64_t b = t / (uint32_t)m.GH;
    return ((b * m.H + (y * m.sy + m.oy)) * m.W + (x * m.sx + m.ox)) * so_r;
}
__device__ __forceinline__ float apply_epilogue(const Epilogue &e, float v, int64_t r, int64_t j)
{
    if (e.bias_j) v += e.bias_j[j];
    if (e.bias_r) v += e.bias_r[r];
    if (e.act == AMSIM_ACT_RELU) v = v < 0.0f ? 0.0f : v;
    return v;
}


struct QArgs {
    QDesc q;
    int64_t K, J;
    int Jp, nchunks, m;
    uint32_t *qw;
    uint32_t *qflags;
    QDesc *qdesc_out;
};

// raw bits of uniform-operand element (k, j) of batch item `base`; zero outside K x J
// (k < 2^31 and j < 2^24 on every path that gets here)
template <typename QD>
__device__ __forceinline__ uint32_t q_raw_bits(const QD &q, const float *base, uint32_t K, uint32_t J, uint32_t k, uint32_t j)
{
    if (k >= K || j >= J) return 0u;
    if (q.kind == Q_DENSE) return f2u(base[(int64_t)k * q.sk + (int64_t)j * q.sj]);
    const uint32_t oc = k % (uint32_t)q.OC, t = k / (uint32_t)q.OC;
    const int fx = q.fx0 + (int)(t % (uint32_t)q.TW) * q.fsx, fy = q.fy0 + (int)(t / (uint32_t)q.TW) * q.fsy;
    return f2u(base[(((int64_t)(q.KH - 1 - fy) * q.KW + (q.KW - 1 - fx)) * q.IC + j) * q.OC + oc]);
}


// sums the split partials in ascending split order (deterministic)
struct RArgs {
    const float *partial;
    float *out;
    int64_t R, J, Rp, so_r, so_j, out_batch_stride;  // R rows starting at row_base
    int Jp, nsplit, batch;
    int64_t row_base;
    Epilogue ep;
};

void launch_reduce(const RArgs &ra, hipStream_t stream);

// raw bits of lane-operand element (r, k) of batch item `base`, whatever the source addressing
// (dense; im2col-style patch, cuda/cuda_kernel.cu:35-60; filter-gradient gather, :327-353);
// zero outside R x K and outside the image.  Element by element with divisions: for passes that
// touch every element once, not for inner loops.
__device__ __forceinline__ uint32_t p_raw_bits(const PDesc &p, const float *base, int64_t R, int64_t K, int64_t r, int64_t k)
{
    if (r >= R || k >= K) return 0u;
    if (p.kind == P_DENSE) return f2u(base[r * p.sr + k * p.sk]);
    int b, y, x, fy, fx, c;
    // (R and K are below 2^31 on every path that gathers: 32-bit divisions)
    const uint32_t r32 = (uint32_t)r, k32 = (uint32_t)k, gw = (uint32_t)p.GW, gh = (uint32_t)p.GH, ch = (uint32_t)p.C;
    if (p.kind == P_PATCH) {
        x = (int)(r32 % gw); const uint32_t t = r32 / gw; y = (int)(t % gh); b = (int)(t / gh);
        c = (int)(k32 % ch); const int u = (int)(k32 / ch); fx = u % p.KW; fy = u / p.KW;
    } else {
        c = (int)(r32 % ch); const int u = (int)(r32 / ch); fx = u % p.KW; fy = u / p.KW;
        x = (int)(k32 % gw); const uint32_t t = k32 / gw; y = (int)(t % gh); b = (int)(t / gh);
    }
    const int iy = y * p.sy - p.pt + fy, ix = x * p.sx - p.pl + fx;
    if ((unsigned)iy >= (unsigned)p.SH || (unsigned)ix >= (unsigned)p.SW) return 0u;
    return f2u(base[(((int64_t)b * p.SH + iy) * p.SW + ix) * p.C + c]);
}

// Decodes the uniform operand into the workspace (qw, qflags) and leaves a copy of its
// descriptor in device memory (defined with the LDS-table engine).
int launch_q_prepass(const QArgs &qa, int q_batches, hipStream_t stream);

}  // namespace amsim
#endif
