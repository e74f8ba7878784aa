// Filter gradients of small layers: the REDUCTION runs over the lanes.
//
// out(r, j) = sum_k P(x(r, k), dy(k, j)), r = (fy, fx, c) a filter element, k = (b, oy, ox) an output
// pixel, j an output channel (cuda/cuda_kernel.cu:327-353 gathers x(r, k), :417-425 multiplies).  A
// LeNet-sized layer has a few dozen to a few hundred filter elements and a few output channels, but
// 10^4..10^5 pixels: with the filter elements over the lanes (the other engines' layout) most lanes of
// a wavefront are idle and every product pays for a wave-uniform operand.  Here a lane owns PIXELS:
//   * a wavefront takes RB filter elements x JB output channels (RB * JB accumulators per lane) and a
//     slice of the pixels, 64 at a time; a lane loads its pixel's JB gradient values (contiguous) and
//     its RB input values (the window test is per lane, the filter element is wave-uniform), decodes
//     each once, and multiplies all RB x JB pairs;
//   * both operands of a product differ from lane to lane, so the LUT gather address is
//     (mantissa of x << m) + mantissa of dy per lane -- scattered over the table, with the bank
//     conflicts that brings -- and nothing in the inner loop reads a scalar register: address add,
//     gather, byte -> factor, FMA, all on vector registers;
//   * zeros need no test: x = 0 gives a zero power of two; dy = 0 points the gather at a zero-filled
//     copy of the table's extent that follows the table in LDS, so its factor is (+-)0;
//   * at the end the lanes' sums are added by a butterfly of fixed order, and each wavefront writes
//     one plane of partial sums; the fixed-order reduction kernel adds the planes.
// The sums are therefore NOT one ascending chain per output: this kernel only serves calls whose
// reductions may be split (result within 1e-5 * sum|products| of the sequential chain, the same bits
// from run to run), and the other engines keep the whole-reduction mode.
#include "amsim_gemm_common.h"

#include <algorithm>

namespace amsim {

namespace {

constexpr int KL_WAVES = WG_THREADS / 64;
constexpr int KLANES_WAVES_PER_CU = 8;  // two wavefronts per SIMD (four measured 5 % slower: more planes to reduce)

struct KLArgs {
    PDesc p;               // P_GF source
    const float *q;        // dy, element (k, j) at q[k * q_sk + j]
    int64_t q_sk;
    int q_pairs;           // q is 8-byte aligned and q_sk even: channel pairs at even offsets can be read as one
    const uint8_t *lut_img;  // byte image indexed (mantissa of x << m) | mantissa of dy
    int m;
    int64_t R, J, K;
    int rblocks, jblocks;  // tiles of RB filter elements x JB output channels
    int nslices;           // slices of the pixels, kslice (a multiple of 64) each
    int64_t kslice;
    float *partial;        // [nslices][Rp][Jp]
    int Rp, Jp;
};

template <int RB, int JB>
__global__ __launch_bounds__(WG_THREADS) void lutgemm_klanes_kernel(KLArgs a)
{
    // the table, then as many zero bytes: (row of x) + (offset of a zero dy) always lands there
    __shared__ __align__(16) uint8_t lut_s[2 * 16384];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = a.m, mshift = 23 - m;
    const uint32_t table_bytes = 1u << (2 * m);
    for (uint32_t i = tid * 16; i < table_bytes; i += WG_THREADS * 16)
        *reinterpret_cast<uint4 *>(lut_s + i) = *reinterpret_cast<const uint4 *>(a.lut_img + i);  // (m >= 2: whole 16-byte groups)
    for (uint32_t i = tid * 16; i < table_bytes; i += WG_THREADS * 16)
        *reinterpret_cast<uint4 *>(lut_s + table_bytes + i) = make_uint4(0, 0, 0, 0);

    // this wavefront's tile and slice: the wavefronts of a workgroup take different tiles of one slice
    // (they read the same pixels)
    const int ntiles = a.rblocks * a.jblocks;
    const int64_t gw = (int64_t)blockIdx.x * KL_WAVES + wave;
    const int tile = (int)(gw % ntiles);
    const int64_t slice = gw / ntiles;
    const bool wave_live = slice < a.nslices;
    const int r0 = (tile % a.rblocks) * RB, j0 = (tile / a.rblocks) * JB;
    const int64_t kbeg = slice * a.kslice;
    const int64_t kend = kbeg + a.kslice < a.K ? kbeg + a.kslice : a.K;

    // wave-uniform description of the RB filter elements
    int tap_off[RB], tap_fy[RB], tap_fx[RB];
#pragma unroll
    for (int rr = 0; rr < RB; ++rr) {
        const int r = r0 + rr < a.R ? r0 + rr : 0;
        const int c = r % a.p.C, t = r / a.p.C;
        tap_fx[rr] = t % a.p.KW;
        tap_fy[rr] = t / a.p.KW;
        tap_off[rr] = (tap_fy[rr] * a.p.SW + tap_fx[rr]) * a.p.C + c;
    }

    float acc[RB][JB];
#pragma unroll
    for (int rr = 0; rr < RB; ++rr)
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) acc[rr][jj] = 0.0f;

    const bool pairs = a.q_pairs && j0 + JB <= a.J;
    // raw operands of the 64 pixels from k0 on: this lane's pixel is k0 + lane
    // This lane's pixel (b, oy, ox) of pass n is pixel kbeg + 64 n + lane: found by division once,
    // then advanced by 64 pixels per pass with compares (64 = adv_rows * GW + adv_cols; a row step
    // wraps the image at most once when GH > adv_rows + 1, else the division is repeated).
    const int adv_rows = 64 / a.p.GW, adv_cols = 64 % a.p.GW;
    const bool stepwise = a.p.GH > adv_rows + 1;
    int ox, oy, b;
    auto locate = [&](int64_t k) {
        const uint32_t k32 = (uint32_t)k;  // (the reduction is shorter than 2^31)
        ox = (int)(k32 % (uint32_t)a.p.GW);
        const uint32_t t = k32 / (uint32_t)a.p.GW;
        oy = (int)(t % (uint32_t)a.p.GH);
        b = (int)(t / (uint32_t)a.p.GH);
    };
    locate(kbeg + lane);
    auto load = [&](int64_t k0, uint32_t (&xr)[RB], uint32_t (&dr)[JB]) {
        const int64_t k = k0 + lane;
        const bool valid = wave_live && k < kend;
        const int iy0 = oy * a.p.sy - a.p.pt, ix0 = ox * a.p.sx - a.p.pl;
        // (modulo 2^32: lanes past the slice's end carry an image index beyond the batch, whose offset would
        // overflow a signed int; it is never dereferenced, and for valid lanes the wrapped sum is the offset)
        const uint32_t pix = (((uint32_t)b * (uint32_t)a.p.SH + (uint32_t)iy0) * (uint32_t)a.p.SW + (uint32_t)ix0) * (uint32_t)a.p.C;
        const float *qrow = a.q + k * a.q_sk + j0;
        if (JB % 2 == 0 && pairs) {  // whole block inside the row, 8-byte aligned: two channels per load
#pragma unroll
            for (int jj = 0; jj < JB; jj += 2) {
                const uint2 t = valid ? *reinterpret_cast<const uint2 *>(qrow + jj) : make_uint2(0u, 0u);
                dr[jj] = t.x; dr[jj + 1] = t.y;
            }
        } else {
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) dr[jj] = (valid && j0 + jj < a.J) ? f2u(qrow[jj]) : 0u;
        }
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) {
            const bool ok = valid && r0 + rr < a.R && (unsigned)(iy0 + tap_fy[rr]) < (unsigned)a.p.SH &&
                            (unsigned)(ix0 + tap_fx[rr]) < (unsigned)a.p.SW;
            xr[rr] = ok ? f2u(a.p.base[pix + (uint32_t)tap_off[rr]]) : 0u;
        }
        // on to the pixel of the next pass
        if (stepwise) {
            ox += adv_cols;
            const int c1 = ox >= a.p.GW ? 1 : 0;
            ox -= c1 ? a.p.GW : 0;
            oy += adv_rows + c1;
            const int c2 = oy >= a.p.GH ? 1 : 0;
            oy -= c2 ? a.p.GH : 0;
            b += c2;
        } else {
            locate(k + 64);
        }
    };
    auto compute = [&](const uint32_t (&xr)[RB], const uint32_t (&dr)[JB]) {
        SafeRange xrange, drange;
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) xrange.add(xr[rr]);
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) drange.add(dr[jj]);
        // every operand passes the quick test, or (second look) the exponent ranges of this pass's inputs
        // and gradients are such that every product can still take the fast form
        bool fast = !__any((xrange.unsafe() || drange.unsafe()) ? 1 : 0);
        if (!fast) fast = spans_compatible(span_word(wave_union(xrange)), span_word(wave_union(drange)));
        if (fast) {
            uint32_t dcol[JB], dse[JB];
#pragma unroll
            for (int jj = 0; jj < JB; ++jj) {
                dse[jj] = dr[jj] & 0xff800000u;
                dcol[jj] = (dr[jj] & 0x7fffffffu) ? ((dr[jj] & 0x7fffffu) >> mshift) : table_bytes;
            }
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const float xta = u2f(xr[rr] & 0xff800000u);
                const uint32_t xrow = ((xr[rr] & 0x7fffffu) >> mshift) << m;
#pragma unroll
                for (int jj = 0; jj < JB; ++jj) {
                    const uint32_t byte = lut_s[xrow + dcol[jj]];
                    // (LUT byte << 16) + sign|exponent bits of dy  ==  dy_pow2 * 1.mant * 2^carry, exactly
                    acc[rr][jj] = __builtin_fmaf(xta, u2f((byte << 16) + dse[jj]), acc[rr][jj]);
                }
            }
        } else {
            // Rare: an operand outside the fast product's range in some lane: the full-domain product
#pragma unroll
            for (int rr = 0; rr < RB; ++rr) {
                const uint32_t xrow = ((xr[rr] & 0x7fffffu) >> mshift) << m;
#pragma unroll
                for (int jj = 0; jj < JB; ++jj) {
                    const uint32_t e16 = (uint32_t)lut_s[xrow + ((dr[jj] & 0x7fffffu) >> mshift)] << 16;
                    acc[rr][jj] += am_exact(xr[rr], dr[jj], e16);
                }
            }
        }
    };

    uint32_t xc[RB], dc[JB], xn[RB], dn[JB];
    load(kbeg, xc, dc);
    __syncthreads();  // the table has landed
    for (int64_t k0 = kbeg; k0 < kend; k0 += 64) {
        load(k0 + 64, xn, dn);  // past the slice's end: zeros, no access
        compute(xc, dc);
#pragma unroll
        for (int rr = 0; rr < RB; ++rr) xc[rr] = xn[rr];
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) dc[jj] = dn[jj];
    }
    if (!wave_live) return;

    // lanes' sums -> one sum per output, in a fixed order (butterfly over lane distances 32 .. 1),
    // element e = rr * JB + jj ends up in lane e (RB * JB <= 64)
    float mine = 0.0f;
#pragma unroll
    for (int rr = 0; rr < RB; ++rr)
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) {
            float v = acc[rr][jj];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
            if (lane == rr * JB + jj) mine = v;
        }
    if (lane < RB * JB) {
        const int rr = lane / JB, jj = lane % JB;
        if (r0 + rr < a.Rp && j0 + jj < a.Jp) a.partial[((size_t)slice * a.Rp + r0 + rr) * a.Jp + j0 + jj] = mine;
    }
}

struct KLPlan {
    int RB, JB, rblocks, jblocks, nslices, Rp, Jp;
    int64_t kslice;
    size_t partial_bytes;
};

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Block shapes on offer (RB * JB <= 64): the one with the least padding wins, larger blocks first
// among equals (more products per loaded operand).
KLPlan plan_klanes(int64_t R, int64_t J, int64_t K, int cus)
{
    KLPlan best{};
    int64_t best_cost = -1;
    for (int RB : {8, 7, 6, 5})
        for (int JB : {8, 6, 4}) {
            const int64_t rb = (R + RB - 1) / RB, jb = (J + JB - 1) / JB;
            // padded products, + the per-pixel operand work (loads, decode) that larger blocks amortise
            const int64_t cost = rb * jb * (RB * JB * 3 + (RB + JB) * 6);
            if (best_cost < 0 || cost < best_cost) {
                best_cost = cost;
                best.RB = RB; best.JB = JB; best.rblocks = (int)rb; best.jblocks = (int)jb;
            }
        }
    const int64_t ntiles = (int64_t)best.rblocks * best.jblocks;
    // about two wavefronts per SIMD, each with at least two passes of 64 pixels
    int64_t nslices = std::max<int64_t>(1, ((int64_t)cus * KLANES_WAVES_PER_CU + ntiles - 1) / ntiles);
    nslices = std::min<int64_t>(nslices, std::max<int64_t>(1, K / 128));
    best.kslice = ((K + nslices - 1) / nslices + 63) / 64 * 64;
    best.nslices = (int)((K + best.kslice - 1) / best.kslice);
    best.Rp = best.rblocks * best.RB;
    best.Jp = best.jblocks * best.JB;
    best.partial_bytes = align256((size_t)best.nslices * best.Rp * best.Jp * sizeof(float));
    return best;
}

template <int RB>
void launch_klanes_rb(const KLArgs &a, int JB, dim3 grid, hipStream_t stream)
{
    switch (JB) {
    case 8: lutgemm_klanes_kernel<RB, 8><<<grid, WG_THREADS, 0, stream>>>(a); break;
    case 6: lutgemm_klanes_kernel<RB, 6><<<grid, WG_THREADS, 0, stream>>>(a); break;
    default: lutgemm_klanes_kernel<RB, 4><<<grid, WG_THREADS, 0, stream>>>(a); break;
    }
}

}  // namespace

// Filter-gradient problems (rows gathered per filter element, gradient matrix row-major) with so few
// filter elements that a wavefront with one per lane would be at least half idle, and a long
// reduction; tables that fit the LDS, one batch item, input small enough for 32-bit element offsets.
// (With more filter elements the rows-over-lanes engines win: their gathers stay inside one table row
// and run conflict-free at about 3.4x the rate of this kernel's scattered ones -- LeNet-5's second
// convolution, 150 filter elements x 16 channels, takes 31 us there and 39 us here.)
bool klanes_shape_eligible(int64_t R, int64_t J, int64_t K, int batch)
{
    return batch == 1 && R <= KLANES_MAX_ROWS && R * J <= KLANES_MAX_OUTPUTS && K >= KLANES_MIN_REDUCTION && K < (1ll << 31);
}

bool klanes_eligible(int m, const GemmDesc &d)
{
    if (m < 2 || m > 7 || d.p.kind != P_GF || d.q.kind != Q_DENSE || d.q.sj != 1 || d.q.batches != 1) return false;
    if (!klanes_shape_eligible(d.R, d.J, d.K, d.batch)) return false;
    return (int64_t)d.p.B * d.p.SH * d.p.SW * d.p.C < (1ll << 31);
}

size_t klanes_workspace_bytes(int64_t R, int64_t J, int64_t K)
{
    size_t need = 0;
    for (int cus : {device_compute_units(), 256, 304}) need = std::max(need, plan_klanes(R, J, K, cus).partial_bytes);
    return need;
}

int run_gemm_klanes(const Lut &lut, const GemmDesc &d, void *workspace, size_t workspace_bytes, hipStream_t stream)
{
    const KLPlan pl = plan_klanes(d.R, d.J, d.K, device_compute_units());
    if (workspace == nullptr || ((uintptr_t)workspace & 255) || workspace_bytes < pl.partial_bytes)
        return fail(AMSIM_ERR_WORKSPACE, "workspace too small for the partial sums");
    KLArgs a{};
    a.p = d.p;
    a.q = d.q.base; a.q_sk = d.q.sk;
    a.q_pairs = (d.q.sk % 2 == 0 && ((uintptr_t)d.q.base & 7) == 0 && pl.JB % 2 == 0) ? 1 : 0;
    a.lut_img = d.lane_first ? lut.img_ab : lut.img_ba;  // row by the mantissa of x: x is the product's first operand iff lane_first
    a.m = lut.m;
    a.R = d.R; a.J = d.J; a.K = d.K;
    a.rblocks = pl.rblocks; a.jblocks = pl.jblocks;
    a.nslices = pl.nslices; a.kslice = pl.kslice;
    a.partial = static_cast<float *>(workspace);
    a.Rp = pl.Rp; a.Jp = pl.Jp;
    const int64_t waves = (int64_t)pl.rblocks * pl.jblocks * pl.nslices;
    const dim3 grid((unsigned)((waves + KL_WAVES - 1) / KL_WAVES));
    switch (pl.RB) {
    case 8: launch_klanes_rb<8>(a, pl.JB, grid, stream); break;
    case 7: launch_klanes_rb<7>(a, pl.JB, grid, stream); break;
    case 6: launch_klanes_rb<6>(a, pl.JB, grid, stream); break;
    default: launch_klanes_rb<5>(a, pl.JB, grid, stream); break;
    }
    AMSIM_HIP_CHECK(hipGetLastError());
    RArgs ra{a.partial, d.out, d.R, d.J, pl.Rp, d.so_r, d.so_j, d.out_batch_stride, pl.Jp, pl.nslices, 1, 0,
             Epilogue{d.bias_j, d.bias_r, d.act, d.omap}};
    launch_reduce(ra, stream);
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

}  // namespace amsim
