// Direct LUT-multiply GEMM for small problems (LeNet-sized layers, narrow outputs): ONE launch,
// no workspace pass over either operand.
//
// out(r, j) = sum_k P(p(r, k), q(k, j)) with the same product, accumulation order and operand roles
// as the LDS-table engine (cuda/gemm.cu:17-58 is the loop nest both restate), but built for latency
// instead of throughput:
//   * a wavefront owns 64 rows (one per lane) x TN columns and walks its slice of the reduction
//     alone; each lane loads its own operands straight from where they lie (dense, im2col-style
//     patch or filter-gradient addressing, cuda/cuda_kernel.cu:35-60, 327-353, 463-502) -- no LDS
//     staging, no barrier in the loop;
//   * the uniform operand is decoded inside the kernel, 64 elements at a time: lane l fetches and
//     decodes element (k0 + l / TN, j0 + l % TN), and the products read each decoded word back as a
//     scalar with v_readlane -- so there is no pre-pass launch;
//   * the reduction can be split over the wavefronts of a workgroup (partial sums combined through
//     LDS in a fixed order) and, for few outputs with a long reduction, over workgroups (partials
//     in the workspace, summed by the fixed-order reduction kernel);
//   * the byte-wide LUT image sits in LDS as in the main engine (all lanes of a gather inside one
//     row: conflict-free).
// Per product: one v_readlane, the address add, the byte -> factor step and the FMA -- about half
// the main engine's rate per instruction slot, which is irrelevant where launches and latencies
// dominate: LeNet-sized layers (30-60 MMAC) run 15-50 % faster here than as pre-pass + main + reduction,
// filter gradients of such layers (few outputs, long reduction) up to 2x.
#include "amsim_gemm_common.h"

#include <algorithm>
#include <cmath>

namespace amsim {


namespace {

constexpr int DIRECT_WAVES = WG_THREADS / 64;
// Reduction steps a wavefront handles per loop iteration (all their loads in flight together).  A
// lone wavefront issues an instruction about every 8 cycles, so an iteration of 16 steps x 16
// columns takes 5 us: 16-column tiles use 8 steps so that short reductions can be cut finer.
constexpr int steps_per_iteration(int tn) { return tn >= 16 ? 8 : 16; }
// ... and per decode of the uniform operand (one element per lane): as many whole steps as 64 lanes
// hold, a divisor of the iteration (six-column tiles: 8 steps on 48 lanes)
constexpr int steps_per_decode(int tn)
{
    int kb = 64 / tn < steps_per_iteration(tn) ? 64 / tn : steps_per_iteration(tn);
    while (steps_per_iteration(tn) % kb) --kb;
    return kb;
}

struct DArgs {
    PDesc p;
    QDesc q;
    const uint8_t *lut_img;  // byte image indexed (uniform mantissa << m) | lane mantissa, + one all-zero row
    int lut_bytes, m, lane_first;
    int64_t R, J, K;
    float *out;
    int64_t so_r, so_j, out_batch_stride;
    int batch, vec_store;
    Epilogue ep;
    unsigned X, Y;   // row tiles of 64, column tiles of TN
    int wks;         // wavefronts of a workgroup that share one tile, each on its own slice of the reduction
    int nsplit;      // slices of the reduction across workgroups (their partial sums go to `partial`)
    int kslice;      // reduction steps per slice
    float *partial;  // [nsplit][batch][Rp][Jp]
    int64_t Rp;
    int Jp;
};

// per-lane view of the lane operand: where this lane's row starts and how to test a window position
struct RowRef {
    int base;      // element offset of the row's origin in the source (may be negative for patches)
    int vy0, vx0;  // P_PATCH: window origin (y * sy - pt, x * sx - pl); P_GF: (fy, fx)
    bool valid;
};

template <int PK>
__device__ __forceinline__ RowRef make_row(const PDesc &p, int64_t r, int64_t R)
{
    RowRef rr{0, 0, 0, r < R};
    if (!rr.valid) return rr;
    if (PK == P_PATCH) {
        const uint32_t r32 = (uint32_t)r, gw = (uint32_t)p.GW, gh = (uint32_t)p.GH;  // (fewer than 2^31 rows)
        const int x = (int)(r32 % gw);
        const uint32_t t = r32 / gw;
        const int y = (int)(t % gh);
        const int b = (int)(t / gh);
        rr.vy0 = y * p.sy - p.pt;
        rr.vx0 = x * p.sx - p.pl;
        rr.base = ((b * p.SH + rr.vy0) * p.SW + rr.vx0) * p.C;
    } else if (PK == P_GF) {
        const int c = (int)((uint32_t)r % (uint32_t)p.C);
        const int t = (int)((uint32_t)r / (uint32_t)p.C);
        rr.vx0 = t % p.KW;
        rr.vy0 = t / p.KW;
        rr.base = (rr.vy0 * p.SW + rr.vx0) * p.C + c;
    }
    return rr;
}

// walks the reduction index of a patch / filter-gradient source with scalar adds
struct KWalk {
    int a, b, c;  // P_PATCH: (fy, fx, channel);  P_GF: (image, oy, ox)
};
template <int PK>
__device__ __forceinline__ KWalk make_walk(const PDesc &p, int64_t k)
{
    KWalk w{0, 0, 0};
    if (PK == P_PATCH) {
        w.c = (int)((uint32_t)k % (uint32_t)p.C);  // (the reduction is shorter than 2^31)
        const int t = (int)((uint32_t)k / (uint32_t)p.C);
        w.b = t % p.KW;
        w.a = t / p.KW;
    } else if (PK == P_GF) {
        w.c = (int)((uint32_t)k % (uint32_t)p.GW);
        const uint32_t t = (uint32_t)k / (uint32_t)p.GW;
        w.b = (int)(t % (uint32_t)p.GH);
        w.a = (int)(t / (uint32_t)p.GH);
    }
    return w;
}
template <int PK>
__device__ __forceinline__ void step_walk(const PDesc &p, KWalk &w)
{
    if (PK == P_PATCH) {
        if (++w.c == p.C) { w.c = 0; if (++w.b == p.KW) { w.b = 0; ++w.a; } }
    } else if (PK == P_GF) {
        if (++w.c == p.GW) { w.c = 0; if (++w.b == p.GH) { w.b = 0; ++w.a; } }
    }
}

// TN  columns per wavefront;  PK lane-operand source;  VEC: reduction steps read per load (4 or 2 where
// the source is contiguous along the reduction and aligned to as many floats: row-major dense
// operands, and the channels of a patch source whose depth is a multiple of VEC -- one window test per
// load instead of one per element)
template <int TN, int PK, int VEC>
__global__ __launch_bounds__(WG_THREADS, 4) void lutgemm_direct_kernel(DArgs a)
{
    constexpr int SI = steps_per_iteration(TN);      // reduction steps per loop iteration
    constexpr int KB = steps_per_decode(TN);         // steps whose uniform operands one decode (one register) covers
    constexpr int NB = SI / KB;                      // decodes per iteration
    __shared__ __align__(16) uint8_t lut_s[LUT_LDS_BYTES];
    static_assert(DIRECT_WAVES * 16 * 64 * sizeof(float) <= LUT_LDS_BYTES, "the partial sums reuse the LUT's LDS");
    float(*red)[TN][64] = reinterpret_cast<float(*)[TN][64]>(lut_s);  // after the loop, behind a barrier

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    {
        constexpr int NVEC = LUT_LDS_BYTES / 16;
#pragma unroll
        for (int i = 0; i * WG_THREADS < NVEC; ++i) {
#if defined(__HIP_DEVICE_COMPILE__)  // the builtin exists in the device pass only
            const int v0 = i * WG_THREADS + wave * 64;
            if ((v0 + lane) * 16 < a.lut_bytes)
                __builtin_amdgcn_global_load_lds(a.lut_img + (v0 + lane) * 16, lut_s + v0 * 16, 16, 0, 0);
#endif
        }
    }
    const int tpw = DIRECT_WAVES / a.wks;  // tiles per workgroup (along the rows)
    const unsigned XG = (a.X + tpw - 1) / tpw;
    unsigned v = blockIdx.x;
    const unsigned xg = v % XG; v /= XG;
    const unsigned by = v % a.Y; v /= a.Y;
    const int split = v % a.nsplit;
    const int bz = v / a.nsplit;
    const int ks = wave % a.wks;
    const unsigned bx = xg * tpw + wave / a.wks;
    const bool tile_live = bx < a.X;
    const int64_t r = (int64_t)bx * 64 + lane;
    const int j0 = by * TN;
    const int m = a.m, mshift = 23 - m;
    const int64_t kbeg = (int64_t)(split * a.wks + ks) * a.kslice;
    const int64_t kend = kbeg + a.kslice < a.K ? kbeg + a.kslice : a.K;

    const float *pbase = a.p.base + (int64_t)bz * a.p.batch_stride;
    const float *qbase = a.q.base + (a.q.batches > 1 ? (int64_t)bz * a.q.batch_stride : 0);
    const RowRef row = make_row<PK>(a.p, tile_live ? r : a.R, a.R);
    const float *prow = pbase + (PK == P_DENSE ? r * a.p.sr : 0);

    float acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = 0.0f;

    // this lane's operand at reduction step k, with the walk state (fy, fx, c) / (image, oy, ox) of k
    auto load_p = [&](int64_t k, const KWalk &w) -> uint32_t {
        if (!row.valid || k >= kend) return 0u;
        if (PK == P_DENSE) return f2u(prow[k * a.p.sk]);
        if (PK == P_PATCH) {
            // source pixel (vy0 + fy, vx0 + fx), zero outside the image
            if ((unsigned)(row.vy0 + w.a) < (unsigned)a.p.SH && (unsigned)(row.vx0 + w.b) < (unsigned)a.p.SW)
                return f2u(pbase[row.base + (w.a * a.p.SW + w.b) * a.p.C + w.c]);
            return 0u;
        }
        // this row's tap (fy, fx) reads input pixel (oy * sy - pt + fy, ox * sx - pl + fx)
        const int iy0 = w.b * a.p.sy - a.p.pt, ix0 = w.c * a.p.sx - a.p.pl;
        if ((unsigned)(iy0 + row.vy0) < (unsigned)a.p.SH && (unsigned)(ix0 + row.vx0) < (unsigned)a.p.SW)
            return f2u(pbase[((w.a * a.p.SH + iy0) * a.p.SW + ix0) * a.p.C + row.base]);
        return 0u;
    };

    // Operands of the SI reduction steps from k0 on.  Every load is issued before anything waits: one
    // memory latency per SI steps.  Uniform operand: in decode nb, lane l (< KB * TN) holds element
    // (k0 + nb * KB + l / TN, j0 + l % TN).
    const bool live = tile_live && kbeg < kend;
    KWalk walk = make_walk<PK>(a.p, live ? kbeg : 0);
    auto issue_loads = [&](int64_t k0, uint32_t (&qraw)[NB], uint32_t (&praw)[SI]) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const uint32_t qk = (uint32_t)k0 + nb * KB + lane / TN, qj = (uint32_t)j0 + lane % TN;
            qraw[nb] = (live && lane < KB * TN && qk < (uint32_t)kend) ? q_raw_bits(a.q, qbase, (uint32_t)a.K, (uint32_t)a.J, qk, qj) : 0u;
        }
        if (PK == P_DENSE && VEC == 4) {
#pragma unroll
            for (int kk = 0; kk < SI; kk += 4) {
                uint4 q4 = make_uint4(0, 0, 0, 0);
                if (live && row.valid && k0 + kk < kend) q4 = *reinterpret_cast<const uint4 *>(prow + k0 + kk);  // kend % 4 == 0 here
                praw[kk] = q4.x; praw[kk + 1] = q4.y; praw[kk + 2] = q4.z; praw[kk + 3] = q4.w;
            }
        } else if (PK == P_PATCH && VEC > 1) {
            // VEC channels of one window position per load: k0, the slice bounds and the depth are
            // multiples of VEC, so a group never straddles a window position or the slice's end
#pragma unroll
            for (int kk = 0; kk < SI; kk += VEC) {
                uint32_t v[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) v[i] = 0u;
                if (live && row.valid && k0 + kk < kend && (unsigned)(row.vy0 + walk.a) < (unsigned)a.p.SH &&
                    (unsigned)(row.vx0 + walk.b) < (unsigned)a.p.SW) {
                    const float *src = pbase + row.base + (walk.a * a.p.SW + walk.b) * a.p.C + walk.c;
                    if (VEC == 4) {
                        const uint4 t = *reinterpret_cast<const uint4 *>(src);
                        v[0] = t.x; v[1] = t.y; v[VEC - 2] = t.z; v[VEC - 1] = t.w;
                    } else {
                        const uint2 t = *reinterpret_cast<const uint2 *>(src);
                        v[0] = t.x; v[1] = t.y;
                    }
                }
#pragma unroll
                for (int i = 0; i < VEC; ++i) praw[kk + i] = v[i];
                walk.c += VEC;
                if (walk.c == a.p.C) { walk.c = 0; if (++walk.b == a.p.KW) { walk.b = 0; ++walk.a; } }
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < SI; ++kk) {
                praw[kk] = live ? load_p(k0 + kk, walk) : 0u;
                step_walk<PK>(a.p, walk);
            }
        }
    };
    auto compute = [&](int64_t k0, const uint32_t (&qraw)[NB], const uint32_t (&praw)[SI]) {
        SafeRange qr, pr;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) qr.add(qraw[nb]);
#pragma unroll
        for (int kk = 0; kk < SI; ++kk) pr.add(praw[kk]);
        // every operand passes the quick test, or (second look) the two operands' exponent ranges over
        // these steps are such that every product can still take the fast form
        bool fast = !__any((qr.unsafe() || pr.unsafe()) ? 1 : 0);
        if (!fast) fast = spans_compatible(span_word(wave_union(pr)), span_word(wave_union(qr)));
        if (fast) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                // sign|exponent in the top 9 bits, LUT row offset below: one register, read back once per product.
                // Zero (and padding) elements select the all-zero LUT row that follows the table.
                const uint32_t qword = (qraw[nb] & 0xff800000u) |
                                       (((qraw[nb] & 0x7fffffffu) ? ((qraw[nb] & 0x7fffffu) >> mshift) : (1u << m)) << m);
                // The KB * TN products of this decode in groups of G: a group's words come back as scalars
                // (v_readlane), its addresses and gathers go out together, and while they are in flight the
                // group before it is finished (byte -> factor, FMA).  The fences keep the scheduler from
                // serialising a group through one scalar register and from draining the LDS queue after
                // every few gathers: a lone wavefront has nothing else to hide that latency with.
                constexpr int PAIRS = KB * TN;
                constexpr int G = PAIRS < 8 ? PAIRS : 8;
                uint32_t lb[2][G], sw[2][G];
                auto gather_group = [&](int g0, uint32_t (&dst)[G], uint32_t (&words)[G]) {
#pragma unroll
                    for (int g = 0; g < G; ++g) words[g] = __builtin_amdgcn_readlane(qword, g0 + g);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const uint32_t pv = praw[nb * KB + (g0 + g) / TN];
                        // LUT address = lane mantissa index + the word's row offset.  A 16-bit add does it without
                        // masking the word first: the row offset (< 2^15) sits in its low half, the sign|exponent
                        // bits drop out, and the instruction clears the upper half of its destination.
                        uint32_t li;
                        asm("v_add_u16 %0, %1, %2" : "=v"(li) : "s"(words[g]), "v"(__builtin_amdgcn_ubfe(pv, (uint32_t)mshift, (uint32_t)m)));
                        dst[g] = lut_s[li];
                    }
                    __builtin_amdgcn_sched_barrier(0);
                };
                auto finish_group = [&](int g0, const uint32_t (&src)[G], const uint32_t (&words)[G], bool next_in_flight) {
                    // one wait for the whole group (all but the next group's G gathers have landed) instead of
                    // one before every product: each wait is an issue slot of a wavefront that has few to spare
                    // (operand: no wait on the vector-memory and export counters, LDS counter in bits 11..8)
                    if (next_in_flight) __builtin_amdgcn_s_waitcnt(0xC07F | (G << 8));
                    else __builtin_amdgcn_s_waitcnt(0xC07F);
                    __builtin_amdgcn_sched_barrier(0);  // (keeps the wait ahead of the group's products)
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const uint32_t pv = praw[nb * KB + (g0 + g) / TN];
                        // (LUT byte << 16) + sign|exponent bits of q  ==  q_pow2 * 1.mant * 2^carry, exactly
                        acc[(g0 + g) % TN] = __builtin_fmaf(u2f(pv & 0xff800000u), u2f((src[g] << 16) + (words[g] & 0xff800000u)),
                                                            acc[(g0 + g) % TN]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                };
                gather_group(0, lb[0], sw[0]);
#pragma unroll
                for (int g0 = 0; g0 < PAIRS; g0 += G) {
                    if (g0 + G < PAIRS) gather_group(g0 + G, lb[((g0 / G) + 1) & 1], sw[((g0 / G) + 1) & 1]);
                    finish_group(g0, lb[(g0 / G) & 1], sw[(g0 / G) & 1], g0 + G < PAIRS);
                }
            }
        } else {
            // Rare: an operand outside the fast product's range somewhere in these steps.  One step
            // at a time, operands fetched again (no register is indexed dynamically, small code).
            const int64_t kstop = k0 + SI < kend ? k0 + SI : kend;
#pragma unroll 1
            for (int64_t k = k0; k < kstop; ++k) {
                const uint32_t raw = load_p(k, make_walk<PK>(a.p, k));
                const uint32_t ia = (raw & 0x7fffffu) >> mshift;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const uint32_t qr = q_raw_bits(a.q, qbase, (uint32_t)a.K, (uint32_t)a.J, (uint32_t)k, (uint32_t)(j0 + j));
                    const uint32_t e16 = (uint32_t)lut_s[(((qr & 0x7fffffu) >> mshift) << m) + ia] << 16;
                    acc[j] += a.lane_first ? am_exact(raw, qr, e16) : am_exact(qr, raw, e16);
                }
            }
        }
    };

    // the first operands travel while the LUT copies land
    uint32_t qcur[NB], pcur[SI], qnxt[NB], pnxt[SI];
    issue_loads(kbeg, qcur, pcur);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the LUT's direct-to-LDS copies are not tracked per register)
    __syncthreads();

    if (live) {
        for (int64_t k0 = kbeg; k0 < kend; k0 += SI) {
            issue_loads(k0 + SI, qnxt, pnxt);  // past the end: all zeros, no access
            compute(k0, qcur, pcur);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) qcur[nb] = qnxt[nb];
#pragma unroll
            for (int kk = 0; kk < SI; ++kk) pcur[kk] = pnxt[kk];
        }
    }
    // slices of one tile inside the workgroup: summed in slice order by the first of them
    if (a.wks > 1) {
        __syncthreads();  // every wavefront of the workgroup is done with the LUT
        if (ks != 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j) red[wave][j][lane] = acc[j];
        }
        __syncthreads();
        if (ks == 0) {
            for (int s = 1; s < a.wks; ++s)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[j] += red[wave + s][j][lane];
        }
    }
    if (ks != 0 || !tile_live || r >= a.R) return;
    if (a.nsplit == 1) {
        float *o = a.out + (int64_t)bz * a.out_batch_stride + out_row_offset(a.ep.omap, r, a.so_r);
        if (a.ep.bias_j || a.ep.bias_r || a.ep.act) {
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] = apply_epilogue(a.ep, acc[j], r, min((int64_t)(j0 + j), a.J - 1));
        }
        if (TN % 4 == 0 && a.vec_store && j0 + TN <= a.J) {
            float4 *o4 = reinterpret_cast<float4 *>(o + j0);
#pragma unroll
            for (int j = 0; j < TN / 4; ++j) o4[j] = make_float4(acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3]);
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j)
                if (j0 + j < a.J) o[(int64_t)(j0 + j) * a.so_j] = acc[j];
        }
    } else {
        float *o = a.partial + (((size_t)split * a.batch + bz) * a.Rp + r) * a.Jp + j0;
#pragma unroll
        for (int j = 0; j < TN; ++j)
            if (j0 + j < a.Jp) o[j] = acc[j];
    }
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

struct DPlan {
    int TN, wks, nsplit, kslice, Jp;
    int64_t Rp;
    size_t partial_bytes;
};

// (six columns: LeNet-5's first convolution has six output channels, its second six input channels)
inline int tn_of(int64_t J) { return J >= 9 ? 16 : J >= 7 ? 8 : J >= 5 ? 6 : J >= 3 ? 4 : J >= 2 ? 2 : 1; }

// How a problem is cut: tiles of 64 rows x TN columns, and the reduction into wks slices inside a
// workgroup times nsplit across workgroups, aiming at a few wavefronts per SIMD with at least a
// couple of decode batches each.
DPlan plan_direct(int64_t R, int64_t J, int64_t K, int batch, bool may_split, int cus)
{
    DPlan pl{};
    pl.TN = tn_of(J);
    const int KB = steps_per_iteration(pl.TN);  // reduction steps per loop iteration of the kernel
    const int64_t tiles = ((R + 63) / 64) * ((J + pl.TN - 1) / pl.TN) * batch;
    const int64_t kbatches = (K + KB - 1) / KB;
    int64_t slices = 1;
    if (may_split) {
        const int64_t want_waves = (int64_t)cus * 4 * 6;  // six wavefronts per SIMD, but at least one iteration each
        slices = std::max<int64_t>(1, std::min<int64_t>(want_waves / std::max<int64_t>(tiles, 1), kbatches));
    }
    pl.wks = slices >= 4 ? 4 : slices >= 2 ? 2 : 1;
    pl.nsplit = (int)std::max<int64_t>(1, std::min<int64_t>((slices + pl.wks - 1) / pl.wks, 4096));
    if (pl.nsplit < 4) pl.nsplit = 1;  // not worth a second launch
    const int64_t total = (int64_t)pl.wks * pl.nsplit;
    int64_t per = (kbatches + total - 1) / total * KB;  // steps per slice, whole decode batches
    pl.kslice = (int)per;
    pl.nsplit = (int)((K + per * pl.wks - 1) / (per * pl.wks));  // drop slices that would be empty
    pl.Rp = (R + 63) / 64 * 64;
    pl.Jp = (int)((J + pl.TN - 1) / pl.TN * pl.TN);
    pl.partial_bytes = pl.nsplit > 1 ? align256((size_t)pl.nsplit * batch * pl.Rp * pl.Jp * sizeof(float)) : 0;
    return pl;
}

template <int TN>
void launch_direct_tn(const DArgs &a, dim3 grid, hipStream_t stream)
{
    const PDesc &p = a.p;
    if (p.kind == P_DENSE) {
        const bool vec = p.sk == 1 && p.sr % 4 == 0 && p.batch_stride % 4 == 0 &&
                         a.K % 4 == 0 && aligned16(p.base);
        if (vec) lutgemm_direct_kernel<TN, P_DENSE, 4><<<grid, WG_THREADS, 0, stream>>>(a);
        else lutgemm_direct_kernel<TN, P_DENSE, 1><<<grid, WG_THREADS, 0, stream>>>(a);
    } else if (p.kind == P_PATCH) {
        const bool even = p.C % 2 == 0 && p.batch_stride % 2 == 0 && ((uintptr_t)p.base & 7) == 0;
        if (p.C % 4 == 0 && p.batch_stride % 4 == 0 && aligned16(p.base))
            lutgemm_direct_kernel<TN, P_PATCH, 4><<<grid, WG_THREADS, 0, stream>>>(a);
        else if (even) lutgemm_direct_kernel<TN, P_PATCH, 2><<<grid, WG_THREADS, 0, stream>>>(a);
        else lutgemm_direct_kernel<TN, P_PATCH, 1><<<grid, WG_THREADS, 0, stream>>>(a);
    } else {
        lutgemm_direct_kernel<TN, P_GF, 1><<<grid, WG_THREADS, 0, stream>>>(a);
    }
}

}  // namespace

// Problems the direct engine takes when engines are picked per problem (measured against the
// LDS-table engine on an MI355X over dense, patch and filter-gradient shapes, both timed from
// captured graphs).  The narrower the output, the longer it stays ahead: the LDS-table engine keeps a
// workgroup's four wavefronts busy only with 32 columns or more.  Up to DIRECT_MAX_MACS_NARROW padded
// products for at most 8 columns (it wins by 25-45 % there), DIRECT_MAX_MACS_16 for at most 16
// (10-35 %; the two meet near 230 million), DIRECT_MAX_MACS beyond (the LDS-table engine is ahead
// from about 60 million on); not single- or two-column outputs of a row-major lane operand, whose
// rows it would read with one strided request per lane.  With any_size (the "direct" engine mode,
// for tests and tuning) everything it can index.
bool direct_shape_eligible(int64_t R, int64_t J, int64_t K, int batch, bool any_size)
{
    if (K <= 0 || R <= 0 || J <= 0 || batch <= 0) return false;
    const int tn = tn_of(J);
    const double tiles = (double)((R + 63) / 64) * (double)((J + tn - 1) / tn) * batch;
    const double padded = tiles * 64.0 * tn * (double)K;
    if (any_size) return padded <= DIRECT_MAX_MACS_ANY;
    return padded <= (J <= 8 ? DIRECT_MAX_MACS_NARROW : J <= 16 ? DIRECT_MAX_MACS_16 : DIRECT_MAX_MACS);
}

bool direct_eligible(int m, const GemmDesc &d, bool any_size)
{
    if (m > 7 || !direct_shape_eligible(d.R, d.J, d.K, d.batch, any_size)) return false;
    if (d.p.kind == P_DENSE) {
        if (!any_size && d.J <= 2 && d.p.sk == 1 && d.p.sr != 1) return false;
        const double span = (double)d.R * std::abs((double)d.p.sr) + (double)d.K * std::abs((double)d.p.sk);
        if (span >= 2147483648.0) return false;
    }
    return d.R < (1ll << 31) && d.K < (1ll << 31) && d.J < (1ll << 24);
}

size_t direct_workspace_bytes(int64_t R, int64_t J, int64_t K, int batch)
{
    // the largest any split mode and device asks for: partial sums of the deepest split
    size_t need = 0;
    for (int cus : {device_compute_units(), 256, 304})
        need = std::max(need, plan_direct(R, J, K, batch, true, cus).partial_bytes);
    return need;
}

int run_gemm_direct(const Lut &lut, const GemmDesc &d, bool may_split, void *workspace, size_t workspace_bytes, hipStream_t stream)
{
    DPlan pl = plan_direct(d.R, d.J, d.K, d.batch, may_split, device_compute_units());
    if (pl.partial_bytes > 0 && (workspace == nullptr || ((uintptr_t)workspace & 255) || workspace_bytes < pl.partial_bytes))
        pl = plan_direct(d.R, d.J, d.K, d.batch, false, device_compute_units());  // runs whole, needs no workspace
    DArgs a{};
    a.p = d.p; a.q = d.q;
    a.lut_img = d.lane_first ? lut.img_ba : lut.img_ab;
    a.lut_bytes = (int)(((size_t)1 << (2 * lut.m)) + ((size_t)1 << lut.m) + 15) / 16 * 16;
    a.m = lut.m; a.lane_first = d.lane_first ? 1 : 0;
    a.R = d.R; a.J = d.J; a.K = d.K;
    a.out = d.out; a.so_r = d.so_r; a.so_j = d.so_j; a.out_batch_stride = d.out_batch_stride;
    a.batch = d.batch;
    a.vec_store = (d.so_j == 1 && d.so_r % 4 == 0 && d.out_batch_stride % 4 == 0 && aligned16(d.out)) ? 1 : 0;
    a.ep = Epilogue{d.bias_j, d.bias_r, d.act, d.omap};
    a.X = (unsigned)((d.R + 63) / 64);
    a.Y = (unsigned)((d.J + pl.TN - 1) / pl.TN);
    a.wks = pl.wks; a.nsplit = pl.nsplit; a.kslice = pl.kslice;
    a.partial = static_cast<float *>(workspace);
    a.Rp = pl.Rp; a.Jp = pl.Jp;
    const int tpw = DIRECT_WAVES / pl.wks;
    const int64_t total = (int64_t)((a.X + tpw - 1) / tpw) * a.Y * pl.nsplit * d.batch;
    if (total >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "workgroup count exceeds the grid limit");
    const dim3 grid((unsigned)total);
    switch (pl.TN) {
    case 16: launch_direct_tn<16>(a, grid, stream); break;
    case 8: launch_direct_tn<8>(a, grid, stream); break;
    case 6: launch_direct_tn<6>(a, grid, stream); break;
    case 4: launch_direct_tn<4>(a, grid, stream); break;
    case 2: launch_direct_tn<2>(a, grid, stream); break;
    default: launch_direct_tn<1>(a, grid, stream); break;
    }
    AMSIM_HIP_CHECK(hipGetLastError());
    if (pl.nsplit > 1) {
        if (d.batch > 65535) return fail(AMSIM_ERR_UNSUPPORTED, "batch exceeds the grid limit");
        RArgs ra{a.partial, d.out, d.R, d.J, pl.Rp, d.so_r, d.so_j, d.out_batch_stride, pl.Jp, pl.nsplit, d.batch, 0, a.ep};
        launch_reduce(ra, stream);
        AMSIM_HIP_CHECK(hipGetLastError());
    }
    return AMSIM_OK;
}

}  // namespace amsim
