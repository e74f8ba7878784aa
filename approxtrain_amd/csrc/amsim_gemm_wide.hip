// Row-staged LUT-multiply GEMM for tables too wide for the LDS (mantissa widths 8..11;
// lut/AMsimulator.inl:18-23 is the reference's lookup for such tables, one texture fetch per
// product).
//
// out(r, j) = sum_k P(p(r, k), q(k, j)) as in the LDS-table engine, lanes = rows r, q wave-uniform.
// At width 11 the table has 2^22 16-bit entries (8 MB): it lives in device memory and is served
// by L2 / MALL.  What makes it tractable is that every product of one (k, j) pair reads the SAME
// 2^m-entry row of the table (the one q(k, j)'s mantissa selects; 4 KB at width 11): a workgroup
// that owns many rows r pulls that row into LDS once and lets all its rows gather from there.
//
//   * one workgroup = 512 threads = 4096 rows (8 per thread) x 8 columns, the whole reduction; two
//     workgroups share a compute unit;
//   * per reduction step k ("stage") the 8 wavefronts copy the 8 table rows of q(k+1, j0..j0+7)
//     into one half of a 64 KB LDS buffer with direct global-to-LDS loads (no registers), while
//     every thread gathers its 8 x 8 entries of stage k from the other half: 32 KB pulled in per
//     32 768 products = 1 byte per product;
//   * the lane operand p is transposed once per call into [k][row] order in the workspace
//     (raw bits, zero-padded), so a thread's operands arrive by fully coalesced 4-byte loads,
//     prefetched one stage ahead, and never touch the LDS;
//   * product form, zero handling and the exact path for flagged 32-deep chunks are those of the
//     LDS-table engine: entry << 8 lands on carry|mantissa, + q's sign|exponent = one factor,
//     fma with p's power of two.
// The gathers are scattered over a 4 KB row (random bank conflicts), which is what bounds the
// kernel: about 5.2 T gathers/s on an MI355X against 17-19 T/s inside the 128-byte rows of the
// narrow tables.
#include "amsim_gemm_common.h"

#include <algorithm>
#include <type_traits>

namespace amsim {

namespace {

// A workgroup is 512 threads = 8 wavefronts (one per staged table row) on 4096 rows x 8 columns, and
// two of them share a compute unit: while one waits at its stage barrier the other gathers (measured
// 4.7 TMAC/s against 4.45 for one 1024-thread workgroup on 16 columns).
constexpr int WIDE_TILE_ROWS = 4096;              // rows per workgroup (half of that when workgroups are too few, below)
constexpr int WIDE_TN = 8;                        // columns per workgroup: half a tile of the pre-decoded operand
constexpr int WIDE_THREADS = WIDE_TN * 64;
constexpr int WIDE_ENTRY_BYTES = WIDE_TN * 2;      // LDS bytes per lane-mantissa value: one 16-bit entry of each staged row
constexpr int WIDE_BUF_BYTES = 2048 * WIDE_ENTRY_BYTES;  // one stage's rows, interleaved (2^11 mantissa values)
constexpr int PT_ROWS = 64;                       // rows per workgroup of the transposing pre-pass

struct PTArgs {
    PDesc p;
    int64_t R, K, Rp;
    int nchunks;
    uint32_t *pt;      // [batch][nchunks * KC][Rp] raw bits
    uint32_t *pflags;  // [batch][nchunks][Rp / 64] operand spans
};

// One workgroup per (64-row group, 32-deep chunk) and batch item (blockIdx.y): reads the tile along
// the source's contiguous direction -- for patch sources this IS the im2col the reference
// materialises (cuda/cuda_kernel.cu:35-60), here transposed -- writes it in [k][row] order, flags it
// if it holds an operand the fast product path cannot take.
__global__ __launch_bounds__(WG_THREADS) void p_linear_kernel(PTArgs a)
{
    __shared__ uint32_t tile[KC][PT_ROWS + 1];
    __shared__ int4 rowinfo[PT_ROWS];  // patch sources: {element offset of the window origin, y origin, x origin, row inside R}
    const int64_t G = a.Rp / PT_ROWS;
    const int64_t g = blockIdx.x % G, ch = blockIdx.x / G;
    const int bz = blockIdx.y;
    const int tid = threadIdx.x;
    const float *pbase = a.p.base + (int64_t)bz * a.p.batch_stride;
    uint32_t *pt = a.pt + (size_t)bz * a.nchunks * KC * a.Rp;
    // lanes along k where the source is contiguous there: row-major dense operands, and patches
    // (channels run fastest in both the image and the reduction index)
    const bool k_fast = a.p.kind == P_PATCH || (a.p.kind == P_DENSE && a.p.sk == 1 && a.p.sr != 1);
    SafeRange range;
    if (a.p.kind == P_PATCH) {
        // A thread's reduction index is the same for all its elements (lanes run along k): decomposed
        // once; the rows' window origins once per workgroup, through LDS -- instead of four divisions
        // per element.
        if (tid < PT_ROWS) {
            const int64_t r = g * PT_ROWS + tid;
            int4 v = make_int4(0, 0, 0, 0);
            if (r < a.R) {
                const uint32_t r32 = (uint32_t)r, gw = (uint32_t)a.p.GW, gh = (uint32_t)a.p.GH;  // (fewer than 2^31 rows)
                const int x = (int)(r32 % gw);
                const uint32_t t = r32 / gw;
                const int y = (int)(t % gh), b = (int)(t / gh);
                const int vy0 = y * a.p.sy - a.p.pt, vx0 = x * a.p.sx - a.p.pl;
                v = make_int4(((b * a.p.SH + vy0) * a.p.SW + vx0) * a.p.C, vy0, vx0, 1);
            }
            rowinfo[tid] = v;
        }
        __syncthreads();
        const int kk = tid % KC;
        const int64_t k = ch * KC + kk;
        const uint32_t k32 = (uint32_t)k, c32 = (uint32_t)a.p.C;
        const int c = (int)(k32 % c32), tap = (int)(k32 / c32);
        const int fx = tap % a.p.KW, fy = tap / a.p.KW;
        const int tapoff = (fy * a.p.SW + fx) * a.p.C + c;
        const bool kvalid = k < a.K;
#pragma unroll
        for (int i = 0; i < KC * PT_ROWS / WG_THREADS; ++i) {
            const int rl = tid / KC + (WG_THREADS / KC) * i;
            const int4 ri = rowinfo[rl];
            uint32_t raw = 0u;
            if (kvalid && ri.w && (unsigned)(ri.y + fy) < (unsigned)a.p.SH && (unsigned)(ri.z + fx) < (unsigned)a.p.SW)
                raw = f2u(pbase[ri.x + tapoff]);
            range.add(raw);
            tile[kk][rl] = raw;
        }
    } else if (a.p.kind == P_GF) {
        // Filter gradients: lanes run along the rows (filter elements; the channel is the contiguous
        // direction of the source), so a thread's row is the same for all its elements: decomposed once;
        // the chunk's 32 pixels once per workgroup, through LDS.
        static_assert(KC <= PT_ROWS, "the pixel bookkeeping reuses the row bookkeeping's LDS");
        if (tid < KC) {
            const int64_t k = ch * KC + tid;
            int4 v = make_int4(0, 0, 0, 0);
            if (k < a.K) {
                const uint32_t k32 = (uint32_t)k, gw = (uint32_t)a.p.GW, gh = (uint32_t)a.p.GH;  // (the reduction is shorter than 2^31)
                const int x = (int)(k32 % gw);
                const uint32_t t = k32 / gw;
                const int y = (int)(t % gh), b = (int)(t / gh);
                const int iy0 = y * a.p.sy - a.p.pt, ix0 = x * a.p.sx - a.p.pl;
                v = make_int4(((b * a.p.SH + iy0) * a.p.SW + ix0) * a.p.C, iy0, ix0, 1);
            }
            rowinfo[tid] = v;
        }
        __syncthreads();
        const int rl = tid % PT_ROWS;
        const int64_t r = g * PT_ROWS + rl;
        const uint32_t r32 = (uint32_t)r, c32 = (uint32_t)a.p.C;
        const int c = (int)(r32 % c32), tap = (int)(r32 / c32);
        const int fx = tap % a.p.KW, fy = tap / a.p.KW;
        const int tapoff = (fy * a.p.SW + fx) * a.p.C + c;
        const bool rvalid = r < a.R;
#pragma unroll
        for (int i = 0; i < KC * PT_ROWS / WG_THREADS; ++i) {
            const int kk = tid / PT_ROWS + (WG_THREADS / PT_ROWS) * i;
            const int4 ki = rowinfo[kk];
            uint32_t raw = 0u;
            if (rvalid && ki.w && (unsigned)(ki.y + fy) < (unsigned)a.p.SH && (unsigned)(ki.z + fx) < (unsigned)a.p.SW)
                raw = f2u(pbase[ki.x + tapoff]);
            range.add(raw);
            tile[kk][rl] = raw;
        }
    } else {
#pragma unroll
    for (int i = 0; i < KC * PT_ROWS / WG_THREADS; ++i) {
        const int e = tid + WG_THREADS * i;
        int kk, rl;
        if (k_fast) { kk = e % KC; rl = e / KC; }
        else { rl = e % PT_ROWS; kk = e / PT_ROWS; }
        const int64_t r = g * PT_ROWS + rl, k = ch * KC + kk;
        const uint32_t raw = p_raw_bits(a.p, pbase, a.R, a.K, r, k);
        range.add(raw);
        tile[kk][rl] = raw;
    }
    }
    // the tile's operand span: per wavefront by shuffles, across the four through LDS
    __shared__ uint32_t wave_range[WG_THREADS / 64][2];
    range = wave_union(range);
    if ((tid & 63) == 0) { wave_range[tid >> 6][0] = range.tmax; wave_range[tid >> 6][1] = range.tmin; }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < KC * PT_ROWS / WG_THREADS; ++i) {
        const int e = tid + WG_THREADS * i;
        const int rl = e % PT_ROWS, kk = e / PT_ROWS;
        pt[(size_t)(ch * KC + kk) * a.Rp + g * PT_ROWS + rl] = tile[kk][rl];
    }
    if (tid == 0) {
        SafeRange all;
#pragma unroll
        for (int w = 0; w < WG_THREADS / 64; ++w) { all.tmax = max(all.tmax, wave_range[w][0]); all.tmin = min(all.tmin, wave_range[w][1]); }
        a.pflags[((size_t)bz * a.nchunks + ch) * G + g] = span_word(all);
    }
}

// LDS byte address of a pointer into a __shared__ object
__device__ __forceinline__ uint32_t lds_addr(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// The 8 products of one row with the 8 staged entries in e (two per dword), accumulated in place:
//   factor = (entry << 8) + sign|exponent bits of q  ==  q_pow2 * 1.mant * 2^carry, exactly, in one
//   instruction (16-bit multiply by 256 of the dword's low or high half, 32-bit add);
//   acc += p_pow2 * factor, fused.
// Written out so that no multiply-add reads a factor written by the instruction just before it (that
// pairing costs a wait state each time) and so that the two temporaries stay two.
__device__ __forceinline__ void mac8(float (&acc)[8], const uint4 &e, float ta, uint32_t c256, const uint32_t (&q)[8])
{
    uint32_t t0, t1;
    asm("v_mad_u32_u16 %[t0], %[ex], %[c], %[q0]\n\t"
        "v_mad_u32_u16 %[t1], %[ex], %[c], %[q1] op_sel:[1,0,0,0]\n\t"
        "v_fmac_f32 %[a0], %[ta], %[t0]\n\t"
        "v_mad_u32_u16 %[t0], %[ey], %[c], %[q2]\n\t"
        "v_fmac_f32 %[a1], %[ta], %[t1]\n\t"
        "v_mad_u32_u16 %[t1], %[ey], %[c], %[q3] op_sel:[1,0,0,0]\n\t"
        "v_fmac_f32 %[a2], %[ta], %[t0]\n\t"
        "v_mad_u32_u16 %[t0], %[ez], %[c], %[q4]\n\t"
        "v_fmac_f32 %[a3], %[ta], %[t1]\n\t"
        "v_mad_u32_u16 %[t1], %[ez], %[c], %[q5] op_sel:[1,0,0,0]\n\t"
        "v_fmac_f32 %[a4], %[ta], %[t0]\n\t"
        "v_mad_u32_u16 %[t0], %[ew], %[c], %[q6]\n\t"
        "v_fmac_f32 %[a5], %[ta], %[t1]\n\t"
        "v_mad_u32_u16 %[t1], %[ew], %[c], %[q7] op_sel:[1,0,0,0]\n\t"
        "v_fmac_f32 %[a6], %[ta], %[t0]\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32 %[a7], %[ta], %[t1]"
        : [a0] "+v"(acc[0]), [a1] "+v"(acc[1]), [a2] "+v"(acc[2]), [a3] "+v"(acc[3]), [a4] "+v"(acc[4]),
          [a5] "+v"(acc[5]), [a6] "+v"(acc[6]), [a7] "+v"(acc[7]), [t0] "=&v"(t0), [t1] "=&v"(t1)
        : [ex] "v"(e.x), [ey] "v"(e.y), [ez] "v"(e.z), [ew] "v"(e.w), [ta] "v"(ta), [c] "v"(c256),
          [q0] "s"(q[0]), [q1] "s"(q[1]), [q2] "s"(q[2]), [q3] "s"(q[3]), [q4] "s"(q[4]), [q5] "s"(q[5]),
          [q6] "s"(q[6]), [q7] "s"(q[7]));
}

// Buffer addressing for the streams of the main loop: a load names a resource (uniform base), a
// uniform byte offset in a scalar register and a 32-bit lane offset, and the hardware adds them --
// no vector instruction is spent on addresses, and none of the 64-bit vector pointers that flat
// addressing would keep alive.  Raw buffers of the maximum extent: offsets are not range-checked
// short of 4 GB.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *uniform_base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(uniform_base), 0, -1, 0x00020000);
}
__device__ __forceinline__ uint32_t load_u32(rsrc_t r, uint32_t lane_offset, uint32_t uniform_offset)
{
    return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_offset, (int)uniform_offset, 0);
}

struct WArgs {
    const uint32_t *pt;
    const uint32_t *pflags;
    const uint8_t *lut16;    // 16-bit image indexed (uniform mantissa << m) | lane mantissa, + one all-zero row
    const uint32_t *qw;      // [Jp/16][Kp][16]
    const uint32_t *qflags;  // [Jp/16][nchunks]
    const QDesc *qdesc;
    int m, lane_first;
    int64_t R, J, K, Rp;
    int Jp, nchunks;
    float *out;
    int64_t so_r, so_j, out_batch_stride;
    int vec_store;
    int q_batches;           // 1: the uniform operand is shared by every batch item
    Epilogue ep;
    unsigned X, Y;           // row tiles, column strips (blockIdx.y runs over the batch)
    int nsplit;              // slices of the reduction (blockIdx.z), each a whole number of chunks
    int chunks_per_split;
    float *partial;          // nsplit > 1: [nsplit][batch][X * tile rows][Jp] partial sums instead of `out`
    // PLANAR (convolution patches read from a channel-major copy of the source instead of an im2col):
    // `pt` is [channel][pixel] with plane_elems pixels per channel, `pflags` [channel chunk][64-pixel group]
    PDesc p;
    int64_t plane_elems;     // B * ph * pw, rounded up to whole 64-pixel groups
    int ph, pw;              // padded image extent: (GH - 1) * sy + KH rows, (GW - 1) * sx + KW columns
    int cchunks;
};

// MPT: pairs of lane-mantissa values each thread stages per reduction step (2 at width 11: 2048 values
// over 512 threads; 1 below, where the wavefronts past the row's end stage nothing).
// RPT: rows per thread, 8 (4096 rows per workgroup: 1 byte of table row pulled per product) or 4 (2048
// rows, 2 bytes per product: for problems that would otherwise leave compute units without a workgroup).
// PLANAR: the lane operand of a convolution (forward / input gradient) is read from a channel-major,
// zero-bordered copy of the source image, xT[c][b][py][px] with py = source row + pad_top and
// px = source column + pad_left, instead of from an im2col in [k][row] order: element
// (row (b, y, x), k (fy, fx, c)) is xT[c][(b * PH + y * sy + fy) * PW + x * sx + fx], so for one
// reduction step all rows read one channel plane at a uniform shift -- consecutive rows read
// consecutive words (stride sx), no window test, no vector instruction spent on addresses -- and the
// copy is the size of the (padded) source, not KH * KW times it.
template <int MPT, int RPT, bool PLANAR>
__global__ __launch_bounds__(WIDE_THREADS, 4) void lutgemm_wide_kernel(WArgs a)
{
    constexpr int TILE_ROWS = WIDE_THREADS * RPT;
    // Two halves, as two objects: the compiler then knows that the stores that stage one half do not
    // alias the gathers from the other, and does not order one behind the other.
    __shared__ __align__(16) uint8_t rows_a[WIDE_BUF_BYTES];
    __shared__ __align__(16) uint8_t rows_b[WIDE_BUF_BYTES];
    const int tid = threadIdx.x, lane = tid & 63;
    // Each XCD (private L2) gets a contiguous run of column strips of one row tile: its
    // workgroups then stream the same transposed lane operand.
    unsigned bx, by;
    {
        const unsigned T = a.X * a.Y, L = blockIdx.x;
        const unsigned xcd = L % NUM_XCD, idx = L / NUM_XCD;
        const unsigned chunk = T / NUM_XCD, rem = T % NUM_XCD;
        const unsigned V = xcd * chunk + (xcd < rem ? xcd : rem) + idx;
        by = V % a.Y;
        bx = V / a.Y;
    }
    const int64_t row0 = (int64_t)bx * TILE_ROWS;
    const int j0 = by * WIDE_TN;
    constexpr int STRIPS_PER_TILE = QT / WIDE_TN;
    const int m = a.m, oshift = 23 - m - 4;           // lane mantissa -> byte offset of its 16-byte group
    const uint32_t omask = ((1u << m) - 1u) << 4;
    const int Kp = a.nchunks * KC;
    const int ch_beg = blockIdx.z * a.chunks_per_split, ch_end = min(ch_beg + a.chunks_per_split, a.nchunks);
    const int kbeg = ch_beg * KC, kend = ch_end * KC;  // this workgroup's slice of the reduction
    const int bz = blockIdx.y, qb = a.q_batches > 1 ? bz : 0;
    const size_t qt_index = (size_t)qb * (a.Jp / QT) + by / STRIPS_PER_TILE;  // tile of the pre-decoded operand
    const cq1_t qtile = (cq1_t)(uintptr_t)(a.qw + qt_index * Kp * QT + (by % STRIPS_PER_TILE) * WIDE_TN);
    const cq1_t qfl = (cq1_t)(uintptr_t)(a.qflags + qt_index * a.nchunks);
    const uint32_t *ptile = a.pt + (size_t)bz * Kp * a.Rp + row0;  // [k][this workgroup's rows]
    const uint32_t voff = (uint32_t)tid * 4u;                        // this thread's byte offset in a run of dwords
    const rsrc_t lut_rsrc = make_rsrc(a.lut16);
    const int64_t G = (PLANAR ? a.plane_elems : a.Rp) / PT_ROWS;  // 64-row (PLANAR: 64-pixel) groups per flag row
    const uint32_t *pfl = a.pflags + (size_t)bz * a.nchunks * G;
    uint32_t c256 = 256u;
    asm volatile("" : "+v"(c256));  // stays in a vector register (the factor instruction has one scalar port)
    float acc[RPT][WIDE_TN];
#pragma unroll
    for (int rr = 0; rr < RPT; ++rr)
#pragma unroll
        for (int j = 0; j < WIDE_TN; ++j) acc[rr][j] = 0.0f;

    // Staging of one reduction step's 8 table rows, interleaved: the entries of the 8 rows at lane
    // mantissa `ma` lie side by side at byte ma * 16, so that ONE 16-byte LDS read serves a row's 8
    // products (eight scattered 2-byte gathers would meet eight rounds of random bank conflicts).
    // A thread fetches the dwords (two adjacent entries) at pair index tid (+ 512) of each of the 8
    // rows, fully coalesced, ...
    uint32_t tl[MPT][WIDE_TN];
    // (a row of a table narrower than 10 bits is shorter than one pass of the workgroup: whole
    // wavefronts then have nothing to stage; rows are multiples of a wavefront's 256 bytes)
    const bool stages = MPT > 1 || (uint32_t)__builtin_amdgcn_readfirstlane(tid) * 4u < (2u << m);
    auto fetch_row = [&](int k, int j) {
        const uint32_t row = (qtile[k * QT + j] & 0x7fffffu) * 2u;  // byte offset of the row q(k, j0 + j) selects
        if (stages) {
#pragma unroll
            for (int i = 0; i < MPT; ++i) tl[i][j] = load_u32(lut_rsrc, voff + i * (WIDE_THREADS * 4), row);
        }
    };
    auto fetch_rows = [&](int k) {
#pragma unroll
        for (int j = 0; j < WIDE_TN; ++j) fetch_row(k, j);
    };
    // ... and regroups them into the 16-byte groups of its two mantissa values (low halves, high halves).
    auto store_rows = [&](uint8_t *half) {
        if (!stages) return;
#pragma unroll
        for (int i = 0; i < MPT; ++i) {
            uint4 lo, hi;
            lo.x = __builtin_amdgcn_perm(tl[i][1], tl[i][0], 0x05040100u); hi.x = __builtin_amdgcn_perm(tl[i][1], tl[i][0], 0x07060302u);
            lo.y = __builtin_amdgcn_perm(tl[i][3], tl[i][2], 0x05040100u); hi.y = __builtin_amdgcn_perm(tl[i][3], tl[i][2], 0x07060302u);
            lo.z = __builtin_amdgcn_perm(tl[i][5], tl[i][4], 0x05040100u); hi.z = __builtin_amdgcn_perm(tl[i][5], tl[i][4], 0x07060302u);
            lo.w = __builtin_amdgcn_perm(tl[i][7], tl[i][6], 0x05040100u); hi.w = __builtin_amdgcn_perm(tl[i][7], tl[i][6], 0x07060302u);
            uint4 *dst = reinterpret_cast<uint4 *>(half + (size_t)(tid + i * WIDE_THREADS) * (2 * WIDE_ENTRY_BYTES));
            dst[0] = lo;
            dst[1] = hi;
        }
    };
    uint32_t pc[RPT], pn[RPT];
    // PLANAR: per row the byte offset of its window origin inside a channel plane; per reduction step
    // (walked, k = (fy, fx, c) with the channel fastest) the channel and the tap.
    uint32_t pixoff[PLANAR ? RPT : 1];
    int w_c = 0, w_tap = 0, w_fx = 0, w_fy = 0;      // the step whose operands load_p fetches next
    if (PLANAR) {
#pragma unroll
        for (int rr = 0; rr < RPT; ++rr) {
            const int64_t r = row0 + rr * WIDE_THREADS + tid;
            uint32_t off = 0u;  // (padding rows read the first pixel: their sums are never stored)
            if (r < a.R) {
                const uint32_t r32 = (uint32_t)r, gw = (uint32_t)a.p.GW, gh = (uint32_t)a.p.GH;  // (fewer than 2^31 rows)
                const uint32_t x = r32 % gw, t = r32 / gw;
                const uint32_t y = t % gh, b = t / gh;
                off = ((b * (uint32_t)a.ph + y * (uint32_t)a.p.sy) * (uint32_t)a.pw + x * (uint32_t)a.p.sx) * 4u;
            }
            pixoff[rr] = off;
        }
        const uint32_t k0 = (uint32_t)kbeg, C = (uint32_t)a.p.C;
        w_c = (int)(k0 % C);
        w_tap = (int)(k0 / C);
        w_fx = w_tap % a.p.KW;
        w_fy = w_tap / a.p.KW;
    }
    // moves the walk on by one reduction step
    auto walk_step = [&]() {
        if (++w_c == a.p.C) {
            w_c = 0;
            ++w_tap;
            if (++w_fx == a.p.KW) { w_fx = 0; ++w_fy; }
        }
    };
    auto load_p = [&](int k, uint32_t (&dst)[RPT]) {
        if constexpr (PLANAR) {
            // reduction steps past the filter (the last chunk's padding) read nothing: a buffer of no
            // records returns zero for every lane
            const bool live = w_tap < a.p.KH * a.p.KW;
            const rsrc_t src = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(a.pt), 0, live ? 0x7fffffff : 0, 0x00020000);
            const uint32_t shift = live ? (uint32_t)((size_t)w_c * a.plane_elems + (size_t)(w_fy * a.pw + w_fx)) * 4u : 0u;
#pragma unroll
            for (int rr = 0; rr < RPT; ++rr) dst[rr] = load_u32(src, pixoff[rr], shift);
        } else {
            const rsrc_t src = make_rsrc(ptile + (size_t)k * a.Rp);
#pragma unroll
            for (int rr = 0; rr < RPT; ++rr) dst[rr] = load_u32(src, voff, rr * (WIDE_THREADS * 4));
        }
    };

    fetch_rows(kbeg);
    load_p(kbeg, pc);
    store_rows(rows_a);
    __syncthreads();

    // Is any chunk of this workgroup's tile flagged (by its column tile or by a 64-row group of its
    // row tile)?  Almost never: then the whole reduction runs the loop nest that holds nothing but
    // fast stages, whose registers the rare path's state cannot crowd.
    int tile_flagged = 0;
    for (int ch = ch_beg + tid; ch < ch_end; ch += WIDE_THREADS)
        tile_flagged |= (int)(a.qflags[qt_index * a.nchunks + ch] >> 31);
    // PLANAR: the 64-pixel groups that the tile's rows can read at any tap, over every channel chunk
    int64_t pg_lo = 0, pg_hi = -1;
    if (PLANAR) {
        auto pixel_of = [&](int64_t r) -> int64_t {
            const uint32_t r32 = (uint32_t)r, gw = (uint32_t)a.p.GW, gh = (uint32_t)a.p.GH;
            const int64_t x = r32 % gw, t = r32 / gw;
            return ((t / gh) * a.ph + (t % gh) * a.p.sy) * a.pw + x * a.p.sx;
        };
        const int64_t last_row = min(row0 + TILE_ROWS, a.R) - 1;
        pg_lo = pixel_of(row0) / PT_ROWS;
        pg_hi = min(a.plane_elems - 1, pixel_of(last_row) + (int64_t)(a.p.KH - 1) * a.pw + (a.p.KW - 1)) / PT_ROWS;
        const int64_t ngroups = pg_hi - pg_lo + 1;
        for (int64_t i = tid; i < ngroups * a.cchunks; i += WIDE_THREADS)
            tile_flagged |= (int)(a.pflags[(size_t)(i / ngroups) * G + pg_lo + i % ngroups] >> 31);
    } else {
    for (int i = tid; i < (ch_end - ch_beg) * (TILE_ROWS / PT_ROWS); i += WIDE_THREADS)
        tile_flagged |= (int)(pfl[(size_t)(ch_beg + i / (TILE_ROWS / PT_ROWS)) * G + (size_t)bx * (TILE_ROWS / PT_ROWS) +
                                  i % (TILE_ROWS / PT_ROWS)] >> 31);
    }
    tile_flagged = __syncthreads_or(tile_flagged);

    // one stage: the rows of stage k + 1 are fetched while stage k gathers from `cur`, and regrouped
    // into `next` once its products are done
    auto stage = [&](auto exact_tag, int k, const uint8_t *cur, uint8_t *next) {
        constexpr bool EXACT = decltype(exact_tag)::value;
        // (the last stage fetches its own rows and operands once more instead of branching: a
        // straight-line stage keeps the compiler from sinking one stage's FMAs into the next)
        const int kn = min(k + 1, kend - 1);
        if (PLANAR && k + 1 < kend) walk_step();
        if constexpr (!EXACT) {
            uint32_t qt[WIDE_TN];
#pragma unroll
            for (int j = 0; j < WIDE_TN; ++j) qt[j] = qtile[k * QT + j] & 0xff800000u;
            fetch_rows(kn);
            load_p(kn, pn);
#pragma unroll
            for (int rr = 0; rr < RPT; ++rr) {
                const uint4 e = *reinterpret_cast<const uint4 *>(cur + ((pc[rr] >> oshift) & omask));
                mac8(acc[rr], e, u2f(pc[rr] & 0xff800000u), c256, qt);
            }
        } else {
            fetch_rows(kn);
            load_p(kn, pn);
            // Rare: full-domain product; q's raw bits come from where the operand lies.  The
            // accumulators take a detour through private memory so that this loop can index them
            // dynamically (small code, one product at a time) while the fast path keeps them in
            // registers.
            const __attribute__((address_space(4))) QDesc &qd = *(const __attribute__((address_space(4))) QDesc *)(uintptr_t)a.qdesc;
            const float *qsrc = qd.base + (int64_t)qb * qd.batch_stride;  // this batch item's operand
            float tmp[RPT * WIDE_TN];
            uint32_t praw[RPT];
#pragma unroll
            for (int rr = 0; rr < RPT; ++rr) {
                praw[rr] = pc[rr];
#pragma unroll
                for (int j = 0; j < WIDE_TN; ++j) tmp[rr * WIDE_TN + j] = acc[rr][j];
            }
#pragma unroll 1
            for (int idx = 0; idx < RPT * WIDE_TN; ++idx) {
                const int rr = idx / WIDE_TN, j = idx % WIDE_TN;
                const uint32_t raw = praw[rr];
                const uint32_t off = (raw >> oshift) & omask;
                const uint32_t e16 = (uint32_t)*reinterpret_cast<const uint16_t *>(cur + off + j * 2) << 8;
                const uint32_t qr = q_raw_bits(qd, qsrc, (uint32_t)a.K, (uint32_t)a.J, (uint32_t)k, (uint32_t)(j0 + j));
                tmp[idx] += a.lane_first ? am_exact(raw, qr, e16) : am_exact(qr, raw, e16);
            }
#pragma unroll
            for (int rr = 0; rr < RPT; ++rr)
#pragma unroll
                for (int j = 0; j < WIDE_TN; ++j) acc[rr][j] = tmp[rr * WIDE_TN + j];
        }
#pragma unroll
        for (int rr = 0; rr < RPT; ++rr) pc[rr] = pn[rr];
        // everyone left `next` at the barrier that ended the stage before; after this one everyone's
        // groups have landed and every wavefront is done gathering from `cur`
        __builtin_amdgcn_sched_barrier(0);
        store_rows(next);
        __syncthreads();
    };
    if (!tile_flagged) {
#pragma unroll 1
        for (int k = kbeg; k < kend; k += 2) {
            stage(std::false_type{}, k, rows_a, rows_b);
            stage(std::false_type{}, k + 1, rows_b, rows_a);
        }
    } else {
        // PLANAR: one span for everything the tile can read (every channel chunk, every pixel group in
        // reach): coarser than a span per chunk, which only matters to inputs that hold values outside
        // the fast product's range in the first place
        uint32_t planar_span = 0u, planar_quick = 0u;
        if (PLANAR) {
            SafeRange join;
            uint32_t quick = 0u, hard = 0u;
            const int64_t ngroups = pg_hi - pg_lo + 1;
            for (int64_t i = lane; i < ngroups * a.cchunks; i += 64) {
                const uint32_t pf = a.pflags[(size_t)(i / ngroups) * G + pg_lo + i % ngroups];
                quick |= pf & SPAN_QUICK_FAIL;
                hard |= pf & SPAN_HARD;
                if ((pf & 0xffffu) != 0xff00u) {  // (not an all-zero group)
                    join.tmax = max(join.tmax, (pf & 255u) << 24);
                    join.tmin = min(join.tmin, ((pf >> 8) & 255u) << 24);
                }
            }
            join = wave_union(join);
            const uint32_t emax = join.tmax >> 24, emin = join.tmin == 0xffffffffu ? 255u : join.tmin >> 24;
            planar_span = (__any(hard != 0u) ? SPAN_HARD : 0u) | (emin << 8) | emax;
            planar_quick = __any(quick != 0u) ? SPAN_QUICK_FAIL : 0u;
        }
        for (int ch = ch_beg; ch < ch_end; ++ch) {
            // spans of the tile's 64-row groups (one per lane: TILE_ROWS / 64 <= 64), joined; the chunk is
            // slow only if a quick test failed AND the joined span is not compatible with the uniform operand's
            SafeRange join;
            uint32_t quick = qfl[ch] & SPAN_QUICK_FAIL, hard = 0u;
            bool unsafe;
            if (PLANAR) {
                unsafe = ((quick | planar_quick) != 0u) && !spans_compatible(planar_span, qfl[ch]);
            } else {
            if (lane < TILE_ROWS / PT_ROWS) {
                const uint32_t pf = pfl[(size_t)ch * G + (size_t)bx * (TILE_ROWS / PT_ROWS) + lane];
                quick |= pf & SPAN_QUICK_FAIL;
                hard = pf & SPAN_HARD;
                if ((pf & 0xffffu) != 0xff00u) {  // (not an all-zero group)
                    join.tmax = (pf & 255u) << 24;
                    join.tmin = ((pf >> 8) & 255u) << 24;
                }
            }
            unsafe = __any(quick != 0u) != 0;
            if (unsafe) {
                join = wave_union(join);
                const uint32_t emax = join.tmax >> 24, emin = join.tmin == 0xffffffffu ? 255u : join.tmin >> 24;
                const uint32_t pspan = (__any(hard != 0u) ? SPAN_HARD : 0u) | (emin << 8) | emax;
                unsafe = !spans_compatible(pspan, qfl[ch]);
            }
            }
            if (!unsafe) {
#pragma unroll 1
                for (int kk = 0; kk < KC; kk += 2) {
                    stage(std::false_type{}, ch * KC + kk, rows_a, rows_b);
                    stage(std::false_type{}, ch * KC + kk + 1, rows_b, rows_a);
                }
            } else {
#pragma unroll 1
                for (int kk = 0; kk < KC; kk += 2) {
                    stage(std::true_type{}, ch * KC + kk, rows_a, rows_b);
                    stage(std::true_type{}, ch * KC + kk + 1, rows_b, rows_a);
                }
            }
        }
    }

    if (a.nsplit > 1) {
        // a slice's sums go to the workspace whole (padding rows and columns included: zeros);
        // the fixed-order reduction kernel adds the slices and applies the epilogue
        const int64_t prows = (int64_t)a.X * TILE_ROWS;
        float *part = a.partial + (((size_t)blockIdx.z * gridDim.y + bz) * prows + row0) * a.Jp + j0;
#pragma unroll
        for (int rr = 0; rr < RPT; ++rr) {
            float4 *o4 = reinterpret_cast<float4 *>(part + (size_t)(rr * WIDE_THREADS + tid) * a.Jp);
#pragma unroll
            for (int j = 0; j < WIDE_TN / 4; ++j)
                o4[j] = make_float4(acc[rr][4 * j], acc[rr][4 * j + 1], acc[rr][4 * j + 2], acc[rr][4 * j + 3]);
        }
        return;
    }
#pragma unroll
    for (int rr = 0; rr < RPT; ++rr) {
        const int64_t r = row0 + rr * WIDE_THREADS + tid;
        if (r >= a.R) continue;
        float *o = a.out + (int64_t)bz * a.out_batch_stride + out_row_offset(a.ep.omap, r, a.so_r);
        if (a.ep.bias_j || a.ep.bias_r || a.ep.act) {
#pragma unroll
            for (int j = 0; j < WIDE_TN; ++j) acc[rr][j] = apply_epilogue(a.ep, acc[rr][j], r, min((int64_t)(j0 + j), a.J - 1));
        }
        if (a.vec_store && j0 + WIDE_TN <= a.J) {
            float4 *o4 = reinterpret_cast<float4 *>(o + j0);
#pragma unroll
            for (int j = 0; j < WIDE_TN / 4; ++j)
                o4[j] = make_float4(acc[rr][4 * j], acc[rr][4 * j + 1], acc[rr][4 * j + 2], acc[rr][4 * j + 3]);
        } else {
#pragma unroll
            for (int j = 0; j < WIDE_TN; ++j)
                if (j0 + j < a.J) o[(int64_t)(j0 + j) * a.so_j] = acc[rr][j];
        }
    }
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
// Rows of the transposed operand: whole tiles of the height the problem will run with (problems of up
// to 2048 rows are one tile of 1024 or 2048 rows, so that filter gradients -- a few hundred to a few
// thousand filter elements over the lanes -- do not pad to 4096).
inline int64_t padded_rows(int64_t R)
{
    if (R <= WIDE_TILE_ROWS / 4) return WIDE_TILE_ROWS / 4;
    if (R <= WIDE_TILE_ROWS / 2) return WIDE_TILE_ROWS / 2;
    return (R + WIDE_TILE_ROWS - 1) / WIDE_TILE_ROWS * WIDE_TILE_ROWS;
}

// How a problem is cut: tile height, and the reduction into nsplit slices of whole chunks when the
// tiles alone would leave half or more of the workgroup slots (two per compute unit) empty and slices
// are allowed.
struct WidePlan {
    int tile_rows, nsplit, chunks_per_split;
    int64_t Rp, X, strips, nchunks;
    size_t pt_bytes, flag_bytes, partial_bytes;
};
// planar_pixels > 0: the lane operand is a convolution's source read from its channel-major copy
// (planar_channels planes of that many pixels) instead of an im2col of K x Rp words
WidePlan wide_plan(int64_t R, int64_t J, int64_t K, int batch, bool may_split, int cus, int64_t planar_pixels = 0,
                   int planar_channels = 0)
{
    WidePlan pl{};
    pl.Rp = padded_rows(R);
    pl.nchunks = (K + KC - 1) / KC;
    pl.strips = (J + QT - 1) / QT * (QT / WIDE_TN);
    const int64_t slots = 2 * (int64_t)cus;
    pl.tile_rows = (int)std::min<int64_t>(pl.Rp, WIDE_TILE_ROWS);
    pl.nsplit = 1;
    pl.chunks_per_split = (int)pl.nchunks;
    // Problems taller than one tile: full-height tiles (1 byte of table row pulled per product, + 0.5 of
    // lane operand) or half-height ones (2 + 0.5), and the reduction whole or in slices of at least 4
    // chunks (128 stages: shorter ones do not pay for their partial sums).  What bounds the kernel is the
    // bytes pulled from L2, shared by the resident workgroups (two per compute unit; a workgroup with a
    // compute unit to itself gets about 1.5 shares), in rounds of as many workgroups as fit; slices add
    // the write + re-read of their partial sums and the reduction launch.  The cheapest combination wins.
    const bool tall = pl.tile_rows == WIDE_TILE_ROWS;
    if (tall) {
        const double pull = 13.5e12, partial_rate = 3.0e12, launch_s = 8.0e-6;
        const int64_t Jp = pl.strips * WIDE_TN;
        double best = 0;
        for (int rows : {WIDE_TILE_ROWS, WIDE_TILE_ROWS / 2}) {
            const int64_t X = (R + rows - 1) / rows, tiles = X * pl.strips * batch;
            const double bytes_per_product = (double)WIDE_TILE_ROWS / rows + 0.5;
            const int64_t smax = may_split ? std::max<int64_t>(1, std::min<int64_t>(pl.nchunks / 4, 65535)) : 1;
            for (int64_t want = 1; want <= smax; ++want) {
                const int64_t cps = (pl.nchunks + want - 1) / want, ns = (pl.nchunks + cps - 1) / cps;
                if (ns != want) continue;
                const int64_t wgs = tiles * ns, rounds = (wgs + slots - 1) / slots;
                const double share = pull / (double)std::max<int64_t>(std::min(wgs, slots), slots * 2 / 3);
                double t = (double)rounds * cps * KC * rows * WIDE_TN * bytes_per_product / share;
                if (ns > 1) t += 2.0 * ns * (double)batch * X * rows * Jp * sizeof(float) / partial_rate + launch_s;
                if (best == 0 || t < best) { best = t; pl.tile_rows = rows; pl.nsplit = (int)ns; pl.chunks_per_split = (int)cps; }
            }
        }
    }
    pl.X = (R + pl.tile_rows - 1) / pl.tile_rows;
    const int64_t tiles = pl.X * pl.strips * batch;
    // one short tile (filter gradients: a few hundred to a few thousand rows, a very long reduction):
    // slices when the tiles alone leave half or more of the slots empty
    if (!tall && may_split && 2 * tiles <= slots && pl.nchunks >= 16) {
        const int64_t want = std::min<int64_t>(pl.nchunks / 4, std::min<int64_t>((slots + tiles - 1) / tiles, 65535));
        pl.chunks_per_split = (int)((pl.nchunks + want - 1) / want);
        pl.nsplit = (int)((pl.nchunks + pl.chunks_per_split - 1) / pl.chunks_per_split);
    }
    pl.pt_bytes = align256((size_t)batch * pl.nchunks * KC * pl.Rp * sizeof(uint32_t));
    pl.flag_bytes = align256((size_t)batch * pl.nchunks * (pl.Rp / PT_ROWS) * sizeof(uint32_t));
    if (planar_pixels > 0) {
        const int64_t pixp = (planar_pixels + PT_ROWS - 1) / PT_ROWS * PT_ROWS, cch = (planar_channels + KC - 1) / KC;
        pl.pt_bytes = align256((size_t)cch * KC * pixp * sizeof(uint32_t));
        pl.flag_bytes = align256((size_t)cch * (pixp / PT_ROWS) * sizeof(uint32_t));
    }
    const int64_t Jp = pl.strips * WIDE_TN;
    pl.partial_bytes = pl.nsplit > 1 ? align256((size_t)pl.nsplit * batch * pl.X * pl.tile_rows * Jp * sizeof(float)) : 0;
    return pl;
}

template <int RPT>
void launch_wide(const WArgs &wa, dim3 grid, int m, bool planar, hipStream_t stream)
{
    if (planar) {
        if (m >= 11) lutgemm_wide_kernel<2, RPT, true><<<grid, WIDE_THREADS, 0, stream>>>(wa);
        else lutgemm_wide_kernel<1, RPT, true><<<grid, WIDE_THREADS, 0, stream>>>(wa);
    } else {
        if (m >= 11) lutgemm_wide_kernel<2, RPT, false><<<grid, WIDE_THREADS, 0, stream>>>(wa);
        else lutgemm_wide_kernel<1, RPT, false><<<grid, WIDE_THREADS, 0, stream>>>(wa);
    }
}

// A convolution's patches can be read from a channel-major, zero-bordered copy of its source when
// the whole copy stays below 2^31 bytes (one buffer resource addresses it) and the batch is folded
// into the rows (the convolution entry points do that).  Returns the pixels of one channel plane, 0 if
// the form does not apply.
struct Planar { int ph, pw; int64_t pixels; };
Planar planar_of(const GemmDesc &d)
{
    Planar pn{0, 0, 0};
    if (d.p.kind != P_PATCH || d.batch != 1 || d.p.KH < 1 || d.p.KW < 1 || d.p.GH < 1 || d.p.GW < 1 || d.p.C < 1) return pn;
    if (d.K != (int64_t)d.p.KH * d.p.KW * d.p.C) return pn;
    const int64_t ph = (int64_t)(d.p.GH - 1) * d.p.sy + d.p.KH, pw = (int64_t)(d.p.GW - 1) * d.p.sx + d.p.KW;
    const int64_t pixels = (int64_t)d.p.B * ph * pw, pixp = (pixels + PT_ROWS - 1) / PT_ROWS * PT_ROWS;
    const int64_t cp = (int64_t)((d.p.C + KC - 1) / KC) * KC;
    if (ph >= (1 << 20) || pw >= (1 << 20) || pixp * cp * 4 >= (1ll << 31) - 4096) return pn;
    pn.ph = (int)ph; pn.pw = (int)pw; pn.pixels = pixels;
    return pn;
}
inline int64_t planar_pixels(const GemmDesc &d) { return planar_of(d).pixels; }

}  // namespace

bool wide_shape_eligible(int64_t R, int batch) { return batch >= 1 && batch <= 65535 && R >= WIDE_MIN_ROWS; }

// Dense, patch (forward / input-gradient convolution) and filter-gradient lane operands.  A problem
// that would run on a handful of workgroups because its reduction may not be sliced (a filter
// gradient in whole-reduction mode: few rows, very long reduction) is left to the global-gather
// variant, which at least fills the machine.
bool wide_eligible(int m, const GemmDesc &d, bool may_split)
{
    if (m <= 7 || !wide_shape_eligible(d.R, d.batch)) return false;
    const int cus = device_compute_units();
    const WidePlan pl = wide_plan(d.R, d.J, d.K, d.batch, may_split, cus);
    const int64_t wgs = pl.X * pl.strips * d.batch * pl.nsplit;
    return wgs * 8 >= cus || pl.nchunks <= 64;
}

size_t wide_workspace_bytes(int64_t R, int64_t J, int64_t K, int batch)
{
    // the larger of what a sliced and a whole reduction ask for, on any device size
    size_t need = 0;
    for (int cus : {device_compute_units(), 256, 304})
        for (bool split : {false, true}) {
            const WidePlan pl = wide_plan(R, J, K, batch, split, cus);
            need = std::max(need, pl.pt_bytes + pl.flag_bytes + pl.partial_bytes);
        }
    return need;
}

size_t wide_workspace_bytes_planar(const GemmDesc &d)
{
    const int64_t pixels = planar_pixels(d);
    if (pixels == 0) return 0;
    size_t need = 0;
    for (int cus : {device_compute_units(), 256, 304})
        for (bool split : {false, true}) {
            const WidePlan pl = wide_plan(d.R, d.J, d.K, d.batch, split, cus, pixels, d.p.C);
            need = std::max(need, pl.pt_bytes + pl.flag_bytes + pl.partial_bytes);
        }
    return need;
}

int run_gemm_wide(const Lut &lut, const GemmDesc &d, const WideQ &q, void *wide_ws, bool planar, bool may_split, hipStream_t stream)
{
    const int64_t pixels = planar ? planar_pixels(d) : 0;
    const WidePlan pl = wide_plan(d.R, d.J, d.K, d.batch, may_split, device_compute_units(), pixels, d.p.C);
    const int64_t Rp = pl.Rp;
    uint8_t *ws = static_cast<uint8_t *>(wide_ws);
    PTArgs pa{};
    pa.pt = reinterpret_cast<uint32_t *>(ws);
    pa.pflags = reinterpret_cast<uint32_t *>(ws + pl.pt_bytes);
    int64_t pwgs;
    const Planar pn = planar_of(d);
    if (pixels > 0) {
        // the zero-bordered source as a [padded pixel][channel] matrix, transposed into channel planes:
        // a 1x1 "convolution" over the padded extent reads source pixel (py - pad_top, px - pad_left), zero outside
        pa.p = PDesc{};
        pa.p.kind = P_PATCH; pa.p.base = d.p.base;
        pa.p.B = d.p.B; pa.p.GH = pn.ph; pa.p.GW = pn.pw; pa.p.KH = 1; pa.p.KW = 1; pa.p.C = d.p.C;
        pa.p.sy = 1; pa.p.sx = 1; pa.p.pt = d.p.pt; pa.p.pl = d.p.pl; pa.p.SH = d.p.SH; pa.p.SW = d.p.SW;
        pa.R = pixels; pa.K = d.p.C;
        pa.Rp = (pixels + PT_ROWS - 1) / PT_ROWS * PT_ROWS;
        pa.nchunks = (d.p.C + KC - 1) / KC;
        pwgs = (pa.Rp / PT_ROWS) * pa.nchunks;
    } else {
        pa.p = d.p; pa.R = d.R; pa.K = d.K; pa.Rp = Rp; pa.nchunks = q.nchunks;
        pwgs = (Rp / PT_ROWS) * q.nchunks;
    }
    if (pwgs >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "lane operand exceeds the grid limit");
    p_linear_kernel<<<dim3((unsigned)pwgs, (unsigned)d.batch), WG_THREADS, 0, stream>>>(pa);
    AMSIM_HIP_CHECK(hipGetLastError());

    WArgs wa{};
    wa.pt = pa.pt; wa.pflags = pa.pflags;
    wa.lut16 = reinterpret_cast<const uint8_t *>(d.lane_first ? lut.img16_ba : lut.img16_ab);
    wa.qw = q.qw; wa.qflags = q.qflags; wa.qdesc = q.qdesc;
    wa.m = lut.m; wa.lane_first = d.lane_first ? 1 : 0;
    wa.R = d.R; wa.J = d.J; wa.K = d.K; wa.Rp = Rp;
    wa.Jp = q.Jp; wa.nchunks = q.nchunks;
    wa.out = d.out; wa.so_r = d.so_r; wa.so_j = d.so_j; wa.out_batch_stride = d.out_batch_stride;
    wa.vec_store = (d.so_j == 1 && d.so_r % 4 == 0 && d.out_batch_stride % 4 == 0 && ((uintptr_t)d.out & 15) == 0) ? 1 : 0;
    wa.q_batches = d.q.batches;
    wa.ep = Epilogue{d.bias_j, d.bias_r, d.act, d.omap};
    wa.X = (unsigned)pl.X;
    wa.Y = (unsigned)(q.Jp / WIDE_TN);
    wa.nsplit = pl.nsplit;
    wa.chunks_per_split = pl.chunks_per_split;
    wa.partial = reinterpret_cast<float *>(ws + pl.pt_bytes + pl.flag_bytes);
    wa.p = d.p;
    wa.plane_elems = pixels > 0 ? pa.Rp : 0;
    wa.ph = pn.ph; wa.pw = pn.pw;
    wa.cchunks = pixels > 0 ? pa.nchunks : 0;
    const int64_t total = (int64_t)wa.X * wa.Y;
    if (total >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "workgroup count exceeds the grid limit");
    const dim3 grid((unsigned)total, (unsigned)d.batch, (unsigned)pl.nsplit);
    switch (pl.tile_rows / WIDE_THREADS) {
    case 8: launch_wide<8>(wa, grid, lut.m, pixels > 0, stream); break;
    case 4: launch_wide<4>(wa, grid, lut.m, pixels > 0, stream); break;
    default: launch_wide<2>(wa, grid, lut.m, pixels > 0, stream); break;
    }
    AMSIM_HIP_CHECK(hipGetLastError());
    if (pl.nsplit > 1) {
        RArgs ra{wa.partial, d.out, d.R, d.J, pl.X * pl.tile_rows, d.so_r, d.so_j, d.out_batch_stride, q.Jp, pl.nsplit,
                 d.batch, 0, wa.ep};
        launch_reduce(ra, stream);
        AMSIM_HIP_CHECK(hipGetLastError());
    }
    return AMSIM_OK;
}

}  // namespace amsim
