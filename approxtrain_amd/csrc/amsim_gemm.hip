// LUT-multiply GEMM engine for gfx950 (MI355X).
//
// out(r, j) = sum_k P(p(r, k), q(k, j)),  P = approximate product through a
// mantissa LUT, FP32 accumulation in ascending k.
//
// Mapping to the machine (VALU/LDS-bound by construction; no MFMA because the
// product is not an IEEE multiply):
//   * r runs over the 64 lanes of a wavefront, j is wave-uniform.  At every
//     LUT gather all lanes share the uniform operand's mantissa, so the 64
//     addresses fall into ONE 2^m-byte row of the byte-wide LUT image in LDS:
//     at most 32 distinct dwords, one per bank -> no bank conflicts ever.
//   * the uniform operand q is pre-decoded once per call into one word per
//     element (sign|exponent in the top 9 bits, LUT row offset in the low 16)
//     laid out in 16-column tiles, and read through the scalar cache (s_load)
//     four reduction rows at a time, so it costs no VALU and no LDS and the
//     scalar-memory latency is paid once per 4 x TN MACs per lane.
//   * the lane operand p is staged through LDS by coalesced (float4 where the
//     source allows) loads -- dense, im2col-style patches, or filter-gradient
//     gathers computed on the fly: no im2col / flipped-filter temporaries in
//     HBM -- in a [k/4][r][4] layout that a lane reads back 16 bytes at a time.
//   * per pair of MACs: one v_lshl_add_u64 (two LUT addresses: the lane's
//     mantissa index in both halves + a pair of row offsets), two
//     ds_read_u8_d16_hi (the LUT byte lands in the upper register half, i.e.
//     shifted into the mantissa/carry position), one v_lshl_add_u64 (the two
//     gathered registers PLUS the uniform operand's sign|exponent bits of both
//     columns = q_pow2 * 1.mant * 2^carry as two floats), two v_fma with the
//     lane operand's power of two (accumulate).  The product inside the fma is
//     exact (power of two times an 8-bit significand), so the fused
//     multiply-add rounds exactly like the reference's product-then-add.
//     Zero uniform operands select an all-zero LUT row, zero lane operands a
//     zero multiplier: no zero test in the loop.
//   * operands outside the "safe" range (subnormal, inf, NaN, |x| < 2^-63 or
//     >= 2^64) flag their 32-deep k chunk; flagged chunks take the exact
//     full-domain product instead (wave-uniform branch), so results are
//     bit-exact everywhere without taxing the fast path.
#include "amsim_internal.h"
#include "amsim_device.h"
#include "amsim_gemm_common.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>

namespace amsim {

static std::atomic<int> g_split_k{1};
static std::atomic<int> g_engine{AMSIM_ENGINE_AUTO};

// staging modes of the lane operand
enum { STAGE_R = 0,   // threads run along r, one element each (source contiguous in r)
       STAGE_K = 1,   // threads run along k, one element each
       STAGE_K4 = 2 };// threads run along k, four consecutive k per 16-byte load

struct KArgs {
    PDesc p;
    const uint8_t *lut_img;  // LUT image indexed (uniform mantissa << m) | lane mantissa: bytes, or uint16 for m > 7
    int lut_bytes;
    int m;
    int lane_first;
    const uint32_t *qw;      // [qb][Jp/16][Kp][16]  sign|exponent | row offset
    const QDesc *qdesc;      // the uniform operand where it lies (a copy of its descriptor in device memory, written
                             // by the pre-pass): flagged chunks read its raw bits from there.  Kept behind a pointer
                             // so that its fields are loaded inside the rare path only and cost the inner loop no
                             // scalar registers.
    const uint32_t *qflags;  // [qb][Jp/16][nchunks] operand spans
    int q_batches;
    int64_t R, J, K;
    int Jp, nchunks;
    float *out;
    int64_t so_r, so_j, out_batch_stride;
    int batch;
    int vec_store;           // outputs of a row are contiguous (so_j == 1) and every row starts 16-byte aligned
    int d16_keeps;           // this device's 16-bit LDS loads keep the register half they do not write (Lut::d16_keeps)
    Epilogue ep;
    // A launch covers up to two row segments, workgroups of seg[0] first in dispatch order:
    // seg[0] the split-reduction tail (if any), seg[1] the main part.
    struct Seg {
        int64_t row_base, Rp;        // first row, padded row count
        float *partial;              // [nsplit][batch][Rp][Jp] when nsplit > 1 (rows relative to row_base)
        int nsplit, chunks_per_split;
        unsigned X, Y, Z;            // row tiles, column groups, batch x splits
        unsigned total;              // X * Y * Z
    } seg[2];
};

// ---------------------------------------------------------------------------
// uniform-operand pre-pass
// ---------------------------------------------------------------------------
// One wavefront per (32-row chunk, 16-column tile): decodes the tile, writes it
// in the tile-major layout the main kernel streams, and records the tile-chunk's
// operand span (exponent range, special values: amsim_device.h).  blockIdx.x runs over
// (chunk, group of four column tiles), blockIdx.y over the batch.
__global__ __launch_bounds__(WG_THREADS) void q_prepass_kernel(QArgs a)
{
    const int ntiles = a.Jp / QT;
    const int tgroups = (ntiles + WG_THREADS / 64 - 1) / (WG_THREADS / 64);
    const int ch = blockIdx.x / tgroups, qb = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int jt = (blockIdx.x % tgroups) * (WG_THREADS / 64) + (threadIdx.x >> 6);
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *a.qdesc_out = a.q;
    if (jt >= ntiles) return;
    const float *base = a.q.base + (int64_t)qb * a.q.batch_stride;
    const size_t Kp = (size_t)a.nchunks * KC;
    const size_t tile = ((size_t)qb * ntiles + jt) * Kp * QT + (size_t)ch * KC * QT;
    uint32_t *qw = a.qw + tile;
    // Lanes follow the source's contiguous direction when reading.  A source that is contiguous
    // along k would then be written with a 64-byte stride between lanes: its decoded words take a
    // turn through LDS instead, so that every store covers consecutive words of the tile.
    const bool k_fast = (a.q.kind == Q_DENSE && a.q.sk == 1 && a.q.sj != 1) || (a.q.kind == Q_FLIP);
    __shared__ uint32_t turn[WG_THREADS / 64][KC][QT + 1];
    const int w = threadIdx.x >> 6;
    SafeRange range;
    // all of a lane's elements are fetched before the first is decoded and stored: the stores cannot be
    // proven not to alias the source, so loads left between them would wait for one another
    constexpr int PER_LANE = KC * QT / 64;
    uint32_t raws[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int e = lane + 64 * i;
        int kk, jj;
        if (k_fast) { kk = e % KC; jj = e / KC; }
        else { jj = e % QT; kk = e / QT; }
        raws[i] = q_raw_bits(a.q, base, (uint32_t)a.K, (uint32_t)a.J, (uint32_t)ch * KC + kk, (uint32_t)jt * QT + jj);
    }
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int e = lane + 64 * i;
        int kk, jj;
        if (k_fast) { kk = e % KC; jj = e / KC; }
        else { jj = e % QT; kk = e / QT; }
        const uint32_t raw = raws[i];
        range.add(raw);
        // zero (and padding) elements select the all-zero LUT row that follows the table:
        // their product term is then exactly +-0 without a test in the inner loop
        const uint32_t mant = (raw & 0x7fffffffu) ? ((raw & 0x7fffffu) >> (23 - a.m)) : (1u << a.m);
        const uint32_t word = (raw & 0xff800000u) | (mant << a.m);
        if (k_fast) turn[w][kk][jj] = word;
        else qw[e] = word;  // e == kk * QT + jj
    }
    if (k_fast) {
        // (the wavefront reads back what it wrote itself: LDS operations of one wavefront stay in order)
#pragma unroll
        for (int i = 0; i < KC * QT / 64; ++i) {
            const int e = lane + 64 * i;
            qw[e] = turn[w][e / QT][e % QT];
        }
    }
    // the tile-chunk's span: top bit = "an operand fails the quick test", below it the exponent range
    const uint32_t span = span_word(wave_union(range));
    if (lane == 0) a.qflags[((size_t)qb * ntiles + jt) * a.nchunks + ch] = span;
}

int launch_q_prepass(const QArgs &qa, int q_batches, hipStream_t stream)
{
    if (q_batches > 65535) return fail(AMSIM_ERR_UNSUPPORTED, "batch exceeds the grid limit");
    const int64_t wgs = (int64_t)qa.nchunks * ((qa.Jp / QT + 3) / 4);
    if (wgs >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "uniform operand exceeds the grid limit");
    q_prepass_kernel<<<dim3((unsigned)wgs, (unsigned)q_batches), WG_THREADS, 0, stream>>>(qa);
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

// ---------------------------------------------------------------------------
// lane-operand row bookkeeping, kept in LDS: one int4 per local row.
//   P_PATCH: {source offset of image b, y*sy - pt, x*sx - pl, source offset of the
//            window origin}; rows past the end get a y origin
//            far outside the source.
//   P_GF:    {(fy*SW + fx)*C + c, fy, fx, 0}; rows past the end get fy far outside.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void fill_rowinfo(const PDesc &p, int64_t R, int64_t row0, int rows, int4 *ri)
{
    for (int rl = threadIdx.x; rl < rows; rl += WG_THREADS) {
        const int64_t r = row0 + rl;
        int4 v = make_int4(0, -(1 << 28), 0, 0);
        if (r < R) {
            if (p.kind == P_PATCH) {
                // (row counts stay below 2^31: 32-bit divisions, a fraction of the 64-bit ones' instructions)
                const uint32_t r32 = (uint32_t)r, gw = (uint32_t)p.GW, gh = (uint32_t)p.GH;
                const int x = (int)(r32 % gw);
                const uint32_t t = r32 / gw;
                const int y = (int)(t % gh);
                const int b = (int)(t / gh);
                const int vy0 = y * p.sy - p.pt, vx0 = x * p.sx - p.pl;
                v = make_int4(b * p.SH * p.SW * p.C, vy0, vx0, (b * p.SH * p.SW + vy0 * p.SW + vx0) * p.C);
            } else if (p.kind == P_GF) {
                const int c = (int)((uint32_t)r % (uint32_t)p.C);
                const int t = (int)((uint32_t)r / (uint32_t)p.C);
                const int fx = t % p.KW, fy = t / p.KW;
                v = make_int4((fy * p.SW + fx) * p.C + c, fy, fx, 0);
            }
        }
        ri[rl] = v;
    }
}

// ---------------------------------------------------------------------------
// main kernel
// ---------------------------------------------------------------------------
// TN     outputs per lane (uniform-dimension tile of one wave)
// WR     row tiles per workgroup (waves are arranged WR x 4/WR); 0: one row tile, one column group,
//        the reduction rows of every chunk dealt out to the four waves (split reductions only)
// PK     lane-operand source (PKind)
// STAGE  how the staging threads walk the tile (STAGE_*)
// LUTG   false: byte LUT image resident in LDS (mantissa width <= 7)
//        true:  16-bit LUT image gathered from global memory through L2 / MALL
//               (widths 8..11; a 2^22-entry table does not fit the 160 KB LDS)
#ifndef AMSIM_D16
#define AMSIM_D16 1
#endif
#ifndef AMSIM_D16_PU
#define AMSIM_D16_PU 4
#endif
constexpr int WR_KSLICES = 0;  // value of WR that selects the reduction-slice arrangement

template <int TN, int WR, int PK, int STAGE, bool LUTG>
__global__ __launch_bounds__(WG_THREADS, (WR > 1 ? 2 : (PK == P_DENSE && STAGE != STAGE_K4) ? WAVES_PER_SIMD - 1 : WAVES_PER_SIMD))
void lutgemm_kernel(KArgs a)
{
    // WR == 0 (WR_KSLICES): one row tile, one column group, and the four wavefronts take a quarter of
    // every chunk's reduction rows each; their sums are added through LDS at the end, in wavefront order
    constexpr bool KSLICES = WR == WR_KSLICES;
    constexpr int WC = KSLICES ? 1 : 4 / (KSLICES ? 1 : WR);
    constexpr int ROWS = KSLICES ? 64 : 64 * WR;
    constexpr int GS = ROWS + 1;  // padded group stride (in uint4): conflict-free transposing stores
    constexpr int ELEMS = ROWS * KC / WG_THREADS;
    constexpr int QUADS = ELEMS / 4;
    constexpr bool D16_LOOP = AMSIM_D16 && !LUTG && TN % 2 == 0;  // the hand-ordered inner loop (below)

    __shared__ __align__(16) uint8_t lut_s[LUTG ? (KSLICES ? 3 * TN * 64 * sizeof(float) : 16) : LUT_LDS_BYTES];
    const uint16_t *__restrict__ lut_g = reinterpret_cast<const uint16_t *>(a.lut_img);
    constexpr int ESHIFT = LUTG ? 8 : 16;  // LUT entry -> carry << 23 | mantissa
    __shared__ uint4 Pt4[NG * GS];
    __shared__ int4 rowinfo[PK == P_DENSE ? 1 : ROWS];
    __shared__ uint32_t pflag[2];  // "this chunk's staged tile holds an unsafe operand", by chunk parity

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = KSLICES ? 0 : wave / WC, wc = KSLICES ? 0 : wave % WC;
    const int g_first = KSLICES ? wave * (NG / 4) : 0, g_last = KSLICES ? g_first + NG / 4 : NG;  // this wavefront's reduction-row groups of a chunk
    // Workgroups are handed to the 8 XCDs round-robin in launch order, and each
    // XCD has its own L2.  Renumber so that each XCD works on a contiguous run
    // of tiles (row tile fastest, then column group, then split / batch): the
    // workgroups that share uniform-operand tiles and input rows then share an L2.
    const bool in_first = blockIdx.x < a.seg[0].total;
    const int64_t seg_row_base = in_first ? a.seg[0].row_base : a.seg[1].row_base;
    const int64_t seg_Rp = in_first ? a.seg[0].Rp : a.seg[1].Rp;
    float *const seg_partial = in_first ? a.seg[0].partial : a.seg[1].partial;
    const int seg_nsplit = in_first ? a.seg[0].nsplit : a.seg[1].nsplit;
    const int seg_cps = in_first ? a.seg[0].chunks_per_split : a.seg[1].chunks_per_split;
    unsigned bx, by, bzz;
    {
        const unsigned X = in_first ? a.seg[0].X : a.seg[1].X, Y = in_first ? a.seg[0].Y : a.seg[1].Y;
        const unsigned T = in_first ? a.seg[0].total : a.seg[1].total;
        const unsigned L = in_first ? blockIdx.x : blockIdx.x - a.seg[0].total;
        const unsigned xcd = L % NUM_XCD, idx = L / NUM_XCD;
        const unsigned chunk = T / NUM_XCD, rem = T % NUM_XCD;
        const unsigned V = xcd * chunk + (xcd < rem ? xcd : rem) + idx;
        bx = V % X;
        by = (V / X) % Y;
        bzz = V / (X * Y);
    }
    const int bz = bzz / seg_nsplit, split = bzz % seg_nsplit;
    const int64_t row0 = seg_row_base + (int64_t)bx * ROWS;
    const int j0 = (by * WC + wc) * TN;
    const bool active = j0 < a.J;
    const int m = a.m;

    if (!LUTG) {
        // The LUT image goes from global memory straight into LDS, 16 bytes per lane and
        // instruction, without passing through registers: the copies are only started here and
        // are waited for together with the first chunk's reads, so a workgroup's start costs
        // one memory latency instead of one per round of the copy.
        constexpr int NVEC = LUT_LDS_BYTES / 16;
#pragma unroll
        for (int i = 0; i * WG_THREADS < NVEC; ++i) {
#if defined(__HIP_DEVICE_COMPILE__)  // the builtin exists in the device pass only
            const int v0 = i * WG_THREADS + wave * 64;  // first vector of this wave's 1 KB slice
            if ((v0 + lane) * 16 < a.lut_bytes)
                __builtin_amdgcn_global_load_lds(a.lut_img + (v0 + lane) * 16, lut_s + v0 * 16, 16, 0, 0);
#endif
        }
    }
    if (PK != P_DENSE) fill_rowinfo(a.p, a.R, row0, ROWS, rowinfo);
    if (tid < 2) pflag[tid] = 0u;
    __syncthreads();

    const float *pbase = a.p.base + (int64_t)bz * a.p.batch_stride;
    const int qb = a.q_batches > 1 ? bz : 0;
    const size_t Kp = (size_t)a.nchunks * KC;
    // The pre-decoded uniform operand was written by an earlier kernel and is
    // read-only here: address it through the constant address space so that the
    // wave-uniform reads become scalar loads (s_load) into SGPRs.
    const size_t qtile = ((size_t)qb * (a.Jp / QT) + (size_t)(j0 / QT)) * Kp * QT + (size_t)(j0 % QT);
    const cq1_t qw = (cq1_t)(uintptr_t)(a.qw + qtile);
    const cq1_t qflags = (cq1_t)(uintptr_t)(a.qflags + ((size_t)qb * (a.Jp / QT) + (size_t)(j0 / QT)) * a.nchunks);

    const int ch_begin = split * seg_cps;
    const int ch_end = min(a.nchunks, ch_begin + seg_cps);

    // Dense sources: one per-thread pointer to the first element this thread
    // stages, a uniform step between its successive elements, and a uniform
    // advance per chunk -- keeps the address arithmetic out of the scalar
    // registers the inner loop needs for the uniform operand.
    const float *dptr = nullptr;
    int64_t dstep = 0, dchunk = 0;
    int drow = 0, dvalid_rows = 0;
    if (PK == P_DENSE) {
        const int64_t left = a.R - row0;
        dvalid_rows = (int)(left < ROWS ? left : ROWS);
        if (STAGE == STAGE_K4) {
            drow = tid >> 3;
            dptr = pbase + (row0 + drow) * a.p.sr + (tid & (KC / 4 - 1)) * 4;
            dstep = (int64_t)(WG_THREADS / (KC / 4)) * a.p.sr;
            dchunk = KC;
        } else if (STAGE == STAGE_K) {
            drow = tid >> 5;
            dptr = pbase + (row0 + drow) * a.p.sr + (int64_t)(tid & (KC - 1)) * a.p.sk;
            dstep = (int64_t)(WG_THREADS / KC) * a.p.sr;
            dchunk = (int64_t)KC * a.p.sk;
        } else {
            drow = tid & (ROWS - 1);
            dptr = pbase + (row0 + drow) * a.p.sr + (int64_t)((tid / ROWS) * ELEMS) * a.p.sk;
            dstep = a.p.sk;
            dchunk = (int64_t)KC * a.p.sk;
        }
        // pin the walking state into vector registers
        asm volatile("" : "+v"(dstep), "+v"(dchunk));
        dptr += (int64_t)(split * seg_cps) * dchunk;
    }

    // Patch sources: (fy, fx, c) of the first k of the next chunk to stage, walked
    // chunk by chunk with scalar adds instead of being re-derived by division.
    int cb_c = 0, cb_fx = 0, cb_fy = 0;
    const bool patch_walk = PK == P_PATCH && a.p.C >= KC;
    if (patch_walk) {
        const uint32_t kb = (uint32_t)(split * seg_cps) * KC;
        cb_c = (int)(kb % (uint32_t)a.p.C);
        const int t = (int)(kb / (uint32_t)a.p.C);
        cb_fx = t % a.p.KW;
        cb_fy = t / a.p.KW;
    }
    auto decompose_k = [&](int64_t k, int koff, int &c, int &fx, int &fy) {
        if (patch_walk) {  // C >= KC: at most one wrap within a chunk
            c = cb_c + koff; fx = cb_fx; fy = cb_fy;
            if (c >= a.p.C) { c -= a.p.C; if (++fx == a.p.KW) { fx = 0; ++fy; } }
        } else {
            const uint32_t k32 = (uint32_t)k, c32 = (uint32_t)a.p.C;  // (k < 2^31)
            c = (int)(k32 % c32);
            const int t = (int)(k32 / c32);
            fx = t % a.p.KW; fy = t / a.p.KW;
        }
    };
    auto advance_chunk_base = [&]() {
        if (patch_walk) {
            cb_c += KC;
            if (cb_c >= a.p.C) { cb_c -= a.p.C; if (++cb_fx == a.p.KW) { cb_fx = 0; ++cb_fy; } }
        }
    };

    // Patch sources whose channel count is a multiple of the chunk depth: every
    // chunk lies inside one filter tap, so the tap offset and the window test are scalar work
    const bool tap_uniform = PK == P_PATCH && STAGE == STAGE_K4 && (a.p.C % KC == 0);

    // Filter-gradient tiles that lie inside one (fy, fx) (channel count a multiple of the tile
    // height, tile fully inside R): wave-uniform window offset
    const bool gf_uniform = PK == P_GF && (a.p.C % ROWS == 0) && row0 + ROWS <= a.R;
    int gf_fy = 0, gf_fx = 0, gf_c0 = 0;
    if (gf_uniform) {
        gf_c0 = (int)((uint32_t)row0 % (uint32_t)a.p.C);
        const int t = (int)((uint32_t)row0 / (uint32_t)a.p.C);
        gf_fx = t % a.p.KW;
        gf_fy = t / a.p.KW;
    }

    uint32_t pv[ELEMS];
    auto load_chunk = [&](int ch) {
        const int64_t k0 = (int64_t)ch * KC;
        if (STAGE == STAGE_K4) {
            // thread -> (row, quad of 4 consecutive k); all four share (fy, fx) because C % 4 == 0
            const int kq = (tid & (KC / 4 - 1)) * 4;
            const int64_t k = k0 + kq;
            const bool kvalid = k < a.K;  // K % 4 == 0 on this path
            int c = 0, fy = 0, fx = 0;
            if (PK == P_PATCH && !tap_uniform) decompose_k(k, kq, c, fx, fy);
            const int tapoff = (cb_fy * a.p.SW + cb_fx) * a.p.C + cb_c + kq;
#pragma unroll
            for (int i = 0; i < QUADS; ++i) {
                const int rl = (tid >> 3) + i * (WG_THREADS / (KC / 4));
                uint4 v = make_uint4(0, 0, 0, 0);
                if (PK == P_PATCH && tap_uniform) {
                    const int4 ri = rowinfo[rl];
                    if ((unsigned)(ri.y + cb_fy) < (unsigned)a.p.SH && (unsigned)(ri.z + cb_fx) < (unsigned)a.p.SW)
                        v = *reinterpret_cast<const uint4 *>(pbase + (ri.w + tapoff));
                } else if (PK == P_DENSE) {
                    // dptr walks this thread's first row; rows i*32 further down are dstep apart
                    if (kvalid && drow + i * (WG_THREADS / (KC / 4)) < dvalid_rows)
                        v = *reinterpret_cast<const uint4 *>(dptr + (int64_t)i * dstep);
                } else {
                    const int4 ri = rowinfo[rl];
                    const int vy = ri.y + fy, vx = ri.z + fx;
                    if (kvalid && (unsigned)vy < (unsigned)a.p.SH && (unsigned)vx < (unsigned)a.p.SW)
                        v = *reinterpret_cast<const uint4 *>(pbase + ri.x + (vy * a.p.SW + vx) * a.p.C + c);
                }
                pv[4 * i + 0] = v.x; pv[4 * i + 1] = v.y; pv[4 * i + 2] = v.z; pv[4 * i + 3] = v.w;
            }
            if (PK == P_DENSE) dptr += dchunk;
        } else if (PK == P_DENSE) {
#pragma unroll
            for (int i = 0; i < ELEMS; ++i) {
                uint32_t v = 0;
                if (STAGE == STAGE_K) {
                    if (k0 + (tid & (KC - 1)) < a.K && drow + i * (WG_THREADS / KC) < dvalid_rows)
                        v = f2u(dptr[(int64_t)i * dstep]);
                } else {
                    const int kk = (tid / ROWS) * ELEMS + i;
                    if (k0 + kk < a.K && drow < dvalid_rows) v = f2u(dptr[(int64_t)i * dstep]);
                }
                pv[i] = v;
            }
            dptr += dchunk;
        } else if (PK == P_PATCH) {  // STAGE_K: this thread's k is fixed for the chunk
            const int kk = tid & (KC - 1);
            const int64_t k = k0 + kk;
            const bool kvalid = k < a.K;
            int c, fx, fy;
            decompose_k(k, kk, c, fx, fy);
#pragma unroll
            for (int i = 0; i < ELEMS; ++i) {
                const int rl = (tid >> 5) + i * (WG_THREADS / KC);
                const int4 ri = rowinfo[rl];
                const int vy = ri.y + fy, vx = ri.z + fx;
                uint32_t v = 0;
                if (kvalid && (unsigned)vy < (unsigned)a.p.SH && (unsigned)vx < (unsigned)a.p.SW)
                    v = f2u(pbase[ri.x + (vy * a.p.SW + vx) * a.p.C + c]);
                pv[i] = v;
            }
        } else {  // P_GF, staged along r: this thread stages ELEMS consecutive k (pixels) of its row
            const int rl = tid & (ROWS - 1);
            const int4 ri = rowinfo[rl];
            // the first pixel of this wave's run, decomposed once (wave-uniform), then walked
            const int64_t kfirst = k0 + __builtin_amdgcn_readfirstlane(tid / ROWS) * ELEMS;
            // (the reduction is shorter than 2^31: 32-bit divisions, a fraction of the 64-bit ones' instructions)
            const uint32_t kf32 = (uint32_t)kfirst, gw32 = (uint32_t)a.p.GW, gh32 = (uint32_t)a.p.GH;
            int x = (int)(kf32 % gw32);
            const uint32_t t = kf32 / gw32;
            int y = (int)(t % gh32);
            int b = (int)(t / gh32);
            if (gf_uniform) {
                // all rows of the tile share (fy, fx): the pixel walk, the window test and the
                // pixel's source offset are wave-uniform and stay in scalar registers; a lane
                // only adds its channel
                x = __builtin_amdgcn_readfirstlane(x);
                y = __builtin_amdgcn_readfirstlane(y);
                b = __builtin_amdgcn_readfirstlane(b);
                int iy = y * a.p.sy - a.p.pt + gf_fy, ix = x * a.p.sx - a.p.pl + gf_fx;
                int soff = ((b * a.p.SH + iy) * a.p.SW + ix) * a.p.C + gf_c0;
                const int step = a.p.sx * a.p.C;
                const uint32_t chan = (uint32_t)rl;
                const int64_t kleft64 = a.K - kfirst;
                const int kleft = kleft64 < ELEMS ? (int)kleft64 : ELEMS;  // elements of this run inside K
                if (a.p.GW % ELEMS == 0) {
                    // runs start at multiples of ELEMS, so one never leaves its output row: (b, y)
                    // and the source row are fixed, only the column advances
                    const bool row_ok = (unsigned)iy < (unsigned)a.p.SH;
#pragma unroll
                    for (int i = 0; i < ELEMS; ++i) {
                        uint32_t v = 0;
                        if (i < kleft && row_ok && (unsigned)ix < (unsigned)a.p.SW) v = f2u((pbase + soff)[chan]);
                        pv[i] = v;
                        ix += a.p.sx;
                        soff += step;
                    }
                } else
#pragma unroll
                for (int i = 0; i < ELEMS; ++i) {
                    uint32_t v = 0;
                    if (i < kleft && (unsigned)iy < (unsigned)a.p.SH && (unsigned)ix < (unsigned)a.p.SW)
                        v = f2u((pbase + soff)[chan]);
                    pv[i] = v;
                    if (++x == a.p.GW) {
                        x = 0;
                        if (++y == a.p.GH) { y = 0; ++b; }
                        iy = y * a.p.sy - a.p.pt + gf_fy;
                        ix = gf_fx - a.p.pl;
                        soff = ((b * a.p.SH + iy) * a.p.SW + ix) * a.p.C + gf_c0;
                    } else {
                        ix += a.p.sx;
                        soff += step;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < ELEMS; ++i) {
                    uint32_t v = 0;
                    if (kfirst + i < a.K) {
                        const int iy0 = y * a.p.sy - a.p.pt, ix0 = x * a.p.sx - a.p.pl;
                        const int iy = iy0 + ri.y, ix = ix0 + ri.z;
                        if ((unsigned)iy < (unsigned)a.p.SH && (unsigned)ix < (unsigned)a.p.SW)
                            v = f2u(pbase[((b * a.p.SH + iy0) * a.p.SW + ix0) * a.p.C + ri.x]);
                    }
                    pv[i] = v;
                    if (++x == a.p.GW) { x = 0; if (++y == a.p.GH) { y = 0; ++b; } }
                }
            }
        }
        if (PK == P_PATCH) advance_chunk_base();
    };
    // Does the chunk held in pv[] contain an operand the fast product path cannot take?  Evaluated
    // when the tile is stored, not when it is loaded: the loads stay in flight during the MACs of
    // the chunk before instead of being waited for straight away.
    auto staged_unsafe = [&]() -> bool {
        SafeRange sr;
#pragma unroll
        for (int i = 0; i < ELEMS; ++i) sr.add(pv[i]);
        return sr.unsafe();
    };
    auto store_chunk = [&]() {
        if (STAGE == STAGE_K4) {
            const int g = tid & (KC / 4 - 1);
#pragma unroll
            for (int i = 0; i < QUADS; ++i) {
                const int rl = (tid >> 3) + i * (WG_THREADS / (KC / 4));
                Pt4[g * GS + rl] = make_uint4(pv[4 * i], pv[4 * i + 1], pv[4 * i + 2], pv[4 * i + 3]);
            }
        } else if (STAGE == STAGE_R) {
            // ELEMS consecutive k of row rl, starting at a multiple of 4: whole uint4 groups
            const int rl = tid & (ROWS - 1);
            const int g0 = (tid / ROWS) * (ELEMS / 4);
#pragma unroll
            for (int i = 0; i < ELEMS / 4; ++i)
                Pt4[(g0 + i) * GS + rl] = make_uint4(pv[4 * i], pv[4 * i + 1], pv[4 * i + 2], pv[4 * i + 3]);
        } else {
            uint32_t *Pt = reinterpret_cast<uint32_t *>(Pt4);
            const int kk = tid & (KC - 1);
#pragma unroll
            for (int i = 0; i < ELEMS; ++i) {
                const int rl = (tid >> 5) + i * (WG_THREADS / KC);
                Pt[((kk >> 2) * GS + rl) * 4 + (kk & 3)] = pv[i];
            }
        }
    };

    float acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = 0.0f;

    if (ch_begin < ch_end) load_chunk(ch_begin);
    // the LUT copies started above have landed in LDS once the vector-memory counter drains;
    // the barriers at the top of the first trip then order them against every wave's gathers
    if (!LUTG) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const int lrow = wr * 64 + lane;
    const int mshift = 23 - m;
    const uint32_t lut_base = lds_address(lut_s);

    // Touching the next chunk's pre-decoded uniform operand (one lane per 128-byte line of this
    // wavefront's 2 KB) a chunk ahead brings it into L2 when it streams from HBM (filter gradients,
    // large GEMMs): the scalar loads of the inner loop are waited for every four rows, and a miss all
    // the way to HBM there stalls the wavefront.  The loaded word is never used; its register stays
    // reserved until the next trip's tile loads -- issued after it, returned after it -- have landed.
    const uint32_t *q_touch_ptr = a.qw + qtile + (size_t)lane * 32;
    uint32_t q_touch = 0;

    for (int ch = ch_begin; ch < ch_end; ++ch) {
        // The instruction arbiter favours a SIMD's oldest waves, so left alone the workgroups
        // that share a CU finish far apart and the last ones run on a mostly empty CU.  Wave
        // priority falls as a workgroup nears its end (more than 1/2, 1/4, 1/8 of its chunks
        // left, then the rest): whoever is behind catches up and the CU stays full to the end.
        {
            const int n = ch_end - ch_begin, rem = ch_end - ch;
            if (2 * rem > n) __builtin_amdgcn_s_setprio(3);
            else if (4 * rem > n) __builtin_amdgcn_s_setprio(2);
            else if (8 * rem > n) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
        }
        __syncthreads();  // every wave is done with the previous chunk's tile
        store_chunk();
        // Unsafe operands are rare: whoever staged one raises the chunk's flag (slot = chunk
        // parity); the slot of the previous chunk is cleared for the chunk after this one,
        // ordered against its writers by the barrier at the top of the next trip.
        if (staged_unsafe()) pflag[ch & 1] = 1u;
        __syncthreads();
        const uint32_t p_unsafe = __builtin_amdgcn_readfirstlane(pflag[ch & 1]);
        if (tid == 0) pflag[(ch & 1) ^ 1] = 0u;
        asm volatile("" ::"v"(q_touch));
        if (ch + 1 < ch_end) {
            if (active && lane < KC * QT * 4 / 128)
                asm volatile("global_load_dword %0, %1, off" : "=v"(q_touch) : "v"(q_touch_ptr + (size_t)(ch + 1) * KC * QT) : "memory");
            load_chunk(ch + 1);  // in flight during the MACs below
        }
        if (!active) continue;
        const uint32_t q_span = qflags[ch];
        const size_t qoff = (size_t)ch * KC * QT;
        // Both operands pass the quick test: fast products.  Else a second look before the slow path:
        // the exponent range of THIS wavefront's rows of the staged tile against the uniform operand's --
        // tiny gradients times ordinary weights, say, are still fast products.
        bool fast = !(p_unsafe | (q_span & SPAN_QUICK_FAIL));
        if (!fast) {
            SafeRange mine;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const uint4 p4 = Pt4[g * GS + lrow];
                mine.add(p4.x); mine.add(p4.y); mine.add(p4.z); mine.add(p4.w);
            }
            fast = spans_compatible(span_word(wave_union(mine)), q_span);
        }
        if (fast) {
          if constexpr (D16_LOOP) {
            // Gathers that deliver the byte already shifted (upper register half): the factors of two
            // columns are then one 64-bit add as well -- per pair of products two instructions that read
            // scalar registers instead of three.  Written out as a software pipeline over "units" of PU
            // column pairs: while one unit's factors and multiply-adds issue, the next unit's addresses and
            // gathers go out between them, so that an instruction that reads scalar registers is always
            // followed by one that does not.  (The uniform operand's words of a group of four rows are
            // loaded and waited for together: scalar loads return out of order, so waiting for one drains
            // the gathers in flight as well -- loading half a group ahead doubled those drains and lost 3 %.)
            constexpr int TN2 = (TN + 1) / 2;
            constexpr int PU = AMSIM_D16_PU < TN2 ? AMSIM_D16_PU : TN2;  // column pairs per unit
            constexpr int UPR = TN2 / PU;                               // units per reduction row
            constexpr int NU = KG * UPR;                                // units of a group of rows
            cq1_t qrow = qw + qoff + g_first * (KG * QT);
            // The gathers' destinations: a gather writes the upper half of its register; the lower half
            // must read as zero.  Devices differ in what such a load does to the other half (kept, or
            // cleared -- probed once per device): where it is kept, the registers start each chunk as zero.
            uint32_t Lh[2][2 * PU];
            if (a.d16_keeps) {
#pragma unroll
                for (int i = 0; i < 4 * PU; ++i) asm volatile("v_mov_b32 %0, 0" : "=v"(Lh[i / (2 * PU)][i % (2 * PU)]));
            } else {
#pragma unroll
                for (int i = 0; i < 4 * PU; ++i) asm volatile("" : "=v"(Lh[i / (2 * PU)][i % (2 * PU)]));
            }
#pragma unroll 1
            for (int g = g_first; g < g_last; ++g) {
                uint64_t qw2[KG][TN2];
#pragma unroll
                for (int r = 0; r < KG; ++r)
#pragma unroll
                    for (int j = 0; j < TN2; ++j) qw2[r][j] = reinterpret_cast<cq2_t>(qrow + r * QT)[j];
                const uint4 p4 = Pt4[g * GS + lrow];
                const uint32_t praw[KG] = {p4.x, p4.y, p4.z, p4.w};
                float ta[KG];
                uint64_t iab2[KG];
#pragma unroll
                for (int r = 0; r < KG; ++r) {
                    ta[r] = u2f(praw[r] & 0xff800000u);
                    const uint32_t iab = __builtin_amdgcn_ubfe(praw[r], (uint32_t)mshift, (uint32_t)m) + lut_base;
                    iab2[r] = ((uint64_t)iab << 32) | iab;
                }
                qrow += KG * QT;
                auto issue = [&](auto uc, auto ic) {
                    constexpr int u = decltype(uc)::value, i = decltype(ic)::value;
                    constexpr int r = u / UPR, pr = (u % UPR) * PU + i;
                    const uint64_t qi2 = qw2[r][pr] & 0x007fffff007fffffull;
                    const uint64_t li2 = add_u64_vs_ordered(iab2[r], qi2);
                    lds_gather_u8_hi(Lh[u & 1][2 * i], (uint32_t)li2);
                    lds_gather_u8_hi(Lh[u & 1][2 * i + 1], (uint32_t)(li2 >> 32));
                };
                static_for<0, PU>([&](auto ic) { issue(std::integral_constant<int, 0>{}, ic); });
                static_for<0, NU>([&](auto uc) {
                    constexpr int u = decltype(uc)::value;
                    constexpr int r = u / UPR;
                    // (a fence per unit: left alone the scheduler hoists every mask operation of the group to
                    // the loop's top and spills their results)
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, PU>([&](auto ic) {
                        constexpr int i = decltype(ic)::value;
                        constexpr int pr = (u % UPR) * PU + i;
                        // gathers issued after this pair's: the rest of this unit and what the next unit
                        // has sent so far
                        constexpr int younger = u + 1 < NU ? 2 * (PU - 1) : 2 * (PU - 1 - i);
                        const uint64_t qt2 = qw2[r][pr] & 0xff800000ff800000ull;
                        const uint64_t g2 = wait_add_u64_vs<younger>(((uint64_t)Lh[u & 1][2 * i + 1] << 32) | Lh[u & 1][2 * i], qt2);
                        fmac_ordered(acc[2 * pr], ta[r], u2f((uint32_t)g2));
                        if constexpr (u + 1 < NU) issue(std::integral_constant<int, u + 1>{}, ic);
                        fmac_ordered(acc[2 * pr + 1], ta[r], u2f((uint32_t)(g2 >> 32)));
                    });
                });
            }
          } else {
            cq1_t qrow = qw + qoff + g_first * (KG * QT);
#pragma unroll 1
            for (int g = g_first; g < g_last; ++g) {
                // column pairs are unpacked with 64-bit scalar ops: half the SALU instructions
                constexpr int TN2 = (TN + 1) / 2;
                uint64_t qw2[KG][TN2];
#pragma unroll
                for (int r = 0; r < KG; ++r)
#pragma unroll
                    for (int j = 0; j < TN2; ++j) {
                        if (TN >= 2) qw2[r][j] = reinterpret_cast<cq2_t>(qrow + r * QT)[j];
                        else qw2[r][j] = qrow[r * QT];
                    }
                const uint4 p4 = Pt4[g * GS + lrow];
                const uint32_t praw[KG] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
                for (int r = 0; r < KG; ++r) {
                    // 256-row workgroups carry more live scalars: fence each row so the scheduler does
                    // not hoist every s_and result to the loop top and spill them
                    __builtin_amdgcn_sched_barrier(0);
                    const float ta = u2f(praw[r] & 0xff800000u);
                    const uint32_t ia = __builtin_amdgcn_ubfe(praw[r], (uint32_t)mshift, (uint32_t)m);
                    uint32_t L[TN];
                    // LUT addresses of two columns with one 64-bit add: the lane's mantissa index in both
                    // halves plus the pair of row offsets (disjoint bits, so no carry crosses the halves).
                    // A vector instruction that reads scalar registers issues at half rate when another
                    // follows it; this halves their number for the address step.
                    const uint64_t ia2 = ((uint64_t)ia << 32) | ia;
#pragma unroll
                    for (int j = 0; j < TN; j += 2) {
                        const uint64_t qi2 = qw2[r][j >> 1] & 0x007fffff007fffffull;
                        const uint64_t li2 = add_u64_vs(ia2, qi2);
                        const uint32_t li0 = (uint32_t)li2, li1 = (uint32_t)(li2 >> 32);
                        L[j] = LUTG ? (uint32_t)lut_g[li0] : (uint32_t)lut_s[li0];
                        if (j + 1 < TN) L[j + 1] = LUTG ? (uint32_t)lut_g[li1] : (uint32_t)lut_s[li1];
                    }
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        // (entry << shift) + sign|exponent bits of q  ==  q_pow2 * 1.mant * 2^carry, exactly
                        const uint64_t qt2 = qw2[r][j >> 1] & 0xff800000ff800000ull;
                        const float g = u2f((L[j] << ESHIFT) + (uint32_t)(qt2 >> (32 * (j & 1))));
                        acc[j] = __builtin_fmaf(ta, g, acc[j]);
                    }
                }
                qrow += KG * QT;
            }
          }
        } else {
            // rare: the uniform operand's raw bits come from where it lies, not from the workspace
            const uint32_t *Pt = reinterpret_cast<const uint32_t *>(Pt4);
            // (the descriptor was written by an earlier kernel: read it through the scalar cache)
            const __attribute__((address_space(4))) QDesc &qd = *(const __attribute__((address_space(4))) QDesc *)(uintptr_t)a.qdesc;
            const float *qsrc = qd.base + (int64_t)qb * qd.batch_stride;
#pragma unroll 1
            for (int kk = g_first * KG; kk < g_last * KG; ++kk) {
                const uint32_t raw = Pt[((kk >> 2) * GS + lrow) * 4 + (kk & 3)];
                const uint32_t ia = (raw & 0x7fffffu) >> mshift;
#pragma unroll 1
                for (int jb = 0; jb < TN; jb += 4) {
#pragma unroll
                    for (int j = jb; j < jb + 4 && j < TN; ++j) {
                        const uint32_t qr = q_raw_bits(qd, qsrc, (uint32_t)a.K, (uint32_t)a.J, (uint32_t)ch * KC + kk, (uint32_t)(j0 + j));
                        const uint32_t li = (((qr & 0x7fffffu) >> mshift) << m) + ia;
                        const uint32_t e16 = (LUTG ? (uint32_t)lut_g[li] : (uint32_t)lut_s[li]) << ESHIFT;
                        acc[j] += a.lane_first ? am_exact(raw, qr, e16) : am_exact(qr, raw, e16);
                    }
                }
            }
        }
    }

    const int64_t r = row0 + lrow;
    if (!active) return;  // (with reduction slices `active` is the same for the whole workgroup)
    if (KSLICES) {
        // the four wavefronts' sums of one output, added in wavefront order through the LUT's LDS
        float(*red)[TN][64] = reinterpret_cast<float(*)[TN][64]>(lut_s);
        static_assert(LUTG || 3 * TN * 64 * sizeof(float) <= LUT_LDS_BYTES, "the slices' sums reuse the LUT's LDS");
        __syncthreads();  // every wavefront is done gathering from the LUT
        if (wave != 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j) red[wave - 1][j][lane] = acc[j];
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int s = 0; s < 3; ++s)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] += red[s][j][lane];
    }
    if (seg_nsplit == 1) {
        if (r < a.R) {
            float *o = a.out + (int64_t)bz * a.out_batch_stride + out_row_offset(a.ep.omap, r, a.so_r);
            if (a.ep.bias_j || a.ep.bias_r || a.ep.act) {
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[j] = apply_epilogue(a.ep, acc[j], r, min((int64_t)(j0 + j), a.J - 1));
            }
            if (TN % 4 == 0 && a.vec_store && j0 + TN <= a.J) {
                // a lane's TN outputs are contiguous and 16-byte aligned: whole float4 stores
                float4 *o4 = reinterpret_cast<float4 *>(o + j0);
#pragma unroll
                for (int j = 0; j < TN / 4; ++j) o4[j] = make_float4(acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3]);
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    if (j0 + j < a.J) o[(int64_t)(j0 + j) * a.so_j] = acc[j];
            }
        }
    } else {
        if (r < a.R) {  // rows past the end are never read by the reduction
            float *o = seg_partial + (((size_t)split * a.batch + bz) * seg_Rp + (r - seg_row_base)) * a.Jp + j0;
#pragma unroll
            for (int j = 0; j < TN; ++j) o[j] = acc[j];
        }
    }
}

// OUTS consecutive outputs per workgroup, WG_THREADS / OUTS threads ("ways") per output.  Each
// way takes every ways-th split in eight interleaved chains (eight loads in flight); the chains
// and then the ways' sums are combined in a fixed order, so the result does not depend on
// scheduling.  Few outputs with many splits use OUTS = 8 (32 ways), else the loop over the
// splits is one long chain of memory latencies.
template <int OUTS>
__global__ __launch_bounds__(WG_THREADS) void splitk_reduce_kernel(RArgs a)
{
    constexpr int WAYS = WG_THREADS / OUTS;
    __shared__ float part[WAYS][OUTS];
    const int o = threadIdx.x % OUTS, way = threadIdx.x / OUTS;
    const int64_t idx = (int64_t)blockIdx.x * OUTS + o;
    const int bz = blockIdx.y;
    const bool valid = idx < a.R * a.J;
    int64_t r = 0, j = 0;
    float c[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (valid) {
        r = idx / a.J;
        j = idx - r * a.J;
        const size_t stride = (size_t)a.batch * a.Rp * a.Jp;
        const float *src = a.partial + ((size_t)bz * a.Rp + r) * a.Jp + j;
        int sp = way;
        for (; sp + 7 * WAYS < a.nsplit; sp += 8 * WAYS) {
#pragma unroll
            for (int u = 0; u < 8; ++u) c[u] += src[(size_t)(sp + u * WAYS) * stride];
        }
        for (int u = 0; sp < a.nsplit; sp += WAYS, ++u) c[u] += src[(size_t)sp * stride];
    }
    part[way][o] = ((c[0] + c[1]) + (c[2] + c[3])) + ((c[4] + c[5]) + (c[6] + c[7]));
    __syncthreads();
    if (way == 0 && valid) {
        float s = part[0][o];
#pragma unroll
        for (int w = 1; w < WAYS; ++w) s += part[w][o];
        a.out[(int64_t)bz * a.out_batch_stride + out_row_offset(a.ep.omap, a.row_base + r, a.so_r) + j * a.so_j] =
            apply_epilogue(a.ep, s, a.row_base + r, j);
    }
}

// Few slices over many outputs whose rows are contiguous (slices of a tall problem's reduction): a
// thread adds four consecutive columns of one row across the slices, in slice order, with 16-byte
// loads and one 16-byte store -- the general kernel above spends a workgroup on 64 outputs.
__global__ __launch_bounds__(WG_THREADS) void splitk_reduce_rows4_kernel(RArgs a)
{
    const int64_t idx = (int64_t)blockIdx.x * WG_THREADS + threadIdx.x;
    const int64_t per_row = a.J / 4;
    if (idx >= a.R * per_row) return;
    const int bz = blockIdx.y;
    const int64_t r = idx / per_row, j = (idx - r * per_row) * 4;
    const size_t stride = (size_t)a.batch * a.Rp * a.Jp;
    const float *src = a.partial + ((size_t)bz * a.Rp + r) * a.Jp + j;
    float4 s = *reinterpret_cast<const float4 *>(src);
    for (int sp = 1; sp < a.nsplit; ++sp) {
        const float4 v = *reinterpret_cast<const float4 *>(src + (size_t)sp * stride);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    s.x = apply_epilogue(a.ep, s.x, a.row_base + r, j);
    s.y = apply_epilogue(a.ep, s.y, a.row_base + r, j + 1);
    s.z = apply_epilogue(a.ep, s.z, a.row_base + r, j + 2);
    s.w = apply_epilogue(a.ep, s.w, a.row_base + r, j + 3);
    *reinterpret_cast<float4 *>(a.out + (int64_t)bz * a.out_batch_stride + out_row_offset(a.ep.omap, a.row_base + r, a.so_r) + j) = s;
}

// Empty reduction: every output is the epilogue of zero (zeros without one).  VEC = 4: a thread
// writes four consecutive columns of a row as one 16-byte store (rows contiguous, 16-byte aligned,
// a multiple of four columns): the pixel classes of a strided grad-input that no filter tap
// reaches are most of that tensor.
template <int VEC>
__global__ __launch_bounds__(WG_THREADS) void fill_empty_kernel(RArgs a)
{
    const int64_t idx = (int64_t)blockIdx.x * WG_THREADS + threadIdx.x;
    const int64_t per_row = a.J / VEC;
    if (idx >= a.R * per_row) return;
    const int64_t r = idx / per_row, j = (idx - r * per_row) * VEC;
    float *o = a.out + (int64_t)blockIdx.y * a.out_batch_stride + out_row_offset(a.ep.omap, a.row_base + r, a.so_r) + j * a.so_j;
    if (VEC == 4) {
        float4 v;
        v.x = apply_epilogue(a.ep, 0.0f, a.row_base + r, j);
        v.y = apply_epilogue(a.ep, 0.0f, a.row_base + r, j + 1);
        v.z = apply_epilogue(a.ep, 0.0f, a.row_base + r, j + 2);
        v.w = apply_epilogue(a.ep, 0.0f, a.row_base + r, j + 3);
        *reinterpret_cast<float4 *>(o) = v;
    } else {
        *o = apply_epilogue(a.ep, 0.0f, a.row_base + r, j);
    }
}

struct PoisonArgs {
    const float *filter;
    int KH, KW, IC, OC, n_classes, out_stride;
    float *out;
    TapClass cls[MAX_TAP_CLASSES];
};

// One wavefront per (class, input channel): lanes run over the output channels of each skipped tap.
__global__ __launch_bounds__(WG_THREADS) void skipped_tap_poison_kernel(PoisonArgs a)
{
    const int lane = threadIdx.x & 63;
    const int ic = blockIdx.x * (WG_THREADS / 64) + (threadIdx.x >> 6);
    if (ic >= a.IC) return;
    const TapClass c = a.cls[blockIdx.y];
    int bad = 0;
    for (int fy = 0; fy < a.KH; ++fy)
        for (int fx = 0; fx < a.KW; ++fx) {
            // flipped-filter indices, as the sub-problem's operand decoder walks them
            const int gy = a.KH - 1 - fy, gx = a.KW - 1 - fx;
            const bool own_y = gy >= c.fy0 && (gy - c.fy0) % c.fsy == 0 && (gy - c.fy0) / c.fsy < c.th;
            const bool own_x = gx >= c.fx0 && (gx - c.fx0) % c.fsx == 0 && (gx - c.fx0) / c.fsx < c.tw;
            if (own_y && own_x) continue;
            const float *w = a.filter + ((int64_t)(fy * a.KW + fx) * a.IC + ic) * a.OC;
            for (int oc = lane; oc < a.OC; oc += 64) bad |= ((f2u(w[oc]) & 0x7f800000u) == 0x7f800000u) ? 1 : 0;
        }
    bad = __any(bad);
    if (lane == 0) a.out[(int64_t)blockIdx.y * a.out_stride + ic] = bad ? u2f(0x7fc00000u) : 0.0f;
}

int launch_skipped_tap_poison(const float *filter, int KH, int KW, int IC, int OC, const TapClass *classes,
                              int n_classes, float *out, int out_stride, hipStream_t stream)
{
    if (n_classes <= 0 || IC <= 0) return AMSIM_OK;
    if (n_classes > MAX_TAP_CLASSES) return fail(AMSIM_ERR_INVALID, "too many tap classes for one launch");
    PoisonArgs a{};
    a.filter = filter; a.KH = KH; a.KW = KW; a.IC = IC; a.OC = OC; a.n_classes = n_classes; a.out_stride = out_stride;
    a.out = out;
    for (int i = 0; i < n_classes; ++i) a.cls[i] = classes[i];
    const int per_wg = WG_THREADS / 64;
    skipped_tap_poison_kernel<<<dim3((unsigned)((IC + per_wg - 1) / per_wg), (unsigned)n_classes), WG_THREADS, 0, stream>>>(a);
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

void launch_reduce(const RArgs &ra, hipStream_t stream)
{
    const int64_t outs = ra.R * ra.J;
    // (the slices of the general kernel are summed as eight interleaved chains per way; with at most
    // eight slices and one way per output that is the plain sum in slice order, which this kernel forms too)
    const bool rows4 = ra.nsplit <= 4 && outs >= (1 << 20) && ra.J % 4 == 0 && ra.Jp % 4 == 0 && ra.so_j == 1 && ra.so_r % 4 == 0 &&
                       ra.out_batch_stride % 4 == 0 && (((uintptr_t)ra.out | (uintptr_t)ra.partial) & 15) == 0 &&
                       (outs / 4 + WG_THREADS - 1) / WG_THREADS < (1ll << 31);
    if (rows4) {
        splitk_reduce_rows4_kernel<<<dim3((unsigned)((outs / 4 + WG_THREADS - 1) / WG_THREADS), (unsigned)ra.batch), WG_THREADS, 0, stream>>>(ra);
        return;
    }
    if (outs * ra.batch <= 16384 && ra.nsplit >= 64)
        splitk_reduce_kernel<8><<<dim3((unsigned)((outs + 7) / 8), (unsigned)ra.batch), WG_THREADS, 0, stream>>>(ra);
    else
        splitk_reduce_kernel<64><<<dim3((unsigned)((outs + 63) / 64), (unsigned)ra.batch), WG_THREADS, 0, stream>>>(ra);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
// Work shaping.  A problem is R/rows row tiles x column groups x batch workgroups ("tiles"),
// each a reduction of nchunks chunks.  The machine holds `slots` workgroups at once and a
// lone workgroup runs about 1/0.74 as fast as one of a full machine, so the time of a launch
// is governed by rounds of `slots` workgroups.  The planner picks
//   * nsplit: every tile's reduction split into that many workgroups (partial sums reduced by
//     splitk_reduce_kernel in a fixed order), and
//   * a tail: when the workgroup count is a little more than a whole number of rounds, the
//     row tiles of the last, mostly empty round are split further so that they fill the
//     machine again (their workgroups dispatch first, in the same launch),
// by minimising a small cost model (unit: one chunk of one workgroup on a full machine).
struct Plan {
    int TN, WR, Jp, nchunks;
    int nsplit, chunks_per_split;  // of the main part
    int64_t Rp;                    // padded rows
    int64_t rows_main;             // rows covered by the main part (== R when there is no tail)
    int tail_nsplit, tail_chunks_per_split;
    size_t off_qw, off_flags, off_qdesc, off_partial_main, off_partial_tail, total;
};

static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

namespace {
struct Shape {
    int nsplit = 1, cps = 0;
    int64_t main_rowtiles = 0;
    int tail_nsplit = 1, tail_cps = 0;
    double cost = 0;
};
// Time of one chunk of one workgroup when a fraction `occ` of the machine's workgroup slots is
// filled, relative to a full machine (measured: 0.735 at 51 %; nearly linear above that).
inline double occupancy_factor(double occ)
{
    if (occ >= 1.0) return 1.0;
    return occ >= 0.51 ? 0.735 + 0.54 * (occ - 0.51) : 0.735 - 0.5 * (0.51 - occ);
}
}  // namespace

static Shape shape_work(int64_t rowtiles, int64_t G, int n, int64_t slots, bool may_peel, double reduce_unit)
{
    // reduce_unit: cost of writing + re-reading one full set of partial sums
    Shape best;
    best.cps = n;
    best.main_rowtiles = rowtiles;
    best.tail_cps = n;
    bool have = false;
    const int64_t wgs = rowtiles * G;
    const int64_t smax = std::min<int64_t>(n, 2 * ((slots + wgs - 1) / wgs) + 1);
    for (int64_t s0 = 1; s0 <= smax; ++s0) {
        Shape c;
        c.cps = (int)((n + s0 - 1) / s0);
        c.nsplit = (n + c.cps - 1) / c.cps;
        if (c.nsplit != s0) continue;  // same shape as a smaller candidate
        c.main_rowtiles = rowtiles;
        c.tail_cps = n;
        const int64_t units = wgs * c.nsplit;
        const int64_t full = units / slots, rem = units - full * slots;
        double t;
        if (full == 0) {
            t = c.cps * occupancy_factor((double)units / slots);
        } else if (rem == 0) {
            t = (double)full * c.cps;
        } else {
            t = (double)full * c.cps + c.cps * occupancy_factor((double)rem / slots);
            const int64_t main_rt = full * slots / (G * c.nsplit);
            const int64_t tail_wgs = (rowtiles - main_rt) * G;
            if (may_peel && main_rt >= 1 && tail_wgs * c.nsplit * 2 <= slots) {
                const int64_t ts0 = std::min<int64_t>(slots / tail_wgs, n);
                const int tcps = (int)((n + ts0 - 1) / ts0);
                const int ts = (n + tcps - 1) / tcps;
                if (ts > c.nsplit) {
                    const double tp = (double)full * c.cps + tcps * occupancy_factor((double)tail_wgs * ts / slots) + 0.8;
                    if (tp < t) { t = tp; c.main_rowtiles = main_rt; c.tail_nsplit = ts; c.tail_cps = tcps; }
                }
            }
        }
        if (c.nsplit > 1) t += 0.4 + reduce_unit * c.nsplit;
        c.cost = t;
        if (!have || t < best.cost - 1e-9) { best = c; have = true; }
    }
    return best;
}

static Plan compute_plan(int64_t R, int64_t J, int64_t K, int batch, int q_batches, bool split_k, int waves64, int cus);

// Plans are pure functions of their arguments; the last few are remembered per thread so that
// the workspace query and the call that follows it do not repeat the search.
// waves64: waves per SIMD the 64-row kernel variant that will run is compiled for
// cus: compute units of the machine the plan is for (0 = the current device)
static Plan make_plan(int64_t R, int64_t J, int64_t K, int batch, int q_batches, bool split_k, int waves64, int cus = 0)
{
    struct Key { int64_t R, J, K; int batch, qb, split; };
    struct Slot { Key k; Plan p; bool used = false; };
    static thread_local Slot memo[16];
    static thread_local unsigned next = 0;
    if (cus <= 0) cus = device_compute_units();
    const Key key{R, J, K, batch, q_batches, (split_k ? 1 : 0) | (waves64 << 1) | (cus << 8)};
    for (const Slot &sl : memo)
        if (sl.used && sl.k.R == R && sl.k.J == J && sl.k.K == K && sl.k.batch == batch && sl.k.qb == q_batches &&
            sl.k.split == key.split)
            return sl.p;
    Slot &sl = memo[next++ % 16];
    sl.k = key;
    sl.p = compute_plan(R, J, K, batch, q_batches, split_k, waves64, cus);
    sl.used = true;
    return sl.p;
}

static Plan compute_plan(int64_t R, int64_t J, int64_t K, int batch, int q_batches, bool split_k, int waves64, int cus)
{
    Plan pl{};
    // Narrow outputs (one column group) stack four row tiles per workgroup and shrink the
    // per-lane column count to fit; with a single row tile there is nothing to stack, and the
    // 64-row kernel (compiled for 16 columns only) runs with its spare columns idle.
    pl.TN = (J >= 9 || R <= 64) ? 16 : J >= 5 ? 8 : J >= 3 ? 4 : (int)std::max<int64_t>(J, 1);
    const int64_t jchunks = (J + pl.TN - 1) / pl.TN;
    pl.WR = (jchunks >= 2 || R <= 64) ? 1 : 4;
    pl.Jp = (int)((J + QT - 1) / QT * QT);
    pl.nchunks = (int)((K + KC - 1) / KC);

    // the work shape of one wave arrangement, and what the cost model says it takes in seconds
    struct Choice { Shape sh; double seconds; int rows; };
    auto evaluate = [&](int WR) {
        Choice c;
        c.rows = WR > 1 ? 64 * WR : 64;
        const int wc = WR == WR_KSLICES ? 1 : 4 / WR;
        const int64_t Rp = (R + c.rows - 1) / c.rows * c.rows;
        const int64_t rowtiles = Rp / c.rows;
        const int64_t G = ((jchunks + wc - 1) / wc) * batch;
        // resident workgroups: the 256-row kernels hold 53 KB of LDS and up to 170 VGPRs, three fit a CU
        const int64_t slots = (int64_t)cus * (WR > 1 ? 3 : waves64);
        c.sh.cps = pl.nchunks;
        c.sh.main_rowtiles = rowtiles;
        c.sh.tail_cps = pl.nchunks;
        // one chunk of one workgroup on a full machine, and one pass over the output, in seconds
        // (reduction slices: a quarter of the products per chunk behind the same staging and barriers -- a full
        // machine of them takes 1.45 x the time per product; priced at 1.3, which picked best over a sweep of
        // ResNet-50's layer shapes at small feature maps, the few-workgroup plans they compete with being
        // underpriced by about as much)
        const double chunk_s = (double)c.rows * (wc * pl.TN) * KC * slots / (MACS_PER_CU_S * cus) * (WR == WR_KSLICES ? 1.3 : 1.0);
        if (split_k && pl.nchunks > 1) {
            const double pass_s = 2.0 * (double)Rp * pl.Jp * batch * sizeof(float) / PARTIAL_BYTES_PER_S;
            c.sh = shape_work(rowtiles, G, pl.nchunks, slots, true, pass_s / chunk_s);
        } else {
            c.sh.cost = pl.nchunks * occupancy_factor((double)(rowtiles * G) / slots);
        }
        const int64_t rounds = (rowtiles * G * c.sh.nsplit + slots - 1) / slots;
        c.seconds = c.sh.cost * chunk_s + rounds * WORKGROUP_START_S;
        return c;
    };
    Choice ch = evaluate(pl.WR);
    // Few workgroups of the usual arrangement (half the slots or fewer) and a reduction that may be
    // split: one column group per workgroup with the reduction rows dealt out to its four waves gives
    // four times the workgroups and sums their slices inside the compute unit, without partial sums.
    if (split_k && pl.nchunks > 1 && pl.TN == 16 && pl.WR == 1) {
        const int64_t wgs = ((R + 63) / 64) * ((jchunks + 3) / 4) * batch;
        if (2 * wgs <= (int64_t)cus * waves64) {
            const Choice alt = evaluate(WR_KSLICES);
            if (alt.seconds < 0.97 * ch.seconds) { ch = alt; pl.WR = WR_KSLICES; }
        }
    }
    const Shape &sh = ch.sh;
    const int rows = ch.rows;
    pl.Rp = (R + rows - 1) / rows * rows;
    const int64_t rowtiles = pl.Rp / rows;
    pl.nsplit = sh.nsplit;
    pl.chunks_per_split = sh.cps;
    pl.rows_main = sh.main_rowtiles == rowtiles ? R : sh.main_rowtiles * rows;
    pl.tail_nsplit = sh.tail_nsplit;
    pl.tail_chunks_per_split = sh.tail_cps;

    const size_t plane = (size_t)pl.nchunks * KC * pl.Jp;
    size_t off = 0;
    pl.off_qw = off;      off = align256(off + (size_t)q_batches * plane * sizeof(uint32_t));
    pl.off_flags = off;   off = align256(off + (size_t)q_batches * (pl.Jp / QT) * std::max(pl.nchunks, 1) * sizeof(uint32_t));
    pl.off_qdesc = off;   off = align256(off + sizeof(QDesc));
    const int64_t main_rows_p = sh.main_rowtiles * rows, tail_rows_p = pl.Rp - main_rows_p;
    pl.off_partial_main = off;
    if (pl.nsplit > 1) off = align256(off + (size_t)pl.nsplit * batch * main_rows_p * pl.Jp * sizeof(float));
    pl.off_partial_tail = off;
    if (pl.rows_main < R && pl.tail_nsplit > 1)
        off = align256(off + (size_t)pl.tail_nsplit * batch * tail_rows_p * pl.Jp * sizeof(float));
    pl.total = off;
    return pl;
}

size_t gemm_workspace_bytes(int64_t R, int64_t J, int64_t K, int batch, int q_batches)
{
    if (R <= 0 || J <= 0 || K <= 0 || batch <= 0) return 0;
    // valid whichever way amsim_set_split_k stands when the call is made, whichever kernel variant
    // (6 or 5 waves per SIMD) the operand layout selects, and -- since the query may be made with no
    // device or another device current -- for every machine size the plans are made for: the
    // current device's compute units, 256 (MI355X) and 304
    size_t need = make_plan(R, J, K, batch, q_batches, false, WAVES_PER_SIMD).total;
    for (int cus : {device_compute_units(), 256, 304})
        for (int w = WAVES_PER_SIMD - 1; w <= WAVES_PER_SIMD; ++w)
            need = std::max(need, make_plan(R, J, K, batch, q_batches, true, w, cus).total);
    if (direct_shape_eligible(R, J, K, batch, true)) need = std::max(need, direct_workspace_bytes(R, J, K, batch));
    if (klanes_shape_eligible(R, J, K, batch)) need = std::max(need, klanes_workspace_bytes(R, J, K));
    return need;
}

// bytes of the unsplit plan: the pre-decoded uniform operand, its flags and its descriptor
static size_t unsplit_bytes(int64_t R, int64_t J, int64_t K, int batch, int q_batches)
{
    return make_plan(R, J, K, batch, q_batches, false, WAVES_PER_SIMD).total;
}

size_t gemm_workspace_bytes_wide(int64_t R, int64_t J, int64_t K, int batch, int q_batches)
{
    if (R <= 0 || J <= 0 || K <= 0 || batch <= 0 || !wide_shape_eligible(R, batch)) return 0;
    return unsplit_bytes(R, J, K, batch, q_batches) + wide_workspace_bytes(R, J, K, batch);
}

size_t gemm_workspace_bytes_wide_planar(const GemmDesc &d)
{
    const size_t planar = wide_workspace_bytes_planar(d);
    if (planar == 0 || !wide_shape_eligible(d.R, d.batch)) return 0;
    return unsplit_bytes(d.R, d.J, d.K, d.batch, d.q.batches) + planar;
}

size_t gemm_workspace_bytes_any_lut(int64_t R, int64_t J, int64_t K, int batch, int q_batches)
{
    const size_t need = gemm_workspace_bytes(R, J, K, batch, q_batches);
    return need ? std::max(need, gemm_workspace_bytes_wide(R, J, K, batch, q_batches)) : 0;
}

// what the planner decides for a problem: {TN, WR, nsplit, chunks per split, rows of the main
// part, tail nsplit, tail chunks per split, chunks} (for tests and tuning)
void gemm_plan_info(int64_t R, int64_t J, int64_t K, int batch, int q_batches, bool split_k, int waves64, int64_t info[8])
{
    const Plan pl = make_plan(R, J, K, batch, q_batches, split_k, waves64);
    info[0] = pl.TN; info[1] = pl.WR; info[2] = pl.nsplit; info[3] = pl.chunks_per_split;
    info[4] = pl.rows_main; info[5] = pl.rows_main < R ? pl.tail_nsplit : 0;
    info[6] = pl.rows_main < R ? pl.tail_chunks_per_split : 0; info[7] = pl.nchunks;
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// staging mode of the lane operand for a problem (which kernel variant runs)
static int stage_of(const PDesc &p, int64_t K)
{
    if (p.kind == P_DENSE) {
        const bool k_contig = p.sk == 1 && p.sr != 1;
        const bool vec = k_contig && (p.sr % 4 == 0) && (K % 4 == 0) && (p.batch_stride % 4 == 0) && aligned16(p.base);
        return vec ? STAGE_K4 : k_contig ? STAGE_K : STAGE_R;
    }
    if (p.kind == P_PATCH) return ((p.C % 4 == 0) && aligned16(p.base)) ? STAGE_K4 : STAGE_K;
    return STAGE_R;
}
// waves per SIMD the 64-row variant of that problem is compiled for (its __launch_bounds__)
static int waves64_of(const PDesc &p, int64_t K)
{
    return (p.kind == P_DENSE && stage_of(p, K) != STAGE_K4) ? WAVES_PER_SIMD - 1 : WAVES_PER_SIMD;
}

template <int TN, int WR, bool LUTG>
static void launch_variant(const KArgs &ka, dim3 grid, hipStream_t stream)
{
    const PDesc &p = ka.p;
    const int stage = stage_of(p, ka.K);
    if (p.kind == P_DENSE) {
        if (stage == STAGE_K4) lutgemm_kernel<TN, WR, P_DENSE, STAGE_K4, LUTG><<<grid, WG_THREADS, 0, stream>>>(ka);
        else if (stage == STAGE_K) lutgemm_kernel<TN, WR, P_DENSE, STAGE_K, LUTG><<<grid, WG_THREADS, 0, stream>>>(ka);
        else lutgemm_kernel<TN, WR, P_DENSE, STAGE_R, LUTG><<<grid, WG_THREADS, 0, stream>>>(ka);
    } else if (p.kind == P_PATCH) {
        if (stage == STAGE_K4) lutgemm_kernel<TN, WR, P_PATCH, STAGE_K4, LUTG><<<grid, WG_THREADS, 0, stream>>>(ka);
        else lutgemm_kernel<TN, WR, P_PATCH, STAGE_K, LUTG><<<grid, WG_THREADS, 0, stream>>>(ka);
    } else {
        lutgemm_kernel<TN, WR, P_GF, STAGE_R, LUTG><<<grid, WG_THREADS, 0, stream>>>(ka);
    }
}

template <bool LUTG>
static void launch_tn(int TN, int WR, const KArgs &k, dim3 grid, hipStream_t stream)
{
    switch (TN) {
    case 16:
        if (WR == 1) launch_variant<16, 1, LUTG>(k, grid, stream);
        else if (WR == WR_KSLICES) launch_variant<16, WR_KSLICES, LUTG>(k, grid, stream);
        else launch_variant<16, 4, LUTG>(k, grid, stream);
        break;
    case 8: launch_variant<8, 4, LUTG>(k, grid, stream); break;
    case 4: launch_variant<4, 4, LUTG>(k, grid, stream); break;
    case 2: launch_variant<2, 4, LUTG>(k, grid, stream); break;
    default: launch_variant<1, 4, LUTG>(k, grid, stream); break;
    }
}

int run_gemm(const Lut &lut, const GemmDesc &d, void *workspace, size_t workspace_bytes, hipStream_t stream)
{
    if (d.R < 0 || d.J < 0 || d.K < 0 || d.batch < 0) return fail(AMSIM_ERR_INVALID, "negative GEMM extent");
    if (d.R == 0 || d.J == 0 || d.batch == 0) return AMSIM_OK;
    if ((lut.m <= 7 && lut.img_ab == nullptr) || (lut.m > 7 && lut.img16_ab == nullptr))
        return fail(AMSIM_ERR_UNSUPPORTED, "LUT handle holds no device image for the GEMM path");
    if (const int rc = check_lut_device(lut)) return rc;
    if (d.R >= (1ll << 31) || d.K >= (1ll << 31) || d.J >= (1ll << 24))
        return fail(AMSIM_ERR_UNSUPPORTED, "GEMM extent too large");
    if (d.K == 0) {
        // empty reduction: the output is all zeros (matmulam.cc:154-160)
        RArgs ra{nullptr, d.out, d.R, d.J, 0, d.so_r, d.so_j, d.out_batch_stride, 0, 0, d.batch, 0,
                 Epilogue{d.bias_j, d.bias_r, d.act, d.omap}};
        if (d.batch > 65535) return fail(AMSIM_ERR_UNSUPPORTED, "batch exceeds the grid limit");
        const bool vec = d.J % 4 == 0 && d.so_j == 1 && d.so_r % 4 == 0 && d.out_batch_stride % 4 == 0 && aligned16(d.out);
        const int64_t threads = d.R * (vec ? d.J / 4 : d.J);
        if ((threads + WG_THREADS - 1) / WG_THREADS >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "output exceeds the grid limit");
        const dim3 grid((unsigned)((threads + WG_THREADS - 1) / WG_THREADS), (unsigned)d.batch);
        if (vec) fill_empty_kernel<4><<<grid, WG_THREADS, 0, stream>>>(ra);
        else fill_empty_kernel<1><<<grid, WG_THREADS, 0, stream>>>(ra);
        AMSIM_HIP_CHECK(hipGetLastError());
        return AMSIM_OK;
    }
    const int engine = lut.engine >= 0 ? lut.engine : g_engine.load();  // the handle's own setting wins
    const bool use_direct = engine != AMSIM_ENGINE_LDS_TABLE && direct_eligible(lut.m, d, engine == AMSIM_ENGINE_DIRECT);
    // the handle's own setting wins over the process default (read once per call)
    const bool may_split = (lut.split_k >= 0 ? lut.split_k != 0 : g_split_k.load() != 0) && !d.no_split;
    // The workspace must be what the query returns (valid for every engine and split mode), whichever
    // engine runs; a call that keeps its reduction whole on purpose needs only its own plan's share.
    const size_t need = !d.no_split ? gemm_workspace_bytes(d.R, d.J, d.K, d.batch, d.q.batches)
                        : use_direct ? 0
                                     : make_plan(d.R, d.J, d.K, d.batch, d.q.batches, false, waves64_of(d.p, d.K)).total;
    if (need && (workspace == nullptr || ((uintptr_t)workspace & 255) || workspace_bytes < need))
        return fail(AMSIM_ERR_WORKSPACE, "workspace missing, not 256-byte aligned or smaller than " +
                                             std::to_string(need) + " bytes");
    // small filter gradients whose reductions may be split: the reduction over the lanes
    if (engine == AMSIM_ENGINE_AUTO && may_split && klanes_eligible(lut.m, d))
        return run_gemm_klanes(lut, d, workspace, workspace_bytes, stream);
    if (use_direct) return run_gemm_direct(lut, d, may_split, workspace, workspace_bytes, stream);
    if (wide_eligible(lut.m, d, may_split)) {
        // tables too wide for the LDS: the row-staged engine, if the workspace also holds the
        // transposed lane operand (else the global-gather variant below does the job, slowly)
        const Plan pq = make_plan(d.R, d.J, d.K, d.batch, d.q.batches, false, WAVES_PER_SIMD);
        // convolution patches: from an im2col in the workspace if it holds one (KH x KW times the source:
        // streamed once, the fastest), else from a zero-bordered channel-major copy of the source (its own
        // size; every plane is re-read once per filter tap, about 25 % slower overall), else -- below --
        // one global gather per product
        const bool ws_ok = workspace != nullptr && ((uintptr_t)workspace & 255) == 0;
        const bool im2col = ws_ok && workspace_bytes >= pq.total + wide_workspace_bytes(d.R, d.J, d.K, d.batch);
        const size_t planar_need = im2col ? 0 : wide_workspace_bytes_planar(d);
        const bool planar = ws_ok && planar_need > 0 && workspace_bytes >= pq.total + planar_need;
        if (im2col || planar) {
            uint8_t *ws = static_cast<uint8_t *>(workspace);
            QArgs qa{};
            qa.q = d.q;
            qa.K = d.K; qa.J = d.J; qa.Jp = pq.Jp; qa.nchunks = pq.nchunks; qa.m = lut.m;
            qa.qw = reinterpret_cast<uint32_t *>(ws + pq.off_qw);
            qa.qflags = reinterpret_cast<uint32_t *>(ws + pq.off_flags);
            qa.qdesc_out = reinterpret_cast<QDesc *>(ws + pq.off_qdesc);
            if (const int rc = launch_q_prepass(qa, d.q.batches, stream)) return rc;
            return run_gemm_wide(lut, d, WideQ{qa.qw, qa.qflags, qa.qdesc_out, pq.Jp, pq.nchunks}, ws + pq.total, planar, may_split, stream);
        }
    }
    const Plan pl = make_plan(d.R, d.J, d.K, d.batch, d.q.batches, may_split, waves64_of(d.p, d.K));
    uint8_t *ws = static_cast<uint8_t *>(workspace);

    QArgs qa{};
    qa.q = d.q;
    qa.K = d.K; qa.J = d.J; qa.Jp = pl.Jp; qa.nchunks = pl.nchunks; qa.m = lut.m;
    qa.qw = reinterpret_cast<uint32_t *>(ws + pl.off_qw);
    qa.qflags = reinterpret_cast<uint32_t *>(ws + pl.off_flags);
    qa.qdesc_out = reinterpret_cast<QDesc *>(ws + pl.off_qdesc);
    if (const int rc = launch_q_prepass(qa, d.q.batches, stream)) return rc;

    KArgs ka{};
    ka.p = d.p;
    if (lut.m <= 7) ka.lut_img = d.lane_first ? lut.img_ba : lut.img_ab;
    else ka.lut_img = reinterpret_cast<const uint8_t *>(d.lane_first ? lut.img16_ba : lut.img16_ab);
    ka.lut_bytes = (int)(((size_t)1 << (2 * lut.m)) + ((size_t)1 << lut.m) + 15) / 16 * 16;
    ka.m = lut.m;
    ka.lane_first = d.lane_first ? 1 : 0;
    ka.qw = qa.qw; ka.qdesc = qa.qdesc_out; ka.qflags = qa.qflags;
    ka.q_batches = d.q.batches;
    ka.R = d.R; ka.J = d.J; ka.K = d.K;
    ka.Jp = pl.Jp; ka.nchunks = pl.nchunks;
    ka.out = d.out; ka.so_r = d.so_r; ka.so_j = d.so_j; ka.out_batch_stride = d.out_batch_stride;
    ka.batch = d.batch;
    ka.ep = Epilogue{d.bias_j, d.bias_r, d.act, d.omap};
    ka.vec_store = (d.so_j == 1 && d.so_r % 4 == 0 && d.out_batch_stride % 4 == 0 && aligned16(d.out)) ? 1 : 0;
    ka.d16_keeps = lut.d16_keeps;

    const int rows = pl.WR > 1 ? 64 * pl.WR : 64, wc = pl.WR == WR_KSLICES ? 1 : 4 / pl.WR;
    const int64_t jchunks = (d.J + pl.TN - 1) / pl.TN;
    const int64_t gy = (jchunks + wc - 1) / wc;

    // One launch: the split-reduction tail's workgroups (if any) come first in dispatch order
    // and share the machine with the first main workgroups; the main workgroups that start
    // after them catch up through wave priority.
    auto fill_seg = [&](KArgs::Seg &sg, int64_t row_base, int64_t row_end, int nsplit, int cps, size_t off_partial) -> int64_t {
        sg.row_base = row_base;
        sg.partial = reinterpret_cast<float *>(ws + off_partial);
        sg.Rp = (row_end - row_base + rows - 1) / rows * rows;
        sg.nsplit = nsplit;
        sg.chunks_per_split = cps;
        const int64_t X = sg.Rp / rows, Z = (int64_t)d.batch * nsplit;
        const int64_t total = X * gy * Z;
        sg.X = (unsigned)X; sg.Y = (unsigned)gy; sg.Z = (unsigned)Z;
        sg.total = (unsigned)total;
        return total;
    };
    const bool has_tail = pl.rows_main < d.R;
    int64_t total = 0;
    if (has_tail) total += fill_seg(ka.seg[0], pl.rows_main, d.R, pl.tail_nsplit, pl.tail_chunks_per_split, pl.off_partial_tail);
    else ka.seg[0] = KArgs::Seg{0, 0, nullptr, 1, 0, 0, 0, 0, 0};
    total += fill_seg(ka.seg[1], 0, pl.rows_main, pl.nsplit, pl.chunks_per_split, pl.off_partial_main);
    if (total >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "workgroup count exceeds the grid limit");
    const dim3 grid((unsigned)total);
    if (lut.m > 7) launch_tn<true>(pl.TN, pl.WR, ka, grid, stream);
    else launch_tn<false>(pl.TN, pl.WR, ka, grid, stream);
    AMSIM_HIP_CHECK(hipGetLastError());

    for (int sgi = 0; sgi < 2; ++sgi) {
        const KArgs::Seg &sg = ka.seg[sgi];
        if (sg.total == 0 || sg.nsplit <= 1) continue;
        if (d.batch > 65535) return fail(AMSIM_ERR_UNSUPPORTED, "batch exceeds the grid limit");
        const int64_t row_end = sgi == 0 ? d.R : pl.rows_main;
        RArgs ra{sg.partial, d.out, row_end - sg.row_base, d.J, sg.Rp, d.so_r, d.so_j, d.out_batch_stride, pl.Jp,
                 sg.nsplit, d.batch, sg.row_base, ka.ep};
        launch_reduce(ra, stream);
        AMSIM_HIP_CHECK(hipGetLastError());
    }
    return AMSIM_OK;
}

// What does a 16-bit LDS load do to the register half it does not write?  One wavefront loads a
// byte into the upper half of a register that holds all ones.
__global__ __launch_bounds__(64) void d16_probe_kernel(uint32_t *out)
{
    __shared__ uint32_t cell[64];
    cell[threadIdx.x] = 0x5au;
    __syncthreads();
    uint32_t d = 0xffffffffu;
    asm volatile("ds_read_u8_d16_hi %0, %1\n\ts_waitcnt lgkmcnt(0)" : "+v"(d) : "v"(lds_address(&cell[threadIdx.x])));
    out[threadIdx.x] = d;
}

int probe_lds_d16_keeps(int *keeps)
{
    constexpr int MAX_DEVICES = 64;
    static std::atomic<int> cache[MAX_DEVICES];  // 0 unknown, 1 clears, 2 keeps
    int dev = 0;
    AMSIM_HIP_CHECK(hipGetDevice(&dev));
    if (dev >= 0 && dev < MAX_DEVICES && cache[dev].load() != 0) {
        *keeps = cache[dev].load() == 2;
        return AMSIM_OK;
    }
    uint32_t *d_out = nullptr, h_out[64];
    AMSIM_HIP_CHECK(hipMalloc(reinterpret_cast<void **>(&d_out), sizeof(h_out)));
    d16_probe_kernel<<<1, 64, 0, nullptr>>>(d_out);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpy(h_out, d_out, sizeof(h_out), hipMemcpyDeviceToHost);
    (void)hipFree(d_out);
    if (e != hipSuccess) return fail(AMSIM_ERR_HIP, std::string("LDS load probe: ") + hipGetErrorString(e));
    for (int i = 0; i < 64; ++i)
        if (h_out[i] != h_out[0] || (h_out[0] != 0x005a0000u && h_out[0] != 0x005affffu))
            return fail(AMSIM_ERR_UNSUPPORTED, "unexpected result of a 16-bit LDS load on this device");
    *keeps = h_out[0] == 0x005affffu;
    if (dev >= 0 && dev < MAX_DEVICES) cache[dev].store(*keeps ? 2 : 1);
    return AMSIM_OK;
}

// ---------------------------------------------------------------------------
// elementwise product (test hook)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(WG_THREADS) void mul_kernel(const uint32_t *lut32, int m, const float *a,
                                                         const float *b, float *out, size_t n)
{
    size_t i = (size_t)blockIdx.x * WG_THREADS + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * WG_THREADS;
    for (; i < n; i += stride) {
        const uint32_t at = f2u(a[i]), bt = f2u(b[i]);
        const uint32_t ma = (at & 0x7fffffu) >> (23 - m), mb = (bt & 0x7fffffu) >> (23 - m);
        out[i] = am_exact(at, bt, lut32[(ma << m) | mb]);
    }
}

int launch_mul(const Lut &lut, const float *a, const float *b, float *out, size_t n, hipStream_t stream)
{
    if (n == 0) return AMSIM_OK;
    if (const int rc = check_lut_device(lut)) return rc;
    const unsigned blocks = (unsigned)std::min<size_t>((n + WG_THREADS - 1) / WG_THREADS, 65535u * 16u);
    mul_kernel<<<blocks, WG_THREADS, 0, stream>>>(lut.lut32, lut.m, a, b, out, n);
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

void set_split_k(int mode) { g_split_k.store(mode ? 1 : 0); }
void set_engine(int mode) { g_engine.store(mode); }

}  // namespace amsim
