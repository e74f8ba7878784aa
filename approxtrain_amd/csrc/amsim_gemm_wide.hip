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
constexpr int WIDE_SLOT_BYTES = 4096;             // LDS bytes reserved per staged table row (2^11 entries x 2)
constexpr int PT_ROWS = 64;                       // rows per workgroup of the transposing pre-pass

struct PTArgs {
    PDesc p;
    int64_t R, K, Rp;
    int nchunks;
    uint32_t *pt;      // [batch][nchunks * KC][Rp] raw bits
    uint32_t *pflags;  // [batch][nchunks][Rp / 64]
};

// One workgroup per (64-row group, 32-deep chunk) and batch item (blockIdx.y): reads the tile along
// the source's contiguous direction -- for patch sources this IS the im2col the reference
// materialises (cuda/cuda_kernel.cu:35-60), here transposed -- writes it in [k][row] order, flags it
// if it holds an operand the fast product path cannot take.
__global__ __launch_bounds__(WG_THREADS) void p_linear_kernel(PTArgs a)
{
    __shared__ uint32_t tile[KC][PT_ROWS + 1];
    const int64_t G = a.Rp / PT_ROWS;
    const int64_t g = blockIdx.x % G, ch = blockIdx.x / G;
    const int bz = blockIdx.y;
    const int tid = threadIdx.x;
    const float *pbase = a.p.base + (int64_t)bz * a.p.batch_stride;
    uint32_t *pt = a.pt + (size_t)bz * a.nchunks * KC * a.Rp;
    // lanes along k where the source is contiguous there: row-major dense operands, and patches
    // (channels run fastest in both the image and the reduction index)
    const bool k_fast = a.p.kind == P_PATCH || (a.p.kind == P_DENSE && a.p.sk == 1 && a.p.sr != 1);
    int unsafe = 0;
#pragma unroll
    for (int i = 0; i < KC * PT_ROWS / WG_THREADS; ++i) {
        const int e = tid + WG_THREADS * i;
        int kk, rl;
        if (k_fast) { kk = e % KC; rl = e / KC; }
        else { rl = e % PT_ROWS; kk = e / PT_ROWS; }
        const int64_t r = g * PT_ROWS + rl, k = ch * KC + kk;
        const uint32_t raw = p_raw_bits(a.p, pbase, a.R, a.K, r, k);
        unsafe |= operand_unsafe(raw) ? 1 : 0;
        tile[kk][rl] = raw;
    }
    const int any = __syncthreads_or(unsafe);
#pragma unroll
    for (int i = 0; i < KC * PT_ROWS / WG_THREADS; ++i) {
        const int e = tid + WG_THREADS * i;
        const int rl = e % PT_ROWS, kk = e / PT_ROWS;
        pt[(size_t)(ch * KC + kk) * a.Rp + g * PT_ROWS + rl] = tile[kk][rl];
    }
    if (tid == 0) a.pflags[((size_t)bz * a.nchunks + ch) * G + g] = (uint32_t)any;
}

// LDS byte address of a pointer into a __shared__ object
__device__ __forceinline__ uint32_t lds_addr(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// The 8 entries at addr + j * 4 KB (one per staged table row), issued back to back and waited for
// together.  Written as one block so that the gathers of a row group stay 8 registers wide (left to
// itself the scheduler hoists all 64 of a stage and spills accumulators), and so that the compiler
// does not order them behind the direct-to-LDS copies in flight for the next stage, which write the
// other half of the buffer.
__device__ __forceinline__ void gather8(uint32_t addr, uint32_t (&e)[8])
{
    asm volatile(
        "ds_read_u16 %0, %8\n\t"
        "ds_read_u16 %1, %8 offset:4096\n\t"
        "ds_read_u16 %2, %8 offset:8192\n\t"
        "ds_read_u16 %3, %8 offset:12288\n\t"
        "ds_read_u16 %4, %8 offset:16384\n\t"
        "ds_read_u16 %5, %8 offset:20480\n\t"
        "ds_read_u16 %6, %8 offset:24576\n\t"
        "ds_read_u16 %7, %8 offset:28672\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(e[0]), "=&v"(e[1]), "=&v"(e[2]), "=&v"(e[3]), "=&v"(e[4]), "=&v"(e[5]), "=&v"(e[6]), "=&v"(e[7])
        : "v"(addr)
        : "memory");
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
};

// PARTS: KB of a table row copied per stage and slot (4 at width 11, 2 at width 10, 1 below: the copy
// of a narrower row runs on into the rows behind it, which the image's padding keeps in bounds).
// RPT: rows per thread, 8 (4096 rows per workgroup: 1 byte of table row pulled per product) or 4 (2048
// rows, 2 bytes per product: for problems that would otherwise leave compute units without a workgroup).
template <int PARTS, int RPT>
__global__ __launch_bounds__(WIDE_THREADS, 4) void lutgemm_wide_kernel(WArgs a)
{
    constexpr int TILE_ROWS = WIDE_THREADS * RPT;
    constexpr int WIDE_BUF_BYTES = WIDE_TN * WIDE_SLOT_BYTES;
    // Two halves of 8 slots x 4 KB, as two objects: the compiler then knows that the direct-to-LDS
    // copies into one half do not alias the gathers from the other, and does not make the gathers
    // wait for the copies.
    __shared__ __align__(16) uint8_t rows_a[WIDE_BUF_BYTES];
    __shared__ __align__(16) uint8_t rows_b[WIDE_BUF_BYTES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    const int m = a.m, mshift = 23 - m;
    const uint32_t mmask = (1u << m) - 1u;
    const int Kp = a.nchunks * KC;
    const int bz = blockIdx.y, qb = a.q_batches > 1 ? bz : 0;
    const size_t qt_index = (size_t)qb * (a.Jp / QT) + by / STRIPS_PER_TILE;  // tile of the pre-decoded operand
    const cq1_t qtile = (cq1_t)(uintptr_t)(a.qw + qt_index * Kp * QT + (by % STRIPS_PER_TILE) * WIDE_TN);
    const cq1_t qfl = (cq1_t)(uintptr_t)(a.qflags + qt_index * a.nchunks);
    const uint32_t *pcol = a.pt + (size_t)bz * Kp * a.Rp + row0 + tid;
    const int64_t G = a.Rp / PT_ROWS;
    const uint32_t *pfl = a.pflags + (size_t)bz * a.nchunks * G;
    float acc[RPT][WIDE_TN];
#pragma unroll
    for (int rr = 0; rr < RPT; ++rr)
#pragma unroll
        for (int j = 0; j < WIDE_TN; ++j) acc[rr][j] = 0.0f;

    // wavefront w copies the table row of column j0 + w for stage k into half `buf`
    auto fill = [&](int k, uint8_t *half) {
        const uint32_t w = qtile[k * QT + wave];
        const uint8_t *src = a.lut16 + (size_t)(w & 0x7fffffu) * 2 + lane * 16;
        uint8_t *dst = half + wave * WIDE_SLOT_BYTES;
#pragma unroll
        for (int part = 0; part < PARTS; ++part) {  // every lane, every part: no branch inside a stage
#if defined(__HIP_DEVICE_COMPILE__)  // the builtin exists in the device pass only
            __builtin_amdgcn_global_load_lds(src + part * 1024, dst + part * 1024, 16, 0, 0);
#endif
        }
    };
    uint32_t pc[RPT], pn[RPT];
    auto load_p = [&](int k, uint32_t (&dst)[RPT]) {
#pragma unroll
        for (int rr = 0; rr < RPT; ++rr) dst[rr] = pcol[(size_t)k * a.Rp + rr * WIDE_THREADS];
    };

    fill(0, rows_a);
    load_p(0, pc);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // Is any chunk of this workgroup's tile flagged (by its column tile or by a 64-row group of its
    // row tile)?  Almost never: then the whole reduction runs the loop nest that holds nothing but
    // fast stages, whose registers the rare path's state cannot crowd.
    int tile_flagged = 0;
    for (int ch = tid; ch < a.nchunks; ch += WIDE_THREADS)
        tile_flagged |= (int)a.qflags[qt_index * a.nchunks + ch];
    for (int i = tid; i < a.nchunks * (TILE_ROWS / PT_ROWS); i += WIDE_THREADS)
        tile_flagged |= (int)pfl[(size_t)(i / (TILE_ROWS / PT_ROWS)) * G + (size_t)bx * (TILE_ROWS / PT_ROWS) +
                                 i % (TILE_ROWS / PT_ROWS)];
    tile_flagged = __syncthreads_or(tile_flagged);

    // one stage: copies for stage k + 1 go into `next` while stage k gathers from `cur`
    auto stage = [&](auto exact_tag, int k, const uint8_t *cur, uint8_t *next) {
        constexpr bool EXACT = decltype(exact_tag)::value;
        // (the last stage copies its own rows and operands once more instead of branching: a
        // straight-line stage keeps the compiler from sinking one stage's FMAs into the next)
        const int kn = min(k + 1, Kp - 1);
        fill(kn, next);  // everyone left that half at the barrier that ended the stage before
        load_p(kn, pn);
        if constexpr (!EXACT) {
            uint32_t qt[WIDE_TN];
#pragma unroll
            for (int j = 0; j < WIDE_TN; ++j) qt[j] = qtile[k * QT + j] & 0xff800000u;
#pragma unroll
            for (int rr = 0; rr < RPT; ++rr) {
                const float ta = u2f(pc[rr] & 0xff800000u);
                const uint32_t off = ((pc[rr] >> mshift) & mmask) << 1;
                uint32_t e[WIDE_TN];
                gather8(lds_addr(cur) + off, e);
#pragma unroll
                for (int j = 0; j < WIDE_TN; ++j)
                    // (entry << 8) + sign|exponent bits of q  ==  q_pow2 * 1.mant * 2^carry, exactly
                    acc[rr][j] = __builtin_fmaf(ta, u2f((e[j] << 8) + qt[j]), acc[rr][j]);
            }
        } else {
            // Rare: full-domain product; q's raw bits come from where the operand lies.  The
            // accumulators take a detour through private memory so that this loop can index them
            // dynamically (small code, one product at a time) while the fast path keeps them in
            // registers.
            const __attribute__((address_space(4))) QDesc &qd = *(const __attribute__((address_space(4))) QDesc *)(uintptr_t)a.qdesc;
            const float *qsrc = qd.base;
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
                const uint32_t off = ((raw >> mshift) & mmask) << 1;
                const uint32_t e16 = (uint32_t)*reinterpret_cast<const uint16_t *>(cur + off + j * WIDE_SLOT_BYTES) << 8;
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
        // my copies for the next stage have landed; after the barrier so have everyone's, and
        // every wavefront is done gathering from this stage's half
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };
    if (!tile_flagged) {
#pragma unroll 1
        for (int k = 0; k < Kp; k += 2) {
            stage(std::false_type{}, k, rows_a, rows_b);
            stage(std::false_type{}, k + 1, rows_b, rows_a);
        }
    } else {
        for (int ch = 0; ch < a.nchunks; ++ch) {
            const uint32_t pf = lane < TILE_ROWS / PT_ROWS ? pfl[(size_t)ch * G + (size_t)bx * (TILE_ROWS / PT_ROWS) + lane] : 0u;
            const bool unsafe = (qfl[ch] != 0u) | (__any(pf != 0u) != 0);
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
inline int64_t padded_rows(int64_t R) { return (R + WIDE_TILE_ROWS - 1) / WIDE_TILE_ROWS * WIDE_TILE_ROWS; }

}  // namespace

bool wide_shape_eligible(int64_t R, int batch) { return batch >= 1 && batch <= 65535 && R >= WIDE_MIN_ROWS; }

// Dense and patch (forward / input-gradient convolution) lane operands; the filter gradient's rows
// are the few filter elements and its reduction the many pixels, the opposite of what this engine
// needs, so it stays on the global-gather variant.
bool wide_eligible(int m, const GemmDesc &d)
{
    return m > 7 && (d.p.kind == P_DENSE || d.p.kind == P_PATCH) && wide_shape_eligible(d.R, d.batch);
}

size_t wide_workspace_bytes(int64_t R, int64_t K, int batch)
{
    const int64_t Rp = padded_rows(R), nchunks = (K + KC - 1) / KC;
    return align256((size_t)batch * nchunks * KC * Rp * sizeof(uint32_t)) +
           align256((size_t)batch * nchunks * (Rp / PT_ROWS) * sizeof(uint32_t));
}

int run_gemm_wide(const Lut &lut, const GemmDesc &d, const WideQ &q, void *wide_ws, hipStream_t stream)
{
    const int64_t Rp = padded_rows(d.R);
    const int64_t G = Rp / PT_ROWS;
    uint8_t *ws = static_cast<uint8_t *>(wide_ws);
    PTArgs pa{};
    pa.p = d.p; pa.R = d.R; pa.K = d.K; pa.Rp = Rp; pa.nchunks = q.nchunks;
    pa.pt = reinterpret_cast<uint32_t *>(ws);
    pa.pflags = reinterpret_cast<uint32_t *>(ws + align256((size_t)d.batch * q.nchunks * KC * Rp * sizeof(uint32_t)));
    const int64_t pwgs = G * q.nchunks;
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
    // half-height tiles when full-height ones would leave workgroup slots (two per compute unit) empty
    const int64_t strips = q.Jp / WIDE_TN;
    const bool half = (Rp / WIDE_TILE_ROWS) * strips * d.batch < 2 * (int64_t)device_compute_units();
    const int tile_rows = half ? WIDE_TILE_ROWS / 2 : WIDE_TILE_ROWS;
    wa.X = (unsigned)((d.R + tile_rows - 1) / tile_rows);
    wa.Y = (unsigned)strips;
    const int64_t total = (int64_t)wa.X * wa.Y;
    if (total >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "workgroup count exceeds the grid limit");
    const dim3 grid((unsigned)total, (unsigned)d.batch);
    const int parts = lut.m >= 11 ? 4 : lut.m == 10 ? 2 : 1;
    if (half) {
        if (parts == 4) lutgemm_wide_kernel<4, 4><<<grid, WIDE_THREADS, 0, stream>>>(wa);
        else if (parts == 2) lutgemm_wide_kernel<2, 4><<<grid, WIDE_THREADS, 0, stream>>>(wa);
        else lutgemm_wide_kernel<1, 4><<<grid, WIDE_THREADS, 0, stream>>>(wa);
    } else {
        if (parts == 4) lutgemm_wide_kernel<4, 8><<<grid, WIDE_THREADS, 0, stream>>>(wa);
        else if (parts == 2) lutgemm_wide_kernel<2, 8><<<grid, WIDE_THREADS, 0, stream>>>(wa);
        else lutgemm_wide_kernel<1, 8><<<grid, WIDE_THREADS, 0, stream>>>(wa);
    }
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

}  // namespace amsim
