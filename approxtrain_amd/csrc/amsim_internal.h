// Internal declarations shared by the amsim translation units (not installed).
#ifndef AMSIM_INTERNAL_H_
#define AMSIM_INTERNAL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <string>

#include "amsim.h"

namespace amsim {

// ---- error plumbing ---------------------------------------------------------
void set_error(const std::string &msg);
int fail(int status, const std::string &msg);
#define AMSIM_HIP_CHECK(expr)                                                                       \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return ::amsim::fail(AMSIM_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

// ---- LUT handle -------------------------------------------------------------
// Device images of one mantissa-product table.
//   img_ab[(ma << m) | mb]  one byte per entry: carry << 7 | mantissa << (7 - m)
//   img_ba[(mb << m) | ma]  the same table transposed
// (m <= 7 only; both are padded to a multiple of 16 bytes; staged into LDS),
//   img16_ab / img16_ba     the same with 16-bit entries for 8 <= m <= 11
// (gathered from global memory), and
//   lut32[(ma << m) | mb]   carry << 23 | mantissa << (23 - m)   (every m)
struct Lut {
    int m = 0;
    int device = 0;
    int split_k = -1;  // how reductions may be run for calls through this handle: -1 process default, 0 whole, 1 split
    int engine = -1;   // which GEMM engine serves calls through this handle: -1 process default, else AMSIM_ENGINE_*
    size_t entries = 0;
    uint8_t *img_ab = nullptr;
    uint8_t *img_ba = nullptr;
    uint32_t *lut32 = nullptr;
    // m > 7 only: carry << 15 | mantissa << (15 - m), and its transpose
    uint16_t *img16_ab = nullptr;
    uint16_t *img16_ba = nullptr;
    // this device's 16-bit LDS loads keep (1) or clear (0) the register half they do not write
    int d16_keeps = 0;
    int d16_keeps_probed = 0;  // the probe's answer (d16_keeps may be forced to 1 by a test hook)
};

}  // namespace amsim

struct amsim_lut {
    amsim::Lut l;
};

namespace amsim {

// ---- the GEMM engine ----------------------------------------------------------
// out(r, j) = sum_k P(p(r, k), q(k, j)).  r is the dimension spread over the
// lanes of a wavefront ("lane operand" p), j the dimension kept wave-uniform
// ("uniform operand" q, pre-decoded into the workspace and read through the
// scalar cache).  lane_first tells which operand indexes the LUT row (ma).
enum PKind { P_DENSE = 0, P_PATCH = 1, P_GF = 2 };
enum QKind { Q_DENSE = 0, Q_FLIP = 1 };

struct PDesc {
    int kind = P_DENSE;
    const float *base = nullptr;
    int64_t batch_stride = 0;
    // P_DENSE: element (r, k) at base[r * sr + k * sk]
    int64_t sr = 0, sk = 0;
    // P_PATCH: r = (b, y, x) over [B, GH, GW], k = (fy, fx, c) over [KH, KW, C];
    //          source pixel (y*sy - pt + fy, x*sx - pl + fx) of [B, SH, SW, C], zero outside.
    // P_GF:    r = (fy, fx, c) over [KH, KW, C], k = (b, y, x) over [B, GH, GW];
    //          source pixel (y*sy - pt + fy, x*sx - pl + fx) of [B, SH, SW, C].
    int B = 0, GH = 0, GW = 0, KH = 0, KW = 0, C = 0;
    int sy = 1, sx = 1, pt = 0, pl = 0, SH = 0, SW = 0;
};

struct QDesc {
    int kind = Q_DENSE;
    const float *base = nullptr;
    int64_t batch_stride = 0;
    int batches = 1;  // 1 = shared by every batch item
    // Q_DENSE: element (k, j) at base[k * sk + j * sj]
    int64_t sk = 0, sj = 0;
    // Q_FLIP: k = (ty, tx, oc) over [TH, TW, OC], j = ic of an HWIO filter [KH, KW, IC, OC] read
    //         flipped, every (fsy, fsx)-th tap from (fy0, fx0): fy = fy0 + ty * fsy, fx = fx0 + tx * fsx,
    //         base[((KH-1-fy) * KW + (KW-1-fx)) * IC * OC + ic * OC + oc]
    int KH = 0, KW = 0, IC = 0, OC = 0;
    int TH = 0, TW = 0, fy0 = 0, fx0 = 0, fsy = 1, fsx = 1;
};

// Optional scatter of the output rows: row r = (b, y, x) over [B, GH, GW] is stored at pixel
// (b, y * sy + oy, x * sx + ox) of a [B, H, W] image (so_r elements per pixel).
struct OutMap {
    int enabled = 0;
    int GH = 0, GW = 0, sy = 1, sx = 1, oy = 0, ox = 0, H = 0, W = 0;
};

struct GemmDesc {
    PDesc p;
    QDesc q;
    int64_t R = 0, J = 0, K = 0;
    int batch = 1;
    float *out = nullptr;
    int64_t so_r = 0, so_j = 0, out_batch_stride = 0;
    bool lane_first = true;
    // optional epilogue on every output element: + bias (indexed by j or by r, whichever
    // dimension carries the output channels), then the activation
    const float *bias_j = nullptr, *bias_r = nullptr;
    int act = AMSIM_ACT_NONE;
    OutMap omap;
    bool no_split = false;  // keep every reduction whole (needs no partial-sum workspace)
};

// Compute units of the current device (read once per device; 256 when no device answers, which
// only steers work splitting, never correctness).
int device_compute_units();
// AMSIM_OK when the handle's images live on the current device, else AMSIM_ERR_INVALID.
int check_lut_device(const Lut &lut);
// how 16-bit LDS loads treat the other register half on the current device (probed once per device)
int probe_lds_d16_keeps(int *keeps);

size_t gemm_workspace_bytes(int64_t R, int64_t J, int64_t K, int batch, int q_batches);
void gemm_plan_info(int64_t R, int64_t J, int64_t K, int batch, int q_batches, bool split_k, int waves64, int64_t info[8]);
int run_gemm(const Lut &lut, const GemmDesc &d, void *workspace, size_t workspace_bytes, hipStream_t stream);

// ---- the row-staged engine for tables too wide for the LDS (mantissa widths 8..11) ----------
// Serves problems with at least WIDE_MIN_ROWS rows per batch item (dense, convolution patches,
// filter-gradient gathers) when the caller's workspace also holds the transposed lane operand and
// the partial sums of a sliced reduction (wide_workspace_bytes on top of the unsplit plan);
// everything else with such tables runs on the LDS-table engine's global-gather variant.
constexpr int64_t WIDE_MIN_ROWS = 512;
struct WideQ {
    const uint32_t *qw;
    const uint32_t *qflags;
    const QDesc *qdesc;
    int Jp, nchunks;
};
bool wide_shape_eligible(int64_t R, int batch);
bool wide_eligible(int m, const GemmDesc &d, bool may_split);
size_t wide_workspace_bytes(int64_t R, int64_t J, int64_t K, int batch);
// what the engine needs on top of the unsplit plan when a convolution's patches are read from a
// channel-major copy of the source (its own size) instead of an im2col; 0 when that form does not apply
size_t wide_workspace_bytes_planar(const GemmDesc &d);
// planar: wide_ws holds wide_workspace_bytes_planar(d), else wide_workspace_bytes(...)
int run_gemm_wide(const Lut &lut, const GemmDesc &d, const WideQ &q, void *wide_ws, bool planar, bool may_split, hipStream_t stream);
// workspace that serves a dense problem with any table: the larger of gemm_workspace_bytes and
// what the row-staged engine needs
size_t gemm_workspace_bytes_any_lut(int64_t R, int64_t J, int64_t K, int batch, int q_batches);
// what the row-staged engine needs for a problem in all (unsplit plan + transposed lane operand)
size_t gemm_workspace_bytes_wide(int64_t R, int64_t J, int64_t K, int batch, int q_batches);
// ... and with a convolution's patches read from a channel-major copy of the source instead of an
// im2col (0 when that form does not apply)
size_t gemm_workspace_bytes_wide_planar(const GemmDesc &d);

// ---- the direct engine for small problems (one launch, operands read where they lie) ----------
// Tables that fit the LDS only; which problems it takes is decided in direct_eligible().
constexpr double DIRECT_MAX_MACS = 48.0e6;          // padded products; outputs of more than 16 columns
constexpr double DIRECT_MAX_MACS_16 = 200.0e6;       // ... of 9 to 16 columns
constexpr double DIRECT_MAX_MACS_NARROW = 400.0e6;   // ... of at most 8 columns
constexpr double DIRECT_MAX_MACS_ANY = 1.0e10;
bool direct_shape_eligible(int64_t R, int64_t J, int64_t K, int batch, bool any_size);
bool direct_eligible(int m, const GemmDesc &d, bool any_size);
size_t direct_workspace_bytes(int64_t R, int64_t J, int64_t K, int batch);
int run_gemm_direct(const Lut &lut, const GemmDesc &d, bool may_split, void *workspace, size_t workspace_bytes, hipStream_t stream);

// ---- filter gradients of small layers: the reduction over the lanes ----------------------------
// At most KLANES_MAX_ROWS filter elements, a long reduction (pixels), tables that fit the LDS,
// reductions that may be split: see amsim_gemm_klanes.hip.
constexpr int64_t KLANES_MAX_ROWS = 32;
constexpr int64_t KLANES_MAX_OUTPUTS = 4096;
constexpr int64_t KLANES_MIN_REDUCTION = 2048;
// the shape part of klanes_eligible (what the workspace query can know)
bool klanes_shape_eligible(int64_t R, int64_t J, int64_t K, int batch);
bool klanes_eligible(int m, const GemmDesc &d);
size_t klanes_workspace_bytes(int64_t R, int64_t J, int64_t K);
int run_gemm_klanes(const Lut &lut, const GemmDesc &d, void *workspace, size_t workspace_bytes, hipStream_t stream);

int launch_mul(const Lut &lut, const float *a, const float *b, float *out, size_t n, hipStream_t stream);

// Strided grad-input runs one sub-problem per residue class of the input pixels, each over the
// filter taps that meet gradient samples.  The reference multiplies the other taps too, with the
// zeros it inserted between the samples: harmless (+0) unless such a weight is inf or NaN, when
// 0 x w = NaN reaches every pixel of the class.  This kernel writes, per class and input channel,
// NaN if a skipped tap holds a non-finite weight and +0 otherwise; the sub-problem adds it as a
// bias.  A class's own taps are flipped-filter indices f0 + t * stride, t < taps, on each axis.
struct TapClass {
    int fy0, fsy, th, fx0, fsx, tw;
};
constexpr int MAX_TAP_CLASSES = 16;  // classes handled by one launch
int launch_skipped_tap_poison(const float *filter, int KH, int KW, int IC, int OC, const TapClass *classes,
                              int n_classes, float *out, int out_stride, hipStream_t stream);

// attention row kernels (in place): scores -> softmax(scores / divisor - 1e9 * mask), and
// d(weights) -> d(scores); mask element (b, r, j) at mask[(b / batch_div) * batch_stride + r * row_stride + j]
int launch_softmax_rows(float *scores, const float *mask, int mask_batch_div, int64_t mask_batch_stride,
                        int64_t mask_row_stride, int64_t batch, int seq_q, int seq_k, float divisor,
                        hipStream_t stream);
int launch_softmax_grad_rows(const float *weights, float *grad, int64_t rows, int seq_k, float divisor,
                             hipStream_t stream);

}  // namespace amsim
#endif
