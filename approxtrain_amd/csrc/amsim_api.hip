// extern "C" entry points: each one describes its reduction to the GEMM engine
// (which operand runs over the lanes, which is wave-uniform, how the lane
// operand is gathered) and launches it.  No device memory is allocated here.
#include "amsim_internal.h"
#include "amsim_bench.h"

#include <algorithm>
#include <mutex>
#include <string>

namespace amsim {
void set_split_k(int mode);
void set_engine(int mode);
}

using namespace amsim;

namespace {

inline int tn_for(int64_t J) { return J >= 9 ? 16 : J >= 5 ? 8 : J >= 3 ? 4 : (int)std::max<int64_t>(J, 1); }

inline int64_t padded_work(int64_t R, int64_t J)
{
    const int tn = tn_for(J);
    return ((R + 63) / 64 * 64) * ((J + tn - 1) / tn * tn);
}

// true: rows of C over the lanes (lane operand = op(A)); false: columns of C
// over the lanes (lane operand = op(B)).  Picks the cheaper orientation: the MACs spent
// including lanes / accumulators wasted on padding (~13 TMAC/s), plus the pre-decode of the
// uniform operand, which moves about 12 bytes per element (~4 TB/s).
inline double orientation_cost(int64_t R, int64_t J, int64_t K)
{
    return (double)padded_work(R, J) * (double)K / 13.0e12 + 12.0 * (double)K * (double)J / 4.0e12;
}
inline bool lanes_along_m(int64_t M, int64_t N, int64_t K) { return orientation_cost(M, N, K) <= orientation_cost(N, M, K); }

struct GemmCall {
    int transA, transB, swap;
    int64_t M, N, K;
    const float *A; int64_t lda;
    const float *B; int64_t ldb;
    float *C; int64_t ldc;
    int64_t batch, strideA, strideB, strideC;
    const float *bias_n = nullptr;  // optional: added to C[.][n]
    int act = AMSIM_ACT_NONE;
};

// wide_table: the LUT is too wide for the LDS (mantissa width above 7).  The row-staged engine that
// serves such tables wants as many rows over the lanes as it can get, so the longer of M and N
// goes there when that makes the problem eligible for it.
GemmDesc describe(const GemmCall &g, bool wide_table)
{
    GemmDesc d;
    d.K = g.K;
    d.batch = (int)g.batch;
    d.out = g.C;
    d.out_batch_stride = g.strideC;
    bool along_m = lanes_along_m(g.M, g.N, g.K);
    if (wide_table && wide_shape_eligible(std::max(g.M, g.N), (int)g.batch)) along_m = g.M >= g.N;
    if (along_m) {
        d.R = g.M; d.J = g.N;
        d.p.kind = P_DENSE; d.p.base = g.A; d.p.batch_stride = g.strideA;
        d.p.sr = g.transA ? 1 : g.lda; d.p.sk = g.transA ? g.lda : 1;
        d.q.kind = Q_DENSE; d.q.base = g.B; d.q.batch_stride = g.strideB;
        d.q.batches = (g.batch > 1 && g.strideB != 0) ? (int)g.batch : 1;
        d.q.sk = g.transB ? 1 : g.ldb; d.q.sj = g.transB ? g.ldb : 1;
        d.so_r = g.ldc; d.so_j = 1;
        d.bias_j = g.bias_n;
        d.lane_first = !g.swap;
    } else {
        d.R = g.N; d.J = g.M;
        d.p.kind = P_DENSE; d.p.base = g.B; d.p.batch_stride = g.strideB;
        d.p.sr = g.transB ? g.ldb : 1; d.p.sk = g.transB ? 1 : g.ldb;
        d.q.kind = Q_DENSE; d.q.base = g.A; d.q.batch_stride = g.strideA;
        d.q.batches = (g.batch > 1 && g.strideA != 0) ? (int)g.batch : 1;
        d.q.sk = g.transA ? g.lda : 1; d.q.sj = g.transA ? 1 : g.lda;
        d.so_r = 1; d.so_j = g.ldc;
        d.bias_r = g.bias_n;
        d.lane_first = g.swap != 0;
    }
    d.act = g.act;
    return d;
}

bool known_activation(int act) { return act == AMSIM_ACT_NONE || act == AMSIM_ACT_RELU; }

int gemm_call(amsim_lut_t lut, const GemmCall &g, void *ws, size_t ws_bytes, void *stream)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (g.M < 0 || g.N < 0 || g.K < 0 || g.batch < 0) return fail(AMSIM_ERR_INVALID, "negative extent");
    if (g.M == 0 || g.N == 0 || g.batch == 0) return AMSIM_OK;
    if (g.C == nullptr || (g.K > 0 && (g.A == nullptr || g.B == nullptr)))
        return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    const int64_t min_lda = g.transA ? g.M : g.K, min_ldb = g.transB ? g.K : g.N;
    if (g.lda < min_lda || g.ldb < min_ldb || g.ldc < g.N)
        return fail(AMSIM_ERR_INVALID, "leading dimension smaller than the row length");
    return run_gemm(lut->l, describe(g, lut->l.m > 7), ws, ws_bytes, static_cast<hipStream_t>(stream));
}

// lut == nullptr: valid for any table (the orientation, and with it the engine, depends on the table's
// width: the larger of both); else what calls through that handle need -- tables that fit the LDS
// never read the row-staged engine's transposed operand copy, most of the table-agnostic figure.
size_t gemm_ws(const GemmCall &g, amsim_lut_t lut = nullptr)
{
    if (g.M <= 0 || g.N <= 0 || g.K <= 0 || g.batch <= 0) return 0;
    const GemmDesc d = describe(g, false), w = describe(g, true);
    if (lut != nullptr && lut->l.m <= 7) return gemm_workspace_bytes(d.R, d.J, d.K, d.batch, d.q.batches);
    if (lut != nullptr) return gemm_workspace_bytes_any_lut(w.R, w.J, w.K, w.batch, w.q.batches);
    return std::max(gemm_workspace_bytes_any_lut(d.R, d.J, d.K, d.batch, d.q.batches),
                    gemm_workspace_bytes_any_lut(w.R, w.J, w.K, w.batch, w.q.batches));
}

bool fits_int32(int64_t elements) { return elements < (1ll << 31); }

}  // namespace

extern "C" {

int amsim_set_split_k(int mode)
{
    amsim::set_split_k(mode);
    return AMSIM_OK;
}

int amsim_set_engine(int mode)
{
    if (mode != AMSIM_ENGINE_AUTO && mode != AMSIM_ENGINE_LDS_TABLE && mode != AMSIM_ENGINE_DIRECT)
        return fail(AMSIM_ERR_INVALID, "unknown engine mode");
    amsim::set_engine(mode);
    return AMSIM_OK;
}

int amsim_mul_f32(amsim_lut_t lut, const float *a, const float *b, float *out, size_t n, void *stream)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (n && (!a || !b || !out)) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    return launch_mul(lut->l, a, b, out, n, static_cast<hipStream_t>(stream));
}

size_t amsim_gemm_workspace_bytes(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t batch)
{
    // sized for per-item operands (no broadcast), the larger case
    GemmCall g{transA, transB, 0, M, N, K, nullptr, 0, nullptr, 0, nullptr, 0, batch, 1, 1, 1};
    return gemm_ws(g);
}

size_t amsim_gemm_workspace_bytes_for(amsim_lut_t lut, int transA, int transB, int64_t M, int64_t N, int64_t K,
                                      int64_t batch)
{
    GemmCall g{transA, transB, 0, M, N, K, nullptr, 0, nullptr, 0, nullptr, 0, batch, 1, 1, 1};
    return gemm_ws(g, lut);
}

int amsim_gemm_plan_info(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t batch, int64_t info[8])
{
    if (!info || M <= 0 || N <= 0 || K <= 0 || batch <= 0) return fail(AMSIM_ERR_INVALID, "bad plan query");
    GemmCall g{transA, transB, 0, M, N, K, nullptr, transA ? M : K, nullptr, transB ? K : N, nullptr, N, batch, 1, 1, 1};
    const GemmDesc d = describe(g, false);
    // contiguous, aligned operands assumed (the float4-staged kernel variants)
    gemm_plan_info(d.R, d.J, d.K, d.batch, d.q.batches, true, d.p.sk == 1 && d.p.sr != 1 ? 6 : 5, info);
    return AMSIM_OK;
}

int amsim_gemm_f32(amsim_lut_t lut, int transA, int transB, int swap_operands, int64_t M, int64_t N, int64_t K,
                   const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                   int64_t batch, int64_t strideA, int64_t strideB, int64_t strideC, void *workspace,
                   size_t workspace_bytes, void *stream)
{
    GemmCall g{transA, transB, swap_operands, M, N, K, A, lda, B, ldb, C, ldc, batch, strideA, strideB, strideC};
    return gemm_call(lut, g, workspace, workspace_bytes, stream);
}

// ---- convolution ------------------------------------------------------------------

}  // extern "C"

namespace {
// im2col rows (b, oy, ox) x columns (fy, fx, c)  [cuda_kernel.cu:35-60], filter as the [K][OC] matrix
GemmDesc forward_desc(int batch, int out_rows, int out_cols, int out_depth, int stride_cols, int stride_rows,
                      int filter_left_offset, int filter_top_offset, int filter_rows, int filter_cols, int in_depth,
                      int input_cols, int input_rows)
{
    GemmDesc d;
    d.R = (int64_t)batch * out_rows * out_cols; d.J = out_depth; d.K = (int64_t)filter_rows * filter_cols * in_depth;
    d.p.kind = P_PATCH;
    d.p.B = batch; d.p.GH = out_rows; d.p.GW = out_cols;
    d.p.KH = filter_rows; d.p.KW = filter_cols; d.p.C = in_depth;
    d.p.sy = stride_rows; d.p.sx = stride_cols; d.p.pt = filter_top_offset; d.p.pl = filter_left_offset;
    d.p.SH = input_rows; d.p.SW = input_cols;
    d.q.kind = Q_DENSE; d.q.sk = out_depth; d.q.sj = 1;
    d.so_r = out_depth; d.so_j = 1;
    d.lane_first = true;  // P(input, filter)
    return d;
}
}  // namespace

extern "C" {

size_t amsim_convam_workspace_bytes(int batch, int out_rows, int out_cols, int out_depth, int filter_rows,
                                    int filter_cols, int in_depth)
{
    return gemm_workspace_bytes((int64_t)batch * out_rows * out_cols, out_depth,
                                (int64_t)filter_rows * filter_cols * in_depth, 1, 1);
}

size_t amsim_convam_workspace_bytes_for(amsim_lut_t lut, int batch, int out_rows, int out_cols, int out_depth,
                                        int filter_rows, int filter_cols, int in_depth)
{
    size_t need = amsim_convam_workspace_bytes(batch, out_rows, out_cols, out_depth, filter_rows, filter_cols, in_depth);
    if (need && lut != nullptr && lut->l.m > 7)  // + the im2col the row-staged engine gathers from
        need = std::max(need, gemm_workspace_bytes_wide((int64_t)batch * out_rows * out_cols, out_depth,
                                                        (int64_t)filter_rows * filter_cols * in_depth, 1, 1));
    return need;
}

size_t amsim_convam_lean_workspace_bytes_for(amsim_lut_t lut, int batch, int out_rows, int out_cols, int out_depth,
                                             int filter_rows, int filter_cols, int in_depth, int stride_rows,
                                             int stride_cols)
{
    size_t need = amsim_convam_workspace_bytes(batch, out_rows, out_cols, out_depth, filter_rows, filter_cols, in_depth);
    if (!need || lut == nullptr || lut->l.m <= 7 || stride_rows < 1 || stride_cols < 1) return need;
    // (the copy's extent follows from the output extent, the strides and the filter: the source's own
    // extent and the pads do not enter)
    const GemmDesc d = forward_desc(batch, out_rows, out_cols, out_depth, stride_cols, stride_rows, 0, 0, filter_rows,
                                    filter_cols, in_depth, (out_cols - 1) * stride_cols + filter_cols,
                                    (out_rows - 1) * stride_rows + filter_rows);
    return std::max(need, gemm_workspace_bytes_wide_planar(d));
}

int amsim_convam_f32(amsim_lut_t lut, const float *input_data, float *output_data, int batch, int out_rows,
                     int out_cols, int out_depth, int stride_cols, int stride_rows, int filter_left_offset,
                     int filter_top_offset, int filter_rows, int filter_cols, int in_depth, int input_cols,
                     int input_rows, const float *filter, void *workspace, size_t workspace_bytes, void *stream)
{
    return amsim_convam_bias_act_f32(lut, input_data, output_data, batch, out_rows, out_cols, out_depth, stride_cols,
                                     stride_rows, filter_left_offset, filter_top_offset, filter_rows, filter_cols,
                                     in_depth, input_cols, input_rows, filter, nullptr, AMSIM_ACT_NONE, workspace,
                                     workspace_bytes, stream);
}

int amsim_convam_bias_act_f32(amsim_lut_t lut, const float *input_data, float *output_data, int batch, int out_rows,
                              int out_cols, int out_depth, int stride_cols, int stride_rows,
                              int filter_left_offset, int filter_top_offset, int filter_rows, int filter_cols,
                              int in_depth, int input_cols, int input_rows, const float *filter, const float *bias,
                              int activation, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!known_activation(activation)) return fail(AMSIM_ERR_INVALID, "unknown activation");
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (batch < 0 || out_rows < 0 || out_cols < 0 || out_depth < 0 || filter_rows < 0 || filter_cols < 0 ||
        in_depth < 0 || input_cols < 0 || input_rows < 0 || stride_cols < 1 || stride_rows < 1)
        return fail(AMSIM_ERR_INVALID, "bad convolution geometry");
    const int64_t R = (int64_t)batch * out_rows * out_cols;
    if (R == 0 || out_depth == 0) return AMSIM_OK;
    if (!input_data || !output_data || !filter) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    if (!fits_int32((int64_t)batch * input_rows * input_cols * in_depth))
        return fail(AMSIM_ERR_UNSUPPORTED, "input tensor has 2^31 or more elements");
    GemmDesc d = forward_desc(batch, out_rows, out_cols, out_depth, stride_cols, stride_rows, filter_left_offset,
                              filter_top_offset, filter_rows, filter_cols, in_depth, input_cols, input_rows);
    d.p.base = input_data;
    d.q.base = filter;
    d.out = output_data;
    d.bias_j = bias; d.act = activation;
    return run_gemm(lut->l, d, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

// ---- allocation-free forward convolution ---------------------------------------------
// The scratch of amsim_convam_noalloc_f32: part of the device image, so it exists on every GPU
// the code object is loaded on, at an address of its own there.  In host code the array's name
// is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
static __device__ __align__(256) unsigned char noalloc_scratch[AMSIM_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int NOALLOC_MAX_DEVICES = 64;
std::mutex g_noalloc_lock;
void *g_noalloc_ptr[NOALLOC_MAX_DEVICES];  // device address of noalloc_scratch, per device (null = not asked yet)

// address of the scratch array on the current device, looked up once per device
int noalloc_scratch_ptr(void **out)
{
    int dev = 0;
    AMSIM_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return fail(AMSIM_ERR_UNSUPPORTED, "device index out of range");
    std::lock_guard<std::mutex> guard(g_noalloc_lock);
    if (g_noalloc_ptr[dev] == nullptr) {
        void *p = nullptr;
        AMSIM_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(noalloc_scratch)));
        if (p == nullptr || ((uintptr_t)p & 255)) return fail(AMSIM_ERR_HIP, "scratch symbol has no usable device address");
        g_noalloc_ptr[dev] = p;
    }
    *out = g_noalloc_ptr[dev];
    return AMSIM_OK;
}
}  // namespace

int amsim_convam_noalloc_f32(amsim_lut_t lut, const float *input_data, float *output_data, int batch, int out_rows,
                             int out_cols, int out_depth, int stride_cols, int stride_rows, int filter_left_offset,
                             int filter_top_offset, int filter_rows, int filter_cols, int in_depth, int input_cols,
                             int input_rows, const float *filter, void *stream)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (batch < 0 || out_rows < 0 || out_cols < 0 || out_depth < 0 || filter_rows < 0 || filter_cols < 0 || in_depth < 0)
        return fail(AMSIM_ERR_INVALID, "bad convolution geometry");
    const size_t need = amsim_convam_workspace_bytes(batch, out_rows, out_cols, out_depth, filter_rows, filter_cols, in_depth);
    if (need > AMSIM_NOALLOC_SCRATCH_BYTES)
        return fail(AMSIM_ERR_UNSUPPORTED, "problem needs " + std::to_string(need) + " bytes of scratch, the allocation-free "
                                           "entry point holds " + std::to_string(AMSIM_NOALLOC_SCRATCH_BYTES));
    void *scratch = nullptr;
    if (const int rc = noalloc_scratch_ptr(&scratch)) return rc;
    return amsim_convam_bias_act_f32(lut, input_data, output_data, batch, out_rows, out_cols, out_depth, stride_cols,
                                     stride_rows, filter_left_offset, filter_top_offset, filter_rows, filter_cols,
                                     in_depth, input_cols, input_rows, filter, nullptr, AMSIM_ACT_NONE, scratch,
                                     AMSIM_NOALLOC_SCRATCH_BYTES, stream);
}

// ---- grad-input ----------------------------------------------------------------------
// The reference dilates the gradient with (stride - 1) zeros between samples and multiplies
// every filter tap with it (cuda_kernel.cu:463-502, 569-583).  Input pixels whose row / column
// index has the same residue modulo the stride meet the same subset of taps (the others hit the
// inserted zeros, whose products are +0 and leave the FP32 sum unchanged), so the problem is
// run as stride_rows x stride_cols undilated sub-problems ("phases"), each over its own pixels
// and taps, in the reference's reduction order.  Stride 1 is the single phase (0, 0).
namespace {

struct Phase {
    int n_out;   // input pixels along this axis in the phase
    int taps;    // filter taps that meet gradient samples
    int f0;      // first such tap (index into the flipped filter)
    int pad;     // leading pad of the undilated patch: source = pixel - pad + tap
};

Phase phase_of(int extent, int stride, int residue, int filter, int back_pad)
{
    Phase ph;
    ph.n_out = residue < extent ? (extent - residue + stride - 1) / stride : 0;
    ph.f0 = ((back_pad - residue) % stride + stride) % stride;
    ph.taps = ph.f0 < filter ? (filter - ph.f0 + stride - 1) / stride : 0;
    ph.pad = -((residue - back_pad + ph.f0) / stride);  // exact: the numerator is a multiple of the stride
    return ph;
}

struct GradInputGeometry {
    int batch, input_rows, input_cols, in_depth, filter_rows, filter_cols, out_depth, out_rows, out_cols;
    int stride_rows, stride_cols, pad_top, pad_left;
};

// floats per residue class (a multiple of 64, so every class's vector is 256-byte aligned)
int poison_stride(int in_depth) { return (in_depth + 63) / 64 * 64; }
size_t poison_bytes(int in_depth) { return (size_t)MAX_TAP_CLASSES * poison_stride(in_depth) * sizeof(float); }

GemmDesc grad_input_phase(const GradInputGeometry &g, int py, int px, const float *grad, const float *filter,
                          float *output)
{
    const Phase y = phase_of(g.input_rows, g.stride_rows, py, g.filter_rows, g.pad_top);
    const Phase x = phase_of(g.input_cols, g.stride_cols, px, g.filter_cols, g.pad_left);
    GemmDesc d;
    d.R = (int64_t)g.batch * y.n_out * x.n_out;
    d.J = g.in_depth;
    d.K = (int64_t)y.taps * x.taps * g.out_depth;
    d.p.kind = P_PATCH; d.p.base = grad;
    d.p.B = g.batch; d.p.GH = y.n_out; d.p.GW = x.n_out;
    d.p.KH = y.taps; d.p.KW = x.taps; d.p.C = g.out_depth;
    d.p.sy = 1; d.p.sx = 1; d.p.pt = y.pad; d.p.pl = x.pad;
    d.p.SH = g.out_rows; d.p.SW = g.out_cols;
    d.q.kind = Q_FLIP; d.q.base = filter;
    d.q.KH = g.filter_rows; d.q.KW = g.filter_cols; d.q.IC = g.in_depth; d.q.OC = g.out_depth;
    d.q.TH = y.taps; d.q.TW = x.taps; d.q.fy0 = y.f0; d.q.fx0 = x.f0; d.q.fsy = g.stride_rows; d.q.fsx = g.stride_cols;
    d.out = output; d.so_r = g.in_depth; d.so_j = 1;
    d.omap.enabled = (g.stride_rows > 1 || g.stride_cols > 1) ? 1 : 0;
    d.omap.GH = y.n_out; d.omap.GW = x.n_out; d.omap.sy = g.stride_rows; d.omap.sx = g.stride_cols;
    d.omap.oy = py; d.omap.ox = px; d.omap.H = g.input_rows; d.omap.W = g.input_cols;
    d.lane_first = true;  // P(grad, filter)
    return d;
}

}  // namespace

size_t amsim_convam_input_grad_workspace_bytes(int batch, int input_rows, int input_cols, int in_depth,
                                               int filter_rows, int filter_cols, int out_depth)
{
    // The strides are not part of the query (as they are not part of the reference's temporaries'
    // shapes): a strided call runs smaller sub-problems than this stride-1 bound in every extent.
    // A strided call also keeps one vector of in_depth floats per residue class, for up to
    // MAX_TAP_CLASSES classes at a time, ahead of the GEMM's own workspace.
    return poison_bytes(in_depth) + gemm_workspace_bytes((int64_t)batch * input_rows * input_cols, in_depth,
                                                         (int64_t)filter_rows * filter_cols * out_depth, 1, 1);
}

size_t amsim_convam_input_grad_strided_workspace_bytes(int batch, int input_rows, int input_cols, int in_depth,
                                                       int filter_rows, int filter_cols, int out_depth,
                                                       int stride_rows, int stride_cols, int pad_top, int pad_left)
{
    size_t need = amsim_convam_input_grad_workspace_bytes(batch, input_rows, input_cols, in_depth, filter_rows,
                                                          filter_cols, out_depth);
    if (stride_rows < 1 || stride_cols < 1 || batch <= 0 || input_rows <= 0 || input_cols <= 0) return need;
    const GradInputGeometry g{batch, input_rows, input_cols, in_depth, filter_rows, filter_cols, out_depth,
                              0, 0, stride_rows, stride_cols, pad_top, pad_left};
    for (int py = 0; py < stride_rows; ++py)
        for (int px = 0; px < stride_cols; ++px) {
            const GemmDesc d = grad_input_phase(g, py, px, nullptr, nullptr, nullptr);
            need = std::max(need, poison_bytes(in_depth) + gemm_workspace_bytes(d.R, d.J, d.K, 1, 1));
        }
    return need;
}

size_t amsim_convam_input_grad_workspace_bytes_for(amsim_lut_t lut, int batch, int input_rows, int input_cols,
                                                   int in_depth, int filter_rows, int filter_cols, int out_depth,
                                                   int stride_rows, int stride_cols, int pad_top, int pad_left)
{
    size_t need = amsim_convam_input_grad_strided_workspace_bytes(batch, input_rows, input_cols, in_depth, filter_rows,
                                                                  filter_cols, out_depth, stride_rows, stride_cols, pad_top,
                                                                  pad_left);
    if (!need || lut == nullptr || lut->l.m <= 7 || stride_rows < 1 || stride_cols < 1) return need;
    const GradInputGeometry g{batch, input_rows, input_cols, in_depth, filter_rows, filter_cols, out_depth,
                              0, 0, stride_rows, stride_cols, pad_top, pad_left};
    for (int py = 0; py < stride_rows; ++py)
        for (int px = 0; px < stride_cols; ++px) {
            const GemmDesc d = grad_input_phase(g, py, px, nullptr, nullptr, nullptr);
            const size_t wide = gemm_workspace_bytes_wide(d.R, d.J, d.K, 1, 1);
            if (wide) need = std::max(need, poison_bytes(in_depth) + wide);
        }
    return need;
}

int amsim_convam_input_grad_f32(amsim_lut_t lut, const float *grad, int hole_grad_width, int hole_grad_height,
                                int pad_top, int pad_left, const float *filter, int filter_rows, int filter_cols,
                                int out_depth, int stride_rows, int stride_cols, int batch, int input_rows,
                                int input_cols, int in_depth, float *output, int out_rows, int out_cols,
                                void *workspace, size_t workspace_bytes, void *stream)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (batch < 0 || input_rows < 0 || input_cols < 0 || in_depth < 0 || filter_rows < 0 || filter_cols < 0 ||
        out_depth < 0 || out_rows < 0 || out_cols < 0 || stride_cols < 1 || stride_rows < 1)
        return fail(AMSIM_ERR_INVALID, "bad convolution geometry");
    if (out_rows > 0 && out_cols > 0 &&
        (hole_grad_height != (out_rows - 1) * stride_rows + 1 || hole_grad_width != (out_cols - 1) * stride_cols + 1))
        return fail(AMSIM_ERR_INVALID, "hole_grad extent must be (out - 1) * stride + 1");
    const int64_t R = (int64_t)batch * input_rows * input_cols;
    if (R == 0 || in_depth == 0) return AMSIM_OK;
    if (!grad || !output || !filter) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    if (!fits_int32((int64_t)batch * out_rows * out_cols * out_depth))
        return fail(AMSIM_ERR_UNSUPPORTED, "gradient tensor has 2^31 or more elements");
    if (!fits_int32(R * in_depth)) return fail(AMSIM_ERR_UNSUPPORTED, "input tensor has 2^31 or more elements");
    const size_t need = amsim_convam_input_grad_workspace_bytes(batch, input_rows, input_cols, in_depth, filter_rows,
                                                                filter_cols, out_depth);
    if (workspace == nullptr || ((uintptr_t)workspace & 255) || workspace_bytes < need)
        return fail(AMSIM_ERR_WORKSPACE, "workspace missing, not 256-byte aligned or smaller than " +
                                             std::to_string(need) + " bytes");
    const GradInputGeometry g{batch, input_rows, input_cols, in_depth, filter_rows, filter_cols, out_depth,
                              out_rows, out_cols, stride_rows, stride_cols, pad_top, pad_left};
    hipStream_t st = static_cast<hipStream_t>(stream);
    float *poison = static_cast<float *>(workspace);
    void *gemm_ws_ptr = static_cast<uint8_t *>(workspace) + poison_bytes(in_depth);
    const size_t gemm_ws_bytes = workspace_bytes - poison_bytes(in_depth);
    const bool strided = stride_rows > 1 || stride_cols > 1;
    // residue classes with pixels, handled MAX_TAP_CLASSES at a time: one launch marks the channels
    // that a class's skipped taps poison, then the class's sub-problems run
    struct Pending { int py, px; };
    Pending pend[MAX_TAP_CLASSES];
    TapClass cls[MAX_TAP_CLASSES];
    int n = 0;
    auto flush = [&]() -> int {
        if (n == 0) return AMSIM_OK;
        if (strided) {
            const int rc = launch_skipped_tap_poison(filter, filter_rows, filter_cols, in_depth, out_depth, cls, n,
                                                     poison, poison_stride(in_depth), st);
            if (rc != AMSIM_OK) return rc;
        }
        for (int i = 0; i < n; ++i) {
            GemmDesc d = grad_input_phase(g, pend[i].py, pend[i].px, grad, filter, output);
            if (strided) d.bias_j = poison + (size_t)i * poison_stride(in_depth);
            // a phase whose best plan wants more partial-sum space than the caller's (stride-agnostic)
            // workspace holds runs unsplit: its pre-decoded filter always fits
            if (gemm_workspace_bytes(d.R, d.J, d.K, 1, 1) > gemm_ws_bytes) d.no_split = true;
            const int rc = run_gemm(lut->l, d, gemm_ws_ptr, gemm_ws_bytes, st);
            if (rc != AMSIM_OK) return rc;
        }
        n = 0;
        return AMSIM_OK;
    };
    for (int py = 0; py < stride_rows; ++py)
        for (int px = 0; px < stride_cols; ++px) {
            const GemmDesc d = grad_input_phase(g, py, px, grad, filter, output);
            if (d.R == 0) continue;
            pend[n] = Pending{py, px};
            cls[n] = TapClass{d.q.fy0, d.q.fsy, d.q.TH, d.q.fx0, d.q.fsx, d.q.TW};
            if (++n == MAX_TAP_CLASSES) {
                const int rc = flush();
                if (rc != AMSIM_OK) return rc;
            }
        }
    return flush();
}

namespace {
// A 1x1 filter at stride 1 without padding makes the filter gradient the plain product
// input^T [C x K] . grad [K x OC]: either operand may then be the pre-decoded one.
GemmCall pointwise_filter_grad(int64_t pixels, int in_depth, int out_depth, const float *input, const float *grad,
                               float *output)
{
    return GemmCall{1, 0, 0, in_depth, out_depth, pixels, input, in_depth, grad, out_depth, output, out_depth, 1, 0, 0, 0};
}
}  // namespace

namespace {
size_t filter_grad_ws(amsim_lut_t lut, int batch, int out_rows, int out_cols, int out_depth, int filter_rows,
                      int filter_cols, int in_depth)
{
    size_t need = gemm_workspace_bytes((int64_t)filter_rows * filter_cols * in_depth, out_depth,
                                       (int64_t)batch * out_rows * out_cols, 1, 1);
    if (filter_rows == 1 && filter_cols == 1)
        need = std::max(need, gemm_ws(pointwise_filter_grad((int64_t)batch * out_rows * out_cols, in_depth, out_depth,
                                                            nullptr, nullptr, nullptr), lut));
    else if (need && lut != nullptr && lut->l.m > 7)
        need = std::max(need, gemm_workspace_bytes_wide((int64_t)filter_rows * filter_cols * in_depth, out_depth,
                                                        (int64_t)batch * out_rows * out_cols, 1, 1));
    return need;
}
}  // namespace

size_t amsim_convam_filter_grad_workspace_bytes(int batch, int out_rows, int out_cols, int out_depth,
                                                int filter_rows, int filter_cols, int in_depth)
{
    return filter_grad_ws(nullptr, batch, out_rows, out_cols, out_depth, filter_rows, filter_cols, in_depth);
}

size_t amsim_convam_filter_grad_workspace_bytes_for(amsim_lut_t lut, int batch, int out_rows, int out_cols,
                                                    int out_depth, int filter_rows, int filter_cols, int in_depth)
{
    return filter_grad_ws(lut, batch, out_rows, out_cols, out_depth, filter_rows, filter_cols, in_depth);
}

int amsim_convam_filter_grad_f32(amsim_lut_t lut, const float *input, const float *grad, int input_rows,
                                 int input_cols, int batch, int in_depth, int out_cols, int out_rows,
                                 int out_depth, int filter_left_offset, int filter_top_offset, int stride_rows,
                                 int stride_cols, int filter_cols, int filter_rows, float *output, void *workspace,
                                 size_t workspace_bytes, void *stream)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (batch < 0 || input_rows < 0 || input_cols < 0 || in_depth < 0 || filter_rows < 0 || filter_cols < 0 ||
        out_depth < 0 || out_rows < 0 || out_cols < 0 || stride_cols < 1 || stride_rows < 1)
        return fail(AMSIM_ERR_INVALID, "bad convolution geometry");
    const int64_t R = (int64_t)filter_rows * filter_cols * in_depth;
    if (R == 0 || out_depth == 0) return AMSIM_OK;
    if (!output) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    const int64_t K = (int64_t)batch * out_rows * out_cols;
    if (K > 0 && (!input || !grad)) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    if (!fits_int32((int64_t)batch * input_rows * input_cols * in_depth))
        return fail(AMSIM_ERR_UNSUPPORTED, "input tensor has 2^31 or more elements");
    if (filter_rows == 1 && filter_cols == 1 && stride_rows == 1 && stride_cols == 1 && filter_top_offset == 0 &&
        filter_left_offset == 0 && out_rows == input_rows && out_cols == input_cols)
        return gemm_call(lut, pointwise_filter_grad(K, in_depth, out_depth, input, grad, output), workspace,
                         workspace_bytes, stream);  // P(input, grad), reduction over (b, oy, ox) as below
    // rows (fy, fx, c) of the filter x reduction over (b, oy, ox)
    // [cuda_kernel.cu:327-353, 417-425]; the gradient is the [K][OC] matrix
    GemmDesc d;
    d.R = R; d.J = out_depth; d.K = K;
    d.p.kind = P_GF; d.p.base = input;
    d.p.B = batch; d.p.GH = out_rows; d.p.GW = out_cols;
    d.p.KH = filter_rows; d.p.KW = filter_cols; d.p.C = in_depth;
    d.p.sy = stride_rows; d.p.sx = stride_cols; d.p.pt = filter_top_offset; d.p.pl = filter_left_offset;
    d.p.SH = input_rows; d.p.SW = input_cols;
    d.q.kind = Q_DENSE; d.q.base = grad; d.q.sk = out_depth; d.q.sj = 1;
    d.out = output; d.so_r = out_depth; d.so_j = 1;
    d.lane_first = true;  // P(input, grad)
    return run_gemm(lut->l, d, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

// ---- dense ----------------------------------------------------------------------------

size_t amsim_denseam_workspace_bytes_for(amsim_lut_t lut, int batch, int units, int input_width)
{
    // the largest of the three GEMMs of the layer
    GemmCall f{0, 0, 0, batch, units, input_width, nullptr, 0, nullptr, 0, nullptr, 0, 1, 0, 0, 0};
    GemmCall w{1, 0, 0, input_width, units, batch, nullptr, 0, nullptr, 0, nullptr, 0, 1, 0, 0, 0};
    GemmCall x{0, 1, 1, batch, input_width, units, nullptr, 0, nullptr, 0, nullptr, 0, 1, 0, 0, 0};
    return std::max(gemm_ws(f, lut), std::max(gemm_ws(w, lut), gemm_ws(x, lut)));
}

size_t amsim_denseam_workspace_bytes(int batch, int units, int input_width)
{
    return amsim_denseam_workspace_bytes_for(nullptr, batch, units, input_width);
}

int amsim_denseam_f32(amsim_lut_t lut, const float *inputs, const float *weights, float *output, int batch,
                      int units, int input_width, void *workspace, size_t workspace_bytes, void *stream)
{
    // denseam_kernel.cu:38-41: P(input, weight)
    GemmCall g{0, 0, 0, batch, units, input_width, inputs, input_width, weights, units, output, units, 1, 0, 0, 0};
    return gemm_call(lut, g, workspace, workspace_bytes, stream);
}

int amsim_denseam_bias_act_f32(amsim_lut_t lut, const float *inputs, const float *weights, float *output, int batch,
                               int units, int input_width, const float *bias, int activation, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    if (!known_activation(activation)) return fail(AMSIM_ERR_INVALID, "unknown activation");
    GemmCall g{0, 0, 0, batch, units, input_width, inputs, input_width, weights, units, output, units, 1, 0, 0, 0};
    g.bias_n = bias;
    g.act = activation;
    return gemm_call(lut, g, workspace, workspace_bytes, stream);
}

int amsim_denseam_weight_grad_f32(amsim_lut_t lut, const float *input, const float *grads, float *output,
                                  int batch, int units, int input_width, void *workspace, size_t workspace_bytes,
                                  void *stream)
{
    // denseam_kernel.cu:64-67: dW[k][j] = sum_i P(input[i][k], grads[i][j])
    GemmCall g{1, 0, 0, input_width, units, batch, input, input_width, grads, units, output, units, 1, 0, 0, 0};
    return gemm_call(lut, g, workspace, workspace_bytes, stream);
}

int amsim_denseam_input_grad_f32(amsim_lut_t lut, const float *weight, const float *grads, float *output,
                                 int batch, int units, int input_width, void *workspace, size_t workspace_bytes,
                                 void *stream)
{
    // denseam_kernel.cu:91-94: dX[i][k] = sum_j P(weight[k][j], grads[i][j]) -- weight is the first LUT operand
    GemmCall g{0, 1, 1, batch, input_width, units, grads, units, weight, units, output, input_width, 1, 0, 0, 0};
    return gemm_call(lut, g, workspace, workspace_bytes, stream);
}

// ---- matmul ---------------------------------------------------------------------------

static int matmul_call(int batch_a, int batch_b, int row_a, int col_a, int row_b, int col_b, GemmCall *g)
{
    if (batch_a < 0 || batch_b < 0 || row_a < 0 || col_a < 0 || row_b < 0 || col_b < 0)
        return fail(AMSIM_ERR_INVALID, "negative extent");
    if (col_a != row_b) return fail(AMSIM_ERR_INVALID, "Does not meet cols of mat a is equal rows of mat b");
    if (batch_a > 1 && batch_b > 1 && batch_a != batch_b)
        return fail(AMSIM_ERR_INVALID, "Does not meet batch of mat a is equal batch of matb");
    const int nb = std::max(std::max(batch_a, batch_b), 1);
    *g = GemmCall{0, 0, 0, row_a, col_b, col_a, nullptr, col_a, nullptr, col_b, nullptr, col_b, nb,
                  batch_a > 1 ? (int64_t)row_a * col_a : 0, batch_b > 1 ? (int64_t)row_b * col_b : 0,
                  (int64_t)row_a * col_b};
    return AMSIM_OK;
}

size_t amsim_matmulam_workspace_bytes_for(amsim_lut_t lut, int batch_a, int batch_b, int row_a, int col_a, int row_b,
                                          int col_b)
{
    GemmCall g;
    if (matmul_call(batch_a, batch_b, row_a, col_a, row_b, col_b, &g) != AMSIM_OK) return 0;
    return gemm_ws(g, lut);
}

size_t amsim_matmulam_workspace_bytes(int batch_a, int batch_b, int row_a, int col_a, int row_b, int col_b)
{
    return amsim_matmulam_workspace_bytes_for(nullptr, batch_a, batch_b, row_a, col_a, row_b, col_b);
}

int amsim_matmulam_f32(amsim_lut_t lut, const float *a, const float *b, int batch_a, int batch_b, int row_a,
                       int col_a, int row_b, int col_b, float *out, void *workspace, size_t workspace_bytes,
                       void *stream)
{
    GemmCall g;
    int rc = matmul_call(batch_a, batch_b, row_a, col_a, row_b, col_b, &g);
    if (rc != AMSIM_OK) return rc;
    g.A = a; g.B = b; g.C = out;
    return gemm_call(lut, g, workspace, workspace_bytes, stream);
}

// ---- dot-product attention --------------------------------------------------------------
// multihead_attention.py:18-30 on contiguous [batch][seq][depth] operands: two strided-batch
// products around the row softmax.  Gradient wiring follows math_ops.py:141-157: the op never
// sees the transpose flags, so every gradient is (grad, b_op^T) and (a_op^T, grad).

namespace {

struct AttnShape {
    int batch, seq_q, seq_k, d_k, d_v;
    int64_t nq() const { return (int64_t)seq_q * d_k; }
    int64_t nk() const { return (int64_t)seq_k * d_k; }
    int64_t nv() const { return (int64_t)seq_k * d_v; }
    int64_t nw() const { return (int64_t)seq_q * seq_k; }
    int64_t no() const { return (int64_t)seq_q * d_v; }
    // scores = q . k^T          P(q, k)
    GemmCall scores(const float *q, const float *k, float *w) const
    { return GemmCall{0, 1, 0, seq_q, seq_k, d_k, q, d_k, k, d_k, w, seq_k, batch, nq(), nk(), nw()}; }
    // out = weights . v         P(weights, v)
    GemmCall context(const float *w, const float *v, float *o) const
    { return GemmCall{0, 0, 0, seq_q, d_v, seq_k, w, seq_k, v, d_v, o, d_v, batch, nw(), nv(), no()}; }
    // d(weights) = d(out) . v^T P(d(out), v)
    GemmCall grad_weights(const float *go, const float *v, float *gw) const
    { return GemmCall{0, 1, 0, seq_q, seq_k, d_v, go, d_v, v, d_v, gw, seq_k, batch, no(), nv(), nw()}; }
    // d(v) = weights^T . d(out) P(weights, d(out))
    GemmCall grad_v(const float *w, const float *go, float *gv) const
    { return GemmCall{1, 0, 0, seq_k, d_v, seq_q, w, seq_k, go, d_v, gv, d_v, batch, nw(), no(), nv()}; }
    // d(q) = d(scores) . k      P(d(scores), k)
    GemmCall grad_q(const float *gs, const float *k, float *gq) const
    { return GemmCall{0, 0, 0, seq_q, d_k, seq_k, gs, seq_k, k, d_k, gq, d_k, batch, nw(), nk(), nq()}; }
    // d(k) = (q^T . d(scores))^T = d(scores)^T . q with the LUT fed as P(q, d(scores))
    GemmCall grad_k(const float *gs, const float *q, float *gk) const
    { return GemmCall{1, 0, 1, seq_k, d_k, seq_q, gs, seq_k, q, d_k, gk, d_k, batch, nw(), nq(), nk()}; }
};

bool attn_shape_ok(const AttnShape &s) { return s.batch >= 0 && s.seq_q >= 0 && s.seq_k >= 0 && s.d_k >= 0 && s.d_v >= 0; }
size_t align256(size_t b) { return (b + 255) / 256 * 256; }

}  // namespace

size_t amsim_attention_workspace_bytes_for(amsim_lut_t lut, int batch, int seq_q, int seq_k, int d_k, int d_v)
{
    const AttnShape s{batch, seq_q, seq_k, d_k, d_v};
    if (!attn_shape_ok(s)) return 0;
    return std::max(gemm_ws(s.scores(nullptr, nullptr, nullptr), lut), gemm_ws(s.context(nullptr, nullptr, nullptr), lut));
}

size_t amsim_attention_workspace_bytes(int batch, int seq_q, int seq_k, int d_k, int d_v)
{
    return amsim_attention_workspace_bytes_for(nullptr, batch, seq_q, seq_k, d_k, d_v);
}

int amsim_attention_f32(amsim_lut_t lut, const float *q, const float *k, const float *v, const float *mask,
                        int mask_batch_div, int64_t mask_batch_stride, int64_t mask_row_stride, int batch, int seq_q,
                        int seq_k, int d_k, int d_v, float divisor, float *weights, float *out, void *workspace,
                        size_t workspace_bytes, void *stream)
{
    const AttnShape s{batch, seq_q, seq_k, d_k, d_v};
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (!attn_shape_ok(s)) return fail(AMSIM_ERR_INVALID, "negative extent");
    if (!(divisor > 0.0f)) return fail(AMSIM_ERR_INVALID, "the score divisor must be positive");
    if (mask && (mask_batch_div < 1 || mask_batch_stride < 0 || mask_row_stride < 0))
        return fail(AMSIM_ERR_INVALID, "bad mask layout");
    if (batch == 0 || seq_q == 0) return AMSIM_OK;
    if (seq_k > 0 && !weights) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    int rc = gemm_call(lut, s.scores(q, k, weights), workspace, workspace_bytes, stream);
    if (rc != AMSIM_OK) return rc;
    rc = launch_softmax_rows(weights, mask, mask_batch_div, mask_batch_stride, mask_row_stride, batch, seq_q, seq_k,
                             divisor, static_cast<hipStream_t>(stream));
    if (rc != AMSIM_OK) return rc;
    return gemm_call(lut, s.context(weights, v, out), workspace, workspace_bytes, stream);
}

size_t amsim_attention_grad_workspace_bytes_for(amsim_lut_t lut, int batch, int seq_q, int seq_k, int d_k, int d_v)
{
    const AttnShape s{batch, seq_q, seq_k, d_k, d_v};
    if (!attn_shape_ok(s)) return 0;
    size_t g = gemm_ws(s.grad_weights(nullptr, nullptr, nullptr), lut);
    g = std::max(g, gemm_ws(s.grad_v(nullptr, nullptr, nullptr), lut));
    g = std::max(g, gemm_ws(s.grad_q(nullptr, nullptr, nullptr), lut));
    g = std::max(g, gemm_ws(s.grad_k(nullptr, nullptr, nullptr), lut));
    return align256((size_t)batch * (size_t)s.nw() * sizeof(float)) + g;
}

size_t amsim_attention_grad_workspace_bytes(int batch, int seq_q, int seq_k, int d_k, int d_v)
{
    return amsim_attention_grad_workspace_bytes_for(nullptr, batch, seq_q, seq_k, d_k, d_v);
}

int amsim_attention_grad_f32(amsim_lut_t lut, const float *q, const float *k, const float *v, const float *weights,
                             const float *grad_out, int batch, int seq_q, int seq_k, int d_k, int d_v, float divisor,
                             float *grad_q, float *grad_k, float *grad_v, void *workspace, size_t workspace_bytes,
                             void *stream)
{
    const AttnShape s{batch, seq_q, seq_k, d_k, d_v};
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (!attn_shape_ok(s)) return fail(AMSIM_ERR_INVALID, "negative extent");
    if (!(divisor > 0.0f)) return fail(AMSIM_ERR_INVALID, "the score divisor must be positive");
    if (batch == 0) return AMSIM_OK;
    const size_t need = amsim_attention_grad_workspace_bytes_for(lut, batch, seq_q, seq_k, d_k, d_v);
    if (need && (workspace == nullptr || ((uintptr_t)workspace & 255) || workspace_bytes < need))
        return fail(AMSIM_ERR_WORKSPACE, "workspace missing, not 256-byte aligned or smaller than " +
                                             std::to_string(need) + " bytes");
    // d(weights), then d(scores) in place, lives at the head of the workspace
    const size_t gw_bytes = align256((size_t)batch * (size_t)s.nw() * sizeof(float));
    float *gw = static_cast<float *>(workspace);
    void *ws = static_cast<uint8_t *>(workspace) + gw_bytes;
    const size_t ws_bytes = workspace_bytes - gw_bytes;
    if ((int64_t)seq_q * seq_k > 0 && !weights) return fail(AMSIM_ERR_INVALID, "null tensor pointer");
    int rc = gemm_call(lut, s.grad_v(weights, grad_out, grad_v), ws, ws_bytes, stream);
    if (rc != AMSIM_OK) return rc;
    rc = gemm_call(lut, s.grad_weights(grad_out, v, gw), ws, ws_bytes, stream);
    if (rc != AMSIM_OK) return rc;
    rc = launch_softmax_grad_rows(weights, gw, (int64_t)batch * seq_q, seq_k, divisor, static_cast<hipStream_t>(stream));
    if (rc != AMSIM_OK) return rc;
    rc = gemm_call(lut, s.grad_q(gw, k, grad_q), ws, ws_bytes, stream);
    if (rc != AMSIM_OK) return rc;
    return gemm_call(lut, s.grad_k(gw, q, grad_k), ws, ws_bytes, stream);
}

// ---- geometry -------------------------------------------------------------------------

int amsim_conv_geometry(int in_size, int filter_size, int stride, int padding, int *out_size, int *pad_before)
{
    if (in_size < 0 || filter_size < 1 || stride < 1 || !out_size || !pad_before)
        return fail(AMSIM_ERR_INVALID, "bad window geometry");
    if (padding == AMSIM_PADDING_VALID) {
        *out_size = in_size - filter_size + stride >= 0 ? (in_size - filter_size + stride) / stride : 0;
        *pad_before = 0;
    } else if (padding == AMSIM_PADDING_SAME) {
        *out_size = (in_size + stride - 1) / stride;
        const int total = std::max((*out_size - 1) * stride + filter_size - in_size, 0);
        *pad_before = total / 2;
    } else {
        return fail(AMSIM_ERR_INVALID, "padding must be AMSIM_PADDING_VALID or AMSIM_PADDING_SAME");
    }
    return AMSIM_OK;
}

}  // extern "C"
