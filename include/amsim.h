/*
 * amsim.h -- C ABI of the MI355X (gfx950) approximate-multiplier simulator.
 *
 * This is the drop-in seam underneath ApproxTrain's custom-op surface: each
 * entry point replaces one of the reference's device functors / kernels, takes
 * plain device pointers, sizes and a HIP stream, and returns a status code
 * (the reference prints and calls exit(); cuda/error.cuh:19-27).
 *
 * Conventions
 *   - all tensors are FP32 in device memory; NHWC activations, HWIO filters,
 *     row-major matrices (as in the reference);
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream); calls
 *     are stream-ordered and never synchronise the device (the reference calls
 *     cudaDeviceSynchronize after every launch);
 *   - the library allocates device memory only in amsim_lut_create /
 *     amsim_lut_load_file; per-call scratch comes from the caller as
 *     `workspace` (size from the matching *_workspace_bytes query, 256-byte
 *     aligned), the way the reference's OpKernels allocate their im2col /
 *     rsfilter temporaries and hand them to the functor;
 *   - the approximate product follows the C functional models
 *     (lut/FPmultMBM_fast16.inl:45-134, lut/Mitchell_16.inl:44-129) bit for
 *     bit on the whole FP32 domain, given the matching LUT;
 *   - every output element is one FP32 accumulation chain in ascending
 *     reduction index when the reduction is not split; the filter gradient and
 *     small problems split the reduction deterministically (fixed chunking,
 *     fixed summation order), so results are reproducible run to run.
 */
#ifndef AMSIM_H_
#define AMSIM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AMSIM_OK 0
#define AMSIM_ERR_INVALID 1     /* bad argument / shape mismatch (OP_REQUIRES InvalidArgument in the reference) */
#define AMSIM_ERR_IO 2          /* LUT file missing or unreadable (exit(1) in approx_mul_lut.h:31-40) */
#define AMSIM_ERR_LUT_FORMAT 3  /* file name without _<m>.bin suffix, unsupported width, short file */
#define AMSIM_ERR_HIP 4         /* a HIP runtime call failed */
#define AMSIM_ERR_WORKSPACE 5   /* workspace missing, misaligned or too small */
#define AMSIM_ERR_UNSUPPORTED 6

/* padding attr values, numerically equal to tensorflow::Padding (convam.cc:552 tests `padding == 1`) */
#define AMSIM_PADDING_VALID 1
#define AMSIM_PADDING_SAME 2

/* output epilogue of the *_bias_act entry points */
#define AMSIM_ACT_NONE 0
#define AMSIM_ACT_RELU 1

typedef struct amsim_lut *amsim_lut_t;

const char *amsim_status_string(int status);
/* message of the last failing call on this thread ("" if none) */
const char *amsim_last_error(void);
/* "gfx950" etc. of the current device, and the number of compute units */
int amsim_device_info(char *arch, size_t arch_len, int *compute_units);

/* ---- LUT handle: replaces approx_mul_lut<GPUDevice>
 *      (approx_mul_lut.h:7-80, cuda/approx_mul_lut.cu:24-53) -------------------
 * amsim_lut_load_file parses the mantissa width from the file name between the
 * last '_' and the last '.' (approx_mul_lut.h:22-25) and reads 2^(2m) entries:
 * 1 byte each (carry<<7 | mantissa, lut/lut_gen.cc:114-121) for m <= 7, 4 bytes
 * each (the legacy layout below) for 8 <= m <= 11, which the reference has no
 * file format for.
 * amsim_lut_create takes the entries from host memory; entry_bytes is 1
 * (layout above, m <= 7) or 4 (legacy layout of lut/AMsimulator.inl:18-20:
 * bit 31 = carry, bits 22..0 = mantissa in place; m <= 11).
 * Both upload the table images to the current device and wait for the copies; the first handle
 * created on a device also runs a one-wavefront probe kernel there (how 16-bit LDS loads treat
 * the other register half, which the GEMM kernels adapt to).  Create handles outside stream
 * capture. */
int amsim_lut_load_file(const char *path, amsim_lut_t *out);
int amsim_lut_create(const void *entries, size_t n_bytes, int mant_width, int entry_bytes, amsim_lut_t *out);
int amsim_lut_destroy(amsim_lut_t lut);
int amsim_lut_mant_width(amsim_lut_t lut);
/* the derived fields of approx_mul_lut.h:26-28 */
int amsim_lut_params(amsim_lut_t lut, uint32_t *mant_mask, int *a_shift, int *b_shift);
/* How calls through this handle may run their reductions (no counterpart in the reference):
 * 0 = every output is one sequential FP32 chain in ascending reduction index, bit-identical to
 * a sequential CPU loop; 1 = problems with few outputs, and the tail rows of large ones, may
 * split the reduction across workgroups (partial sums added in a fixed order: reproducible run
 * to run, within 1e-5 * sum|products| of the sequential chain); -1 (initial value) = follow the
 * process default of amsim_set_split_k.  The mode is read once per call; a workspace sized by
 * the *_workspace_bytes queries is large enough for either mode.  Use one handle per thread
 * (handles are cheap) when threads need different modes. */
int amsim_lut_set_split_k(amsim_lut_t lut, int mode);

/* ---- LUT generation (host side): replaces lut/lut_gen.cc:86-127 + lut/lut_gen.sh
 * A table holds, for every pair (i, j) of m-bit mantissas, the product of 1.i and
 * 1.j at biased exponent 127: its top m mantissa bits and whether its exponent
 * went up ("carry").  entry_bytes 1 (m <= 7): carry << 7 | mantissa, the file
 * format of lut_gen.cc:114-121; entry_bytes 4 (m <= 11): carry << 31 | mantissa
 * in place (lut/AMsimulator.inl:18-20).  `entries` is host memory of
 * 2^(2m) * entry_bytes bytes; pass it to amsim_lut_create or write it to
 * "<NAME>_<m>.bin" for amsim_lut_load_file (1-byte entries for m <= 7, 4-byte
 * entries above).
 * amsim_lut_generate evaluates a caller-supplied multiplier, the plug-in route
 * of developer.md:38-86 (a C function taking and returning float);
 * amsim_lut_generate_builtin knows "MBM" (lut/FPmultMBM_fast*.inl), "MIT"
 * (lut/Mitchell_*.inl), "ACC" (lut/bfloat.inl at any width) and "ZEROS". */
typedef float (*amsim_multiplier_fn)(float a, float b, void *user);
int amsim_lut_generate(amsim_multiplier_fn fn, void *user, int mant_width, int entry_bytes, void *entries,
                       size_t n_bytes);
int amsim_lut_generate_builtin(const char *name, int mant_width, int entry_bytes, void *entries, size_t n_bytes);

/* ---- elementwise product (test hook): the device function AMsimulator
 *      (cuda/AMsimulator.inl:13-36) with the functional models' semantics ---- */
int amsim_mul_f32(amsim_lut_t lut, const float *a, const float *b, float *out, size_t n, void *stream);

/* ---- GEMM: replaces gemm<float> (cuda/gemm.cu:17-58) ------------------------
 * C[i][j] = sum_k P(opA(i,k), opB(k,j)); opA is M x K (A[i*lda+k], or
 * A[k*lda+i] if transA), opB is K x N.  swap_operands feeds the LUT as
 * P(B element, A element) (denseam_kernel.cu:93).  batch > 1 runs a strided
 * batch (stride 0 broadcasts an operand), replacing the per-item launch loop
 * of cuda/matmulam_kernel.cu:30-98. */
size_t amsim_gemm_workspace_bytes(int transA, int transB, int64_t M, int64_t N, int64_t K, int64_t batch);
/* The query above is an upper bound over every table: it includes the transposed operand copy
 * that only tables of 8..11 mantissa bits read (the row-staged engine), several times what a
 * table that fits the LDS needs.  The query for a given table returns what calls through that
 * handle use; amsim_denseam_ / amsim_matmulam_ / amsim_attention_ / amsim_attention_grad_
 * workspace_bytes_for below are the same for their entry points.  A NULL handle gives the upper
 * bound. */
size_t amsim_gemm_workspace_bytes_for(amsim_lut_t lut, int transA, int transB, int64_t M, int64_t N, int64_t K,
                                      int64_t batch);
int amsim_gemm_f32(amsim_lut_t lut, int transA, int transB, int swap_operands, int64_t M, int64_t N,
                   int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                   int64_t ldc, int64_t batch, int64_t strideA, int64_t strideB, int64_t strideC,
                   void *workspace, size_t workspace_bytes, void *stream);

/* ---- convolution functors ----------------------------------------------------
 * Argument names and order follow convam.h:71-104; the im2col / rsfilter
 * temporaries of the reference are replaced by `workspace`. */

/* ConvamFunctor<GPUDevice,float>::operator() (convam.h:71-79, cuda_kernel.cu:181-321) */
size_t amsim_convam_workspace_bytes(int batch, int out_rows, int out_cols, int out_depth, int filter_rows,
                                    int filter_cols, int in_depth);
int amsim_convam_f32(amsim_lut_t lut, const float *input_data, float *output_data, int batch, int out_rows,
                     int out_cols, int out_depth, int stride_cols, int stride_rows, int filter_left_offset,
                     int filter_top_offset, int filter_rows, int filter_cols, int in_depth, int input_cols,
                     int input_rows, const float *filter, void *workspace, size_t workspace_bytes,
                     void *stream);
/* The query for a given table.  For tables of up to 7 mantissa bits it equals the one above.  For
 * wider tables (8..11 bits) it adds what the row-staged engine needs -- an im2col of the input, the
 * temporary the reference also allocates (convam.cc:518-546) -- so that the call runs on that engine
 * at its best (the im2col is streamed once).  A call given less still runs: with at least the "lean"
 * amount below, on the same engine from a zero-bordered channel-major copy of the input (the size
 * of the input instead of filter_rows x filter_cols times it; about 25 % slower, every channel plane
 * being re-read once per filter tap); with only the table-agnostic amount, by one global gather per
 * product (about 10x slower). */
size_t amsim_convam_workspace_bytes_for(amsim_lut_t lut, int batch, int out_rows, int out_cols, int out_depth,
                                        int filter_rows, int filter_cols, int in_depth);
size_t amsim_convam_lean_workspace_bytes_for(amsim_lut_t lut, int batch, int out_rows, int out_cols, int out_depth,
                                             int filter_rows, int filter_cols, int in_depth, int stride_rows,
                                             int stride_cols);

/* amsim_convam_f32 for callers that cannot allocate device memory or bring a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The call takes its scratch (pre-decoded filter, partial sums of
 * split reductions) from a buffer of AMSIM_NOALLOC_SCRATCH_BYTES that is part of the library's
 * device image -- every GPU the library runs on holds it from the first call until the process
 * ends -- and calls no hipMalloc, hipFree or other allocating routine.  Problems whose
 * amsim_convam_workspace_bytes exceeds that size are refused with AMSIM_ERR_UNSUPPORTED.
 * Results are bit-identical to amsim_convam_f32 on the same inputs when that call is given a
 * workspace of AMSIM_NOALLOC_SCRATCH_BYTES (for tables of up to 7 mantissa bits: any workspace its
 * query returns; wider tables pick their engine by the workspace they are given, and engines
 * differ in how they round split reductions).  The first call on a device also looks the buffer's
 * address up (hipGetSymbolAddress): make one call outside a graph capture first.  All calls on one
 * GPU share the one buffer: calls that may overlap there (different streams or threads) race; issue them
 * on one stream, or order them with events.  Nothing in the buffer needs to start at zero (each
 * call writes what it later reads). */
#define AMSIM_NOALLOC_SCRATCH_BYTES ((size_t)32 << 20)
int amsim_convam_noalloc_f32(amsim_lut_t lut, const float *input_data, float *output_data, int batch, int out_rows,
                             int out_cols, int out_depth, int stride_cols, int stride_rows, int filter_left_offset,
                             int filter_top_offset, int filter_rows, int filter_cols, int in_depth, int input_cols,
                             int input_rows, const float *filter, void *stream);

/* The same with the layer's epilogue fused into the store: output = act(conv + bias[out_depth]).
 * Replaces Convam followed by BiasAdd and the activation op in AMConv2D.call
 * (python/keras/layers/am_convolutional.py:248-276); bias may be NULL.  Bit-identical to the
 * unfused sequence (the same FP32 add, then max with zero that keeps NaN). */
int amsim_convam_bias_act_f32(amsim_lut_t lut, const float *input_data, float *output_data, int batch, int out_rows,
                              int out_cols, int out_depth, int stride_cols, int stride_rows,
                              int filter_left_offset, int filter_top_offset, int filter_rows, int filter_cols,
                              int in_depth, int input_cols, int input_rows, const float *filter, const float *bias,
                              int activation, void *workspace, size_t workspace_bytes, void *stream);

/* ConvamInputGradFunctor<GPUDevice,float>::operator() (convam.h:84-92,
 * cuda_kernel.cu:590-657).  pad_top/pad_left are the BACK pads
 * filter - 1 - forward_pad (convam.cc:1083-1084); hole_grad_* is the
 * stride-dilated gradient extent (convam.cc:1066-1067). */
size_t amsim_convam_input_grad_workspace_bytes(int batch, int input_rows, int input_cols, int in_depth,
                                               int filter_rows, int filter_cols, int out_depth);
/* With strides above 1 the call runs one undilated sub-problem per residue class of the input
 * pixels modulo the stride (the gradient's inserted zeros are never multiplied).  The query
 * above does not know the strides; a workspace of the size below lets every sub-problem use its
 * best split of the reduction (with less, sub-problems that would need more run unsplit). */
size_t amsim_convam_input_grad_strided_workspace_bytes(int batch, int input_rows, int input_cols, int in_depth,
                                                       int filter_rows, int filter_cols, int out_depth,
                                                       int stride_rows, int stride_cols, int pad_top, int pad_left);
/* The strided query for a given table: as amsim_convam_workspace_bytes_for, for the input gradient. */
size_t amsim_convam_input_grad_workspace_bytes_for(amsim_lut_t lut, int batch, int input_rows, int input_cols,
                                                   int in_depth, int filter_rows, int filter_cols, int out_depth,
                                                   int stride_rows, int stride_cols, int pad_top, int pad_left);
int amsim_convam_input_grad_f32(amsim_lut_t lut, const float *grad, int hole_grad_width, int hole_grad_height,
                                int pad_top, int pad_left, const float *filter, int filter_rows,
                                int filter_cols, int out_depth, int stride_rows, int stride_cols, int batch,
                                int input_rows, int input_cols, int in_depth, float *output, int out_rows,
                                int out_cols, void *workspace, size_t workspace_bytes, void *stream);

/* ConvamFilterGradFunctor<GPUDevice,float>::operator() (convam.h:97-104,
 * cuda_kernel.cu:431-461) */
size_t amsim_convam_filter_grad_workspace_bytes(int batch, int out_rows, int out_cols, int out_depth,
                                                int filter_rows, int filter_cols, int in_depth);
/* The query for a given table: as amsim_convam_workspace_bytes_for, for the filter gradient (the
 * transposed gather of the input that the row-staged engine reads, padded to 1024 rows, + the
 * partial sums of its sliced reduction: about 4x faster than one global gather per product). */
size_t amsim_convam_filter_grad_workspace_bytes_for(amsim_lut_t lut, int batch, int out_rows, int out_cols,
                                                    int out_depth, int filter_rows, int filter_cols, int in_depth);
int amsim_convam_filter_grad_f32(amsim_lut_t lut, const float *input, const float *grad, int input_rows,
                                 int input_cols, int batch, int in_depth, int out_cols, int out_rows,
                                 int out_depth, int filter_left_offset, int filter_top_offset, int stride_rows,
                                 int stride_cols, int filter_cols, int filter_rows, float *output,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* ---- dense functors (denseam.h:9-27, cuda/denseam_kernel.cu:98-145) ---------- */
size_t amsim_denseam_workspace_bytes(int batch, int units, int input_width);
size_t amsim_denseam_workspace_bytes_for(amsim_lut_t lut, int batch, int units, int input_width);
/* DenseamFunctor: output[batch][units] = inputs[batch][input_width] . weights[input_width][units] */
int amsim_denseam_f32(amsim_lut_t lut, const float *inputs, const float *weights, float *output, int batch,
                      int units, int input_width, void *workspace, size_t workspace_bytes, void *stream);
/* DenseamFunctor with the layer's epilogue fused: output = act(inputs . weights + bias[units])
 * (amdenselayer.py:211-226: matmul, bias_add, activation); bias may be NULL. */
int amsim_denseam_bias_act_f32(amsim_lut_t lut, const float *inputs, const float *weights, float *output, int batch,
                               int units, int input_width, const float *bias, int activation, void *workspace,
                               size_t workspace_bytes, void *stream);
/* DenseamWeightGradFunctor: grad_weights[k][j] = sum_i P(input[i][k], grads[i][j]) */
int amsim_denseam_weight_grad_f32(amsim_lut_t lut, const float *input, const float *grads, float *output,
                                  int batch, int units, int input_width, void *workspace,
                                  size_t workspace_bytes, void *stream);
/* DenseamInputGradFunctor: grad_inputs[i][k] = sum_j P(weight[k][j], grads[i][j]) */
int amsim_denseam_input_grad_f32(amsim_lut_t lut, const float *weight, const float *grads, float *output,
                                 int batch, int units, int input_width, void *workspace,
                                 size_t workspace_bytes, void *stream);

/* ---- LaunchMatMul<GPUDevice,float> (matmulam.h:12-17, matmulam_kernel.cu:12-99)
 * batch_a / batch_b: 0 for a rank-2 operand, else its leading dimension; a
 * batch of 1 broadcasts (matmulam.cc:86-147). */
size_t amsim_matmulam_workspace_bytes(int batch_a, int batch_b, int row_a, int col_a, int row_b, int col_b);
size_t amsim_matmulam_workspace_bytes_for(amsim_lut_t lut, int batch_a, int batch_b, int row_a, int col_a, int row_b,
                                          int col_b);
int amsim_matmulam_f32(amsim_lut_t lut, const float *a, const float *b, int batch_a, int batch_b, int row_a,
                       int col_a, int row_b, int col_b, float *out, void *workspace, size_t workspace_bytes,
                       void *stream);

/* ---- DotProductAttention.call (ammha/multihead_attention.py:9-30) -------------
 * for `batch` independent (batch x head) items on contiguous operands
 * q[batch][seq_q][d_k], k[batch][seq_k][d_k], v[batch][seq_k][d_v]:
 *   scores  = matmulam(q, k^T) / divisor  [+ -1e9 * mask]     (:18-24)
 *   weights = softmax(scores) over the key axis                (:27)
 *   out     = matmulam(weights, v)                             (:30)
 * Both products go through the LUT (one strided-batch launch each instead of
 * the per-item loop of cuda/matmulam_kernel.cu:30-98); the division, mask and
 * softmax are plain FP32 like the TensorFlow ops the reference uses there.
 * weights[batch][seq_q][seq_k] is an output (the gradient needs it),
 * out[batch][seq_q][d_v].  mask may be NULL; otherwise its element for item b,
 * query r, key j is mask[(b / mask_batch_div) * mask_batch_stride +
 * r * mask_row_stride + j], which covers a mask shared by the heads of one
 * sample (mask_batch_div = heads) and masks broadcast over queries (row stride 0). */
size_t amsim_attention_workspace_bytes(int batch, int seq_q, int seq_k, int d_k, int d_v);
size_t amsim_attention_workspace_bytes_for(amsim_lut_t lut, int batch, int seq_q, int seq_k, int d_k, int d_v);
int amsim_attention_f32(amsim_lut_t lut, const float *q, const float *k, const float *v, const float *mask,
                        int mask_batch_div, int64_t mask_batch_stride, int64_t mask_row_stride, int batch, int seq_q,
                        int seq_k, int d_k, int d_v, float divisor, float *weights, float *out, void *workspace,
                        size_t workspace_bytes, void *stream);
/* Gradient of the above with MatMulAM's gradient rule (python/ops/math_ops.py:141-157: the op
 * never sees the transpose flags, so each product's gradients are matmulam(grad, b_op^T) and
 * matmulam(a_op^T, grad)):  d(v) = weights^T . d(out),  d(weights) = d(out) . v^T,
 * d(scores) = softmax gradient / divisor,  d(q) = d(scores) . k,  d(k) = (q^T . d(scores))^T.
 * The workspace also holds d(scores) (batch * seq_q * seq_k floats). */
size_t amsim_attention_grad_workspace_bytes(int batch, int seq_q, int seq_k, int d_k, int d_v);
size_t amsim_attention_grad_workspace_bytes_for(amsim_lut_t lut, int batch, int seq_q, int seq_k, int d_k, int d_v);
int amsim_attention_grad_f32(amsim_lut_t lut, const float *q, const float *k, const float *v, const float *weights,
                             const float *grad_out, int batch, int seq_q, int seq_k, int d_k, int d_v, float divisor,
                             float *grad_q, float *grad_k, float *grad_v, void *workspace, size_t workspace_bytes,
                             void *stream);

/* ---- op-level host logic (what the OpKernel::Compute bodies derive) ----------
 * TensorFlow 2.3 GetWindowedOutputSizeVerbose for dilation 1 as used at
 * convam.cc:382-387, 553-572, 1071-1084: output extent and leading pad. */
int amsim_conv_geometry(int in_size, int filter_size, int stride, int padding, int *out_size, int *pad_before);

/* ---- knobs (no counterpart in the reference) -------------------------------------
 * amsim_set_split_k sets the process default that handles in mode -1 follow (see
 * amsim_lut_set_split_k for the two modes and their tolerance); the initial default is 1. */
int amsim_set_split_k(int mode);
/* Which GEMM engine serves tables that fit the LDS (process-wide default; for tests and tuning):
 * AUTO picks per problem -- the direct engine (one launch, operands read where they lie, built
 * for latency) for small problems, the LDS-table engine (operand pre-pass, LDS-staged tiles, built
 * for throughput) for the rest; LDS_TABLE never uses the direct engine; DIRECT uses it for
 * everything it can index.  Results agree bit for bit between the engines when reductions stay
 * whole, and within the split tolerance otherwise. */
#define AMSIM_ENGINE_AUTO 0
#define AMSIM_ENGINE_LDS_TABLE 1
#define AMSIM_ENGINE_DIRECT 2
int amsim_set_engine(int mode);
/* The same choice for calls through one handle (-1, the initial value, follows the process-wide
 * setting): lets threads hold different settings without sharing mutable state. */
int amsim_lut_set_engine(amsim_lut_t lut, int mode);

#ifdef __cplusplus
}
#endif
#endif /* AMSIM_H_ */
