// Row kernels between the two matrix products of dot-product attention
// (ammha/multihead_attention.py:18-28): scores / sqrt(d_k) [+ -1e9 * mask],
// softmax over the key axis, and the gradient of that chain.  Plain FP32 -- the
// reference computes these steps with exact TensorFlow ops; only the matrix
// products go through the approximate multiplier.
//
// One wavefront owns one row (query position): the row is read once into
// registers, reduced with cross-lane shuffles, and written once.  Rows of up
// to 1024 keys whose length is a multiple of four (and 16-byte aligned) move
// as float4, 1 / 2 / 4 per lane; other rows of up to 1024 keys keep 16 scalars
// per lane; longer rows are re-read from memory, which stays in L2.
// HBM-bound: 8 bytes per score forward, 12 backward.
#include "amsim_internal.h"

namespace amsim {

namespace {

constexpr int WG = 256;
constexpr int ROWS_PER_WG = WG / 64;
constexpr int CACHE = 16;  // values a lane keeps in registers

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

struct SoftmaxArgs {
    float *scores;          // [rows][cols], in place: scores -> weights
    const float *mask;      // optional, col stride 1
    int64_t rows;           // batch * seq_q
    int seq_q, cols;
    float divisor;
    int mask_batch_div;
    int64_t mask_batch_stride, mask_row_stride;
};

__device__ __forceinline__ float scaled(const SoftmaxArgs &a, const float *mrow, float s, int j)
{
    float x = s / a.divisor;
    if (mrow) x += -1e9f * mrow[j];
    return x;
}

__global__ __launch_bounds__(WG) void softmax_rows_kernel(SoftmaxArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= a.rows) return;
    float *s = a.scores + row * a.cols;
    const float *mrow = nullptr;
    if (a.mask) {
        const int64_t b = row / a.seq_q, r = row % a.seq_q;
        mrow = a.mask + (b / a.mask_batch_div) * a.mask_batch_stride + r * a.mask_row_stride;
    }
    const bool cached = a.cols <= 64 * CACHE;
    float v[CACHE];
    float mx = -INFINITY;
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int j = lane + 64 * i;
            v[i] = j < a.cols ? scaled(a, mrow, s[j], j) : -INFINITY;
            mx = fmaxf(mx, v[i]);
        }
    } else {
        for (int j = lane; j < a.cols; j += 64) mx = fmaxf(mx, scaled(a, mrow, s[j], j));
    }
    mx = wave_max(mx);
    float sum = 0.0f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            v[i] = lane + 64 * i < a.cols ? expf(v[i] - mx) : 0.0f;
            sum += v[i];
        }
    } else {
        for (int j = lane; j < a.cols; j += 64) sum += expf(scaled(a, mrow, s[j], j) - mx);
    }
    sum = wave_sum(sum);
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int j = lane + 64 * i;
            if (j < a.cols) s[j] = v[i] / sum;
        }
    } else {
        for (int j = lane; j < a.cols; j += 64) s[j] = expf(scaled(a, mrow, s[j], j) - mx) / sum;
    }
}

struct SoftmaxGradArgs {
    const float *weights;   // [rows][cols] softmax output
    float *grad;            // [rows][cols], in place: d(weights) -> d(scores)
    int64_t rows;
    int cols;
    float divisor;
};

// d(scores) = (g - sum_j g_j w_j) * w / divisor
__global__ __launch_bounds__(WG) void softmax_grad_rows_kernel(SoftmaxGradArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= a.rows) return;
    const float *w = a.weights + row * a.cols;
    float *g = a.grad + row * a.cols;
    const bool cached = a.cols <= 64 * CACHE;
    float gv[CACHE], wv[CACHE];
    float dot = 0.0f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int j = lane + 64 * i;
            gv[i] = j < a.cols ? g[j] : 0.0f;
            wv[i] = j < a.cols ? w[j] : 0.0f;
            dot += gv[i] * wv[i];
        }
    } else {
        for (int j = lane; j < a.cols; j += 64) dot += g[j] * w[j];
    }
    dot = wave_sum(dot);
    if (cached) {
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
            const int j = lane + 64 * i;
            if (j < a.cols) g[j] = (gv[i] - dot) * wv[i] / a.divisor;
        }
    } else {
        for (int j = lane; j < a.cols; j += 64) g[j] = (g[j] - dot) * w[j] / a.divisor;
    }
}

// float4 variants: lane l holds columns 4l .. 4l+3 (+ 256 per further vector)
template <int NV>
__global__ __launch_bounds__(WG) void softmax_rows_vec_kernel(SoftmaxArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= a.rows) return;
    float *s = a.scores + row * a.cols;
    const float *mrow = nullptr;
    if (a.mask) {
        const int64_t b = row / a.seq_q, r = row % a.seq_q;
        mrow = a.mask + (b / a.mask_batch_div) * a.mask_batch_stride + r * a.mask_row_stride;
    }
    float v[NV][4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = 4 * lane + 256 * i;
        if (c < a.cols) {
            const float4 t = *reinterpret_cast<const float4 *>(s + c);
            v[i][0] = scaled(a, mrow, t.x, c);     v[i][1] = scaled(a, mrow, t.y, c + 1);
            v[i][2] = scaled(a, mrow, t.z, c + 2); v[i][3] = scaled(a, mrow, t.w, c + 3);
        } else {
            v[i][0] = v[i][1] = v[i][2] = v[i][3] = -INFINITY;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) mx = fmaxf(mx, v[i][e]);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[i][e] = 4 * lane + 256 * i < a.cols ? expf(v[i][e] - mx) : 0.0f;
            sum += v[i][e];
        }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = 4 * lane + 256 * i;
        if (c < a.cols)
            *reinterpret_cast<float4 *>(s + c) = make_float4(v[i][0] / sum, v[i][1] / sum, v[i][2] / sum, v[i][3] / sum);
    }
}

template <int NV>
__global__ __launch_bounds__(WG) void softmax_grad_rows_vec_kernel(SoftmaxGradArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= a.rows) return;
    const float *w = a.weights + row * a.cols;
    float *g = a.grad + row * a.cols;
    float4 gv[NV], wv[NV];
    float dot = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = 4 * lane + 256 * i;
        gv[i] = wv[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (c < a.cols) {
            gv[i] = *reinterpret_cast<const float4 *>(g + c);
            wv[i] = *reinterpret_cast<const float4 *>(w + c);
        }
        dot += gv[i].x * wv[i].x;
        dot += gv[i].y * wv[i].y;
        dot += gv[i].z * wv[i].z;
        dot += gv[i].w * wv[i].w;
    }
    dot = wave_sum(dot);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = 4 * lane + 256 * i;
        if (c < a.cols)
            *reinterpret_cast<float4 *>(g + c) =
                make_float4((gv[i].x - dot) * wv[i].x / a.divisor, (gv[i].y - dot) * wv[i].y / a.divisor,
                            (gv[i].z - dot) * wv[i].z / a.divisor, (gv[i].w - dot) * wv[i].w / a.divisor);
    }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }
// float4 per lane for rows that can move as vectors, 0 otherwise
inline int vectors_per_lane(int cols) { return (cols % 4 || cols > 1024) ? 0 : cols <= 256 ? 1 : cols <= 512 ? 2 : 4; }

}  // namespace

int launch_softmax_rows(float *scores, const float *mask, int mask_batch_div, int64_t mask_batch_stride,
                        int64_t mask_row_stride, int64_t batch, int seq_q, int seq_k, float divisor,
                        hipStream_t stream)
{
    const int64_t rows = batch * seq_q;
    if (rows == 0 || seq_k == 0) return AMSIM_OK;
    const int64_t blocks = (rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
    if (blocks >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "too many attention rows for one launch");
    SoftmaxArgs a{scores, mask, rows, seq_q, seq_k, divisor, mask_batch_div > 0 ? mask_batch_div : 1,
                  mask_batch_stride, mask_row_stride};
    const dim3 grid((unsigned)blocks);
    switch (aligned16(scores) ? vectors_per_lane(seq_k) : 0) {
    case 1: softmax_rows_vec_kernel<1><<<grid, WG, 0, stream>>>(a); break;
    case 2: softmax_rows_vec_kernel<2><<<grid, WG, 0, stream>>>(a); break;
    case 4: softmax_rows_vec_kernel<4><<<grid, WG, 0, stream>>>(a); break;
    default: softmax_rows_kernel<<<grid, WG, 0, stream>>>(a); break;
    }
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

int launch_softmax_grad_rows(const float *weights, float *grad, int64_t rows, int seq_k, float divisor,
                             hipStream_t stream)
{
    if (rows == 0 || seq_k == 0) return AMSIM_OK;
    const int64_t blocks = (rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
    if (blocks >= (1ll << 31)) return fail(AMSIM_ERR_UNSUPPORTED, "too many attention rows for one launch");
    SoftmaxGradArgs a{weights, grad, rows, seq_k, divisor};
    const dim3 grid((unsigned)blocks);
    switch (aligned16(weights) && aligned16(grad) ? vectors_per_lane(seq_k) : 0) {
    case 1: softmax_grad_rows_vec_kernel<1><<<grid, WG, 0, stream>>>(a); break;
    case 2: softmax_grad_rows_vec_kernel<2><<<grid, WG, 0, stream>>>(a); break;
    case 4: softmax_grad_rows_vec_kernel<4><<<grid, WG, 0, stream>>>(a); break;
    default: softmax_grad_rows_kernel<<<grid, WG, 0, stream>>>(a); break;
    }
    AMSIM_HIP_CHECK(hipGetLastError());
    return AMSIM_OK;
}

}  // namespace amsim
