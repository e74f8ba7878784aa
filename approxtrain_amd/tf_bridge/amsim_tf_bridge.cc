// TensorFlow bridge: the GPU functor specialisations and the GPU LUT class of
// ApproxTrain's custom ops, implemented on top of libamsim's C ABI (amsim.h).
//
// This one translation unit takes the place of the reference's device objects
//   cuda/cuda_kernel.cu  cuda/gemm.cu  cuda/reverseNswapdim23.cu
//   cuda/denseam_kernel.cu  cuda/matmulam_kernel.cu  cuda/approx_mul_lut.cu
// in convam_gpu.so, denseam_gpu.so and matmulam.so (Makefile:21-46).  The op
// registrations, attribute checks, shape functions and OpKernel::Compute bodies
// (convam.cc, denseam.cc, matmulam.cc) and the Python layers stay as they are:
// they reach the device only through the functors declared in convam.h:69-143,
// denseam.h:7-53 and matmulam.h:10-28, which are defined here.
//
// Build (ROCm build of TensorFlow >= 2.3; -DGOOGLE_CUDA=1 as in Makefile:3 so
// that the headers declare the GPU specialisations):
//   hipcc -std=c++14 -O2 -fPIC -DGOOGLE_CUDA=1 -DEIGEN_USE_GPU -DEIGEN_USE_HIP
//         -DTENSORFLOW_USE_ROCM=1 $TF_CFLAGS -I<ApproxTrain> -I<this repo>/include \
//         -c amsim_tf_bridge.cc -o amsim_tf_bridge.o
//   g++ -shared convam.o amsim_tf_bridge.o $TF_LFLAGS -L<this repo>/approxtrain_amd -lamsim
//         -L/opt/rocm/lib -lamdhip64 -o convam_gpu.so        (same for denseam_gpu.so, matmulam.so)
//
// Scratch memory.  The C ABI never allocates: every entry point takes a
// workspace (pre-decoded uniform operand, partial sums of split reductions)
// whose size the matching *_workspace_bytes_for query returns.  The dense and
// matmul functors of the reference carry no temporary at all and the
// convolution functors an im2col buffer sized for another algorithm, so each
// functor here takes a temporary from TensorFlow's own allocator through the
// Eigen device it is handed: GpuDevice::allocate / deallocate forward to the
// stream interface TensorFlow installs for the running op (EigenGpuStreamDevice
// in common_runtime/gpu/gpu_device.cc), which allocates from the op's device
// allocator -- the functor-level form of OpKernelContext::allocate_temp -- and
// defers the release until the stream has passed the kernels enqueued before
// it.  No lock, no hipMalloc, no synchronisation; two ops running concurrently
// hold separate temporaries.  The im2col / rsfilter temporaries of convam.cc
// are unused here and can shrink to one element.
//
// int32 kernels: the reference registers them (convam.cc:620 etc.) but its
// device product treats the integers as floats.  They are not provided; the
// instantiations exist so that the registrations link, and abort with a
// message when run.
#define EIGEN_USE_GPU
#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/platform/logging.h"

#include "amsim.h"
#include "approx_mul_lut.h"
#include "convam.h"
#include "denseam.h"
#include "matmulam.h"

using GPUDevice = Eigen::GpuDevice;
using tensorflow::int32;

namespace {

// ---- scratch from TensorFlow's allocator, for the duration of one functor call -------------
class Scratch {
public:
    Scratch(const GPUDevice &d, size_t bytes) : d_(d), bytes_(bytes)
    {
        if (bytes_ == 0) return;
        raw_ = d_.allocate(bytes_ + 256);  // the C ABI wants 256-byte alignment; the allocator promises less
        if (raw_ == nullptr) LOG(FATAL) << "amsim bridge: cannot allocate " << bytes_ << " bytes of scratch";
        ptr_ = reinterpret_cast<void *>((reinterpret_cast<uintptr_t>(raw_) + 255) & ~static_cast<uintptr_t>(255));
    }
    // handed back once the call's kernels are enqueued: the release is ordered behind them on the stream
    ~Scratch() { if (raw_) d_.deallocate(raw_); }
    Scratch(const Scratch &) = delete;
    Scratch &operator=(const Scratch &) = delete;
    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }

private:
    const GPUDevice &d_;
    size_t bytes_;
    void *raw_ = nullptr, *ptr_ = nullptr;
};

void check(int status, const char *what)
{
    // the reference prints and exits on device errors (cuda/error.cuh:9-27)
    if (status != AMSIM_OK) LOG(FATAL) << what << ": " << amsim_status_string(status) << ": " << amsim_last_error();
}

amsim_lut_t handle_of(approx_mul_lut<GPUDevice> &l)
{
    return reinterpret_cast<amsim_lut_t>(static_cast<uintptr_t>(l.get_mant_mul_lut_text_()));
}

[[noreturn]] void no_int32(const char *op)
{
    LOG(FATAL) << op << "<int32> on the GPU is not provided by libamsim (float only)";
    abort();
}

}  // namespace

// ---- approx_mul_lut<GPUDevice> (approx_mul_lut.h:73-78, cuda/approx_mul_lut.cu:24-53)
// The base class has read the file into mant_mul_lut_ and derived the width
// from its name; the device image lives in an amsim_lut_t whose pointer is
// kept in the 64-bit slot the reference uses for its texture object.
template <>
approx_mul_lut<GPUDevice>::approx_mul_lut(tensorflow::OpKernelConstruction *context) : approx_mul_lut_base(context)
{
    mant_mul_lut_cuda_ = nullptr;
    amsim_lut_t h = nullptr;
    const int rc = amsim_lut_create(mant_mul_lut_.data(), mant_mul_lut_.size(), mant_width_, 1, &h);
    OP_REQUIRES(context, rc == AMSIM_OK, tensorflow::errors::InvalidArgument("mant_mul_lut: ", amsim_last_error()));
    mant_mul_lut_text_ = static_cast<cudaTextureObject_t>(reinterpret_cast<uintptr_t>(h));
}

template <>
approx_mul_lut<GPUDevice>::~approx_mul_lut()
{
    if (mant_mul_lut_text_) amsim_lut_destroy(handle_of(*this));
}

// ---- convolution (convam.h:71-104) --------------------------------------------
template <typename T>
void ConvamFunctor<GPUDevice, T>::operator()(const GPUDevice &d, const T *input_data, T *output_data, const int batch,
                                             const int out_rows, const int out_cols, const int out_depth,
                                             const int stride_cols, const int stride_rows,
                                             const int filter_left_offset, const int filter_top_offset,
                                             const int filter_rows, const int filter_cols, const int in_depth,
                                             const int input_cols, const int input_rows, const T *filter,
                                             T * /*im2col*/, const int /*padding*/,
                                             approx_mul_lut<GPUDevice> &mul_lut)
{
    // (the table-aware queries: tables wider than 7 bits also get the staged operand their engine reads)
    const size_t ws = amsim_convam_workspace_bytes_for(handle_of(mul_lut), batch, out_rows, out_cols, out_depth, filter_rows,
                                                       filter_cols, in_depth);
    Scratch scratch(d, ws);
    check(amsim_convam_f32(handle_of(mul_lut), input_data, output_data, batch, out_rows, out_cols, out_depth,
                           stride_cols, stride_rows, filter_left_offset, filter_top_offset, filter_rows, filter_cols,
                           in_depth, input_cols, input_rows, filter, scratch.ptr(), scratch.bytes(), d.stream()),
          "Convam");
}
template <>
void ConvamFunctor<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, int32 *, const int, const int,
                                                 const int, const int, const int, const int, const int, const int,
                                                 const int, const int, const int, const int, const int, const int32 *,
                                                 int32 *, const int, approx_mul_lut<GPUDevice> &)
{
    no_int32("Convam");
}

template <typename T>
void ConvamInputGradFunctor<GPUDevice, T>::operator()(const GPUDevice &d, const T *grad, T * /*im2col*/,
                                                      const int hole_grad_width, const int hole_grad_height,
                                                      const int pad_top, const int pad_left, const T *filter,
                                                      T * /*rsfilter*/, const int filter_rows, const int filter_cols,
                                                      const int out_depth, const int stride_rows,
                                                      const int stride_cols, const int batch, const int input_rows,
                                                      const int input_cols, const int in_depth, T *output,
                                                      const int out_rows, const int out_cols,
                                                      approx_mul_lut<GPUDevice> &mul_lut)
{
    // with strides the call is a set of undilated sub-problems: size the scratch so each may split its reduction
    const size_t ws = amsim_convam_input_grad_workspace_bytes_for(handle_of(mul_lut), batch, input_rows, input_cols,
                                                                  in_depth, filter_rows, filter_cols, out_depth,
                                                                  stride_rows, stride_cols, pad_top, pad_left);
    Scratch scratch(d, ws);
    check(amsim_convam_input_grad_f32(handle_of(mul_lut), grad, hole_grad_width, hole_grad_height, pad_top, pad_left,
                                      filter, filter_rows, filter_cols, out_depth, stride_rows, stride_cols, batch,
                                      input_rows, input_cols, in_depth, output, out_rows, out_cols,
                                      scratch.ptr(), scratch.bytes(), d.stream()),
          "ConvamInputGrad");
}
template <>
void ConvamInputGradFunctor<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, int32 *, const int,
                                                          const int, const int, const int, const int32 *, int32 *,
                                                          const int, const int, const int, const int, const int,
                                                          const int, const int, const int, const int, int32 *,
                                                          const int, const int, approx_mul_lut<GPUDevice> &)
{
    no_int32("ConvamInputGrad");
}

template <typename T>
void ConvamFilterGradFunctor<GPUDevice, T>::operator()(const GPUDevice &d, const T *input, const T *grad,
                                                       T * /*im2col*/, const int input_rows, const int input_cols,
                                                       const int batch, const int in_depth, const int out_cols,
                                                       const int out_rows, const int out_depth,
                                                       const int filter_left_offset, const int filter_top_offset,
                                                       const int stride_rows, const int stride_cols,
                                                       const int filter_cols, const int filter_rows, T *output,
                                                       approx_mul_lut<GPUDevice> &mul_lut)
{
    const size_t ws = amsim_convam_filter_grad_workspace_bytes_for(handle_of(mul_lut), batch, out_rows, out_cols, out_depth,
                                                                   filter_rows, filter_cols, in_depth);
    Scratch scratch(d, ws);
    check(amsim_convam_filter_grad_f32(handle_of(mul_lut), input, grad, input_rows, input_cols, batch, in_depth,
                                       out_cols, out_rows, out_depth, filter_left_offset, filter_top_offset,
                                       stride_rows, stride_cols, filter_cols, filter_rows, output,
                                       scratch.ptr(), scratch.bytes(), d.stream()),
          "ConvamFilterGrad");
}
template <>
void ConvamFilterGradFunctor<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, const int32 *, int32 *,
                                                           const int, const int, const int, const int, const int,
                                                           const int, const int, const int, const int, const int,
                                                           const int, const int, const int, int32 *,
                                                           approx_mul_lut<GPUDevice> &)
{
    no_int32("ConvamFilterGrad");
}

template struct ConvamFunctor<GPUDevice, float>;
template struct ConvamFunctor<GPUDevice, int32>;
template struct ConvamInputGradFunctor<GPUDevice, float>;
template struct ConvamInputGradFunctor<GPUDevice, int32>;
template struct ConvamFilterGradFunctor<GPUDevice, float>;
template struct ConvamFilterGradFunctor<GPUDevice, int32>;

// ---- dense (denseam.h:9-27) -----------------------------------------------------
template <typename T>
void DenseamFunctor<GPUDevice, T>::operator()(const GPUDevice &d, const T *inputs, const T *weights, T *output,
                                              const int batch, const int units, const int input_width,
                                              approx_mul_lut<GPUDevice> &mul_lut)
{
    const size_t ws = amsim_denseam_workspace_bytes_for(handle_of(mul_lut), batch, units, input_width);
    Scratch scratch(d, ws);
    check(amsim_denseam_f32(handle_of(mul_lut), inputs, weights, output, batch, units, input_width,
                            scratch.ptr(), scratch.bytes(), d.stream()),
          "Denseam");
}
template <>
void DenseamFunctor<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, const int32 *, int32 *, const int,
                                                  const int, const int, approx_mul_lut<GPUDevice> &)
{
    no_int32("Denseam");
}

template <typename T>
void DenseamWeightGradFunctor<GPUDevice, T>::operator()(const GPUDevice &d, const T *input, const T *grads, T *output,
                                                        const int batch, const int units, const int input_width,
                                                        approx_mul_lut<GPUDevice> &mul_lut)
{
    const size_t ws = amsim_denseam_workspace_bytes_for(handle_of(mul_lut), batch, units, input_width);
    Scratch scratch(d, ws);
    check(amsim_denseam_weight_grad_f32(handle_of(mul_lut), input, grads, output, batch, units, input_width,
                                        scratch.ptr(), scratch.bytes(), d.stream()),
          "DenseamGrad (weights)");
}
template <>
void DenseamWeightGradFunctor<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, const int32 *, int32 *,
                                                            const int, const int, const int,
                                                            approx_mul_lut<GPUDevice> &)
{
    no_int32("DenseamGrad");
}

template <typename T>
void DenseamInputGradFunctor<GPUDevice, T>::operator()(const GPUDevice &d, const T *weight, const T *grads, T *output,
                                                       const int batch, const int units, const int input_width,
                                                       approx_mul_lut<GPUDevice> &mul_lut)
{
    const size_t ws = amsim_denseam_workspace_bytes_for(handle_of(mul_lut), batch, units, input_width);
    Scratch scratch(d, ws);
    check(amsim_denseam_input_grad_f32(handle_of(mul_lut), weight, grads, output, batch, units, input_width,
                                       scratch.ptr(), scratch.bytes(), d.stream()),
          "DenseamGrad (inputs)");
}
template <>
void DenseamInputGradFunctor<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, const int32 *, int32 *,
                                                           const int, const int, const int,
                                                           approx_mul_lut<GPUDevice> &)
{
    no_int32("DenseamGrad");
}

template struct DenseamFunctor<GPUDevice, float>;
template struct DenseamFunctor<GPUDevice, int32>;
template struct DenseamWeightGradFunctor<GPUDevice, float>;
template struct DenseamWeightGradFunctor<GPUDevice, int32>;
template struct DenseamInputGradFunctor<GPUDevice, float>;
template struct DenseamInputGradFunctor<GPUDevice, int32>;

// ---- MatMulAM (matmulam.h:12-17) ---------------------------------------------------
// One strided-batch call instead of the per-item launch loop of matmulam_kernel.cu:30-98;
// batch_a / batch_b are 0 for rank-2 operands exactly as MatMulAMOp::Compute passes them
// (matmulam.cc:86-147).
template <typename T>
void LaunchMatMul<GPUDevice, T>::operator()(const GPUDevice &d, const T *a, const T *b, const int batch_a,
                                            const int batch_b, const int row_a, const int col_a, const int row_b,
                                            const int col_b, T *out, approx_mul_lut<GPUDevice> &mul_lut)
{
    const size_t ws = amsim_matmulam_workspace_bytes_for(handle_of(mul_lut), batch_a, batch_b, row_a, col_a, row_b, col_b);
    Scratch scratch(d, ws);
    check(amsim_matmulam_f32(handle_of(mul_lut), a, b, batch_a, batch_b, row_a, col_a, row_b, col_b, out,
                             scratch.ptr(), scratch.bytes(), d.stream()),
          "MatMulAM");
}
template <>
void LaunchMatMul<GPUDevice, int32>::operator()(const GPUDevice &, const int32 *, const int32 *, const int, const int,
                                                const int, const int, const int, const int, int32 *,
                                                approx_mul_lut<GPUDevice> &)
{
    no_int32("MatMulAM");
}

template struct LaunchMatMul<GPUDevice, float>;
template struct LaunchMatMul<GPUDevice, int32>;
