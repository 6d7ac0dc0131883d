// TensorFlow custom-op library over the C ABI of libffi_hip.so (include/ffi_hip.h): the four ops the reference's
// Python side loads from libsparseops.so (sparse/ops/fixed_fan_in_ops.py:6-12), declared with the names, attrs,
// inputs and outputs of tfsparse/cc/ops/fixed_fan_in_ops.cpp:55-93, and their eight DEVICE_GPU kernels
// (tfsparse/cc/kernels/register.cpp:81-82,90-91,99-100,108-109).  A Compute body extracts raw pointers, shapes
// and TensorFlow's compute stream and makes one C-ABI call; there is no arithmetic in this file.
//
// Built only when a TensorFlow installation is handed to CMake (see ../CMakeLists.txt: FFI_TF_INCLUDE_DIR,
// FFI_TF_LIBRARY); this image has none, so the file is compiled by whoever integrates the library into a ROCm
// TensorFlow.  The eight DEVICE_CPU kernels of the same ops (register.cpp:79-80,88-89,97-98,106-107) are in
// ffi_tf_cpu_ops.cc, part of the same CMake target: one `sparseops` library registers all sixteen.
#define EIGEN_USE_GPU
#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/shape_inference.h"
#include "third_party/eigen3/unsupported/Eigen/CXX11/Tensor"

#include "ffi_hip.h"

namespace {

using ::tensorflow::OpKernel;
using ::tensorflow::OpKernelContext;
using ::tensorflow::Tensor;
using ::tensorflow::TensorShape;
using ::tensorflow::shape_inference::DimensionHandle;
using ::tensorflow::shape_inference::InferenceContext;
using ::tensorflow::shape_inference::ShapeHandle;

// ---- shape functions: the rules of fixed_fan_in_ops.cpp:14-30 (forward) and :32-53 (gradient) -----------------
// every input has rank 2; lookup and weights agree; the batch is dim 0 of features, or dim 1 for the "Tp" ops
template <bool Transposed>
::tensorflow::Status ForwardShape(InferenceContext* c) {
    ShapeHandle features, lookup, weights, connections;
    TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 2, &features));
    TF_RETURN_IF_ERROR(c->WithRank(c->input(1), 2, &lookup));
    TF_RETURN_IF_ERROR(c->WithRank(c->input(2), 2, &weights));
    TF_RETURN_IF_ERROR(c->Merge(lookup, weights, &connections));
    c->set_output(0, c->Matrix(c->Dim(features, Transposed ? 1 : 0), c->Dim(connections, 0)));
    return ::tensorflow::OkStatus();
}

template <bool Transposed>
::tensorflow::Status GradShape(InferenceContext* c) {
    ShapeHandle features, lookup, weights, connections, out_grad, expected;
    TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 2, &features));
    TF_RETURN_IF_ERROR(c->WithRank(c->input(1), 2, &lookup));
    TF_RETURN_IF_ERROR(c->WithRank(c->input(2), 2, &weights));
    TF_RETURN_IF_ERROR(c->WithRank(c->input(3), 2, &out_grad));
    TF_RETURN_IF_ERROR(c->Merge(lookup, weights, &connections));
    // the upstream gradient has the shape of the forward result: [batch, units]
    TF_RETURN_IF_ERROR(c->Merge(out_grad, c->Matrix(c->Dim(features, Transposed ? 1 : 0), c->Dim(connections, 0)), &expected));
    c->set_output(0, features);
    c->set_output(1, connections);
    return ::tensorflow::OkStatus();
}

// TensorFlow's compute stream for this op, as the hipStream_t the C ABI takes: the stream of the op's Eigen GPU device,
// which is what the reference launches on (forward.cu:50-68, backward.cu:59-64: device.stream()) and what every
// TensorFlow 2.x has
void* ComputeStream(OpKernelContext* ctx) {
    return static_cast<void*>(ctx->eigen_device<Eigen::GpuDevice>().stream());
}

struct LayerShape { int64_t batch, num_features, num_units, fan_in; };
template <bool Transposed>
LayerShape ShapeOf(const Tensor& features, const Tensor& lookup) {      // register.cpp:26-27
    return {features.dim_size(Transposed ? 1 : 0), features.dim_size(Transposed ? 0 : 1), lookup.dim_size(0), lookup.dim_size(1)};
}

// int32 and uint32 ids share the entry points: valid ids have the same bits
template <typename Int>
const int32_t* Ids(const Tensor& lookup) { return reinterpret_cast<const int32_t*>(lookup.flat<Int>().data()); }

template <typename Int, bool Transposed>
class FanInSparseMatmulGpuOp : public OpKernel {                        // register.cpp:13-39
 public:
    using OpKernel::OpKernel;
    void Compute(OpKernelContext* ctx) override {
        const Tensor& features = ctx->input(0);
        const Tensor& lookup = ctx->input(1);
        const Tensor& weights = ctx->input(2);
        const LayerShape s = ShapeOf<Transposed>(features, lookup);
        Tensor* result = nullptr;
        OP_REQUIRES_OK(ctx, ctx->allocate_output(0, TensorShape({s.batch, s.num_units}), &result));
        const int status = ffi_forward_f32(features.flat<float>().data(), Ids<Int>(lookup), weights.flat<float>().data(),
                                           result->flat<float>().data(), s.batch, s.num_features, s.num_units, s.fan_in,
                                           Transposed ? 1 : 0, ComputeStream(ctx));
        OP_REQUIRES(ctx, status == FFI_OK, ::tensorflow::errors::Internal("ffi_forward_f32: ", ffi_status_string(status)));
    }
};

template <typename Int, bool Transposed>
class FanInSparseMatmulGradGpuOp : public OpKernel {                    // register.cpp:42-72
 public:
    using OpKernel::OpKernel;
    void Compute(OpKernelContext* ctx) override {
        const Tensor& features = ctx->input(0);
        const Tensor& lookup = ctx->input(1);
        const Tensor& weights = ctx->input(2);
        const Tensor& out_grad = ctx->input(3);
        const LayerShape s = ShapeOf<Transposed>(features, lookup);
        Tensor* feature_grad = nullptr;
        Tensor* weight_grad = nullptr;
        OP_REQUIRES_OK(ctx, ctx->allocate_output(0, features.shape(), &feature_grad));
        OP_REQUIRES_OK(ctx, ctx->allocate_output(1, weights.shape(), &weight_grad));
        const int status = ffi_backward_f32(features.flat<float>().data(), Ids<Int>(lookup), weights.flat<float>().data(),
                                            out_grad.flat<float>().data(), feature_grad->flat<float>().data(),
                                            weight_grad->flat<float>().data(), s.batch, s.num_features, s.num_units, s.fan_in,
                                            Transposed ? 1 : 0, ComputeStream(ctx));
        OP_REQUIRES(ctx, status == FFI_OK, ::tensorflow::errors::Internal("ffi_backward_f32: ", ffi_status_string(status)));
    }
};

}  // namespace

// ---- op declarations (fixed_fan_in_ops.cpp:55-93) ---------------------------------------------------------------
#define FFI_DECLARE_FORWARD_OP(NAME, TRANSPOSED) \
    REGISTER_OP(NAME).Attr("T: type").Attr("I: type").Input("features: T").Input("lookup: I").Input("weights: T") \
        .Output("result: T").SetShapeFn(ForwardShape<TRANSPOSED>)
#define FFI_DECLARE_GRAD_OP(NAME, TRANSPOSED) \
    REGISTER_OP(NAME).Attr("T: type").Attr("I: type").Input("features: T").Input("lookup: I").Input("weights: T") \
        .Input("output: T").Output("feature_grad: T").Output("weight_grad: T").SetShapeFn(GradShape<TRANSPOSED>)

FFI_DECLARE_FORWARD_OP("FanInSparseMatmul", false);
FFI_DECLARE_FORWARD_OP("FanInSparseMatmulTp", true);
FFI_DECLARE_GRAD_OP("FanInSparseMatmulGrad", false);
FFI_DECLARE_GRAD_OP("FanInSparseMatmulGradTp", true);

// ---- the eight GPU kernels (register.cpp:81-82,90-91,99-100,108-109) -------------------------------------------
#define FFI_REGISTER_GPU(OP, CLASS, INT, TRANSPOSED)                                                                      \
    REGISTER_KERNEL_BUILDER(                                                                                              \
        Name(OP).Device(::tensorflow::DEVICE_GPU).TypeConstraint<float>("T").TypeConstraint<::tensorflow::INT>("I"),      \
        CLASS<::tensorflow::INT, TRANSPOSED>)

FFI_REGISTER_GPU("FanInSparseMatmul", FanInSparseMatmulGpuOp, int32, false);
FFI_REGISTER_GPU("FanInSparseMatmul", FanInSparseMatmulGpuOp, uint32, false);
FFI_REGISTER_GPU("FanInSparseMatmulTp", FanInSparseMatmulGpuOp, int32, true);
FFI_REGISTER_GPU("FanInSparseMatmulTp", FanInSparseMatmulGpuOp, uint32, true);
FFI_REGISTER_GPU("FanInSparseMatmulGrad", FanInSparseMatmulGradGpuOp, int32, false);
FFI_REGISTER_GPU("FanInSparseMatmulGrad", FanInSparseMatmulGradGpuOp, uint32, false);
FFI_REGISTER_GPU("FanInSparseMatmulGradTp", FanInSparseMatmulGradGpuOp, int32, true);
FFI_REGISTER_GPU("FanInSparseMatmulGradTp", FanInSparseMatmulGradGpuOp, uint32, true);
