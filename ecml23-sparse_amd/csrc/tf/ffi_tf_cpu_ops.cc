// The eight DEVICE_CPU kernels of the TensorFlow op library (tfsparse/cc/kernels/register.cpp:79-80,88-89,97-98,
// 106-107 registers CPU kernels for every op; the ops themselves are declared in ffi_tf_ops.cc), over the host
// implementation in ../host/ffi_host_kernels.cc.  Work is split over TensorFlow's intra-op thread pool the way the
// reference's functors split it (forward and weight gradient by units, input gradient by batch entries:
// forward.cpp:27-43, backward.cpp:26-35,58-72).
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/lib/core/threadpool.h"

#include "ffi_hip.h"

#include <atomic>

namespace {

using ::tensorflow::OpKernel;
using ::tensorflow::OpKernelContext;
using ::tensorflow::Tensor;
using ::tensorflow::TensorShape;

struct LayerShape { int64_t batch, num_features, num_units, fan_in; };
template <bool Transposed>
LayerShape ShapeOf(const Tensor& features, const Tensor& lookup) {      // register.cpp:26-27
    return {features.dim_size(Transposed ? 1 : 0), features.dim_size(Transposed ? 0 : 1), lookup.dim_size(0), lookup.dim_size(1)};
}
template <typename Int>
const int32_t* Ids(const Tensor& lookup) { return reinterpret_cast<const int32_t*>(lookup.flat<Int>().data()); }

::tensorflow::thread::ThreadPool* Pool(OpKernelContext* ctx) { return ctx->device()->tensorflow_cpu_worker_threads()->workers; }

template <typename Int, bool Transposed>
class FanInSparseMatmulCpuOp : public OpKernel {                        // register.cpp:13-39
 public:
    using OpKernel::OpKernel;
    void Compute(OpKernelContext* ctx) override {
        const Tensor& features = ctx->input(0);
        const Tensor& lookup = ctx->input(1);
        const Tensor& weights = ctx->input(2);
        const LayerShape s = ShapeOf<Transposed>(features, lookup);
        Tensor* result = nullptr;
        OP_REQUIRES_OK(ctx, ctx->allocate_output(0, TensorShape({s.batch, s.num_units}), &result));
        std::atomic<int> status{FFI_OK};
        Pool(ctx)->ParallelFor(s.num_units, s.batch * s.fan_in * 2, [&](int64_t begin, int64_t end) {
            const int st = ffi_host_forward_f32(features.flat<float>().data(), Ids<Int>(lookup), weights.flat<float>().data(),
                                                result->flat<float>().data(), s.batch, s.num_features, s.num_units, s.fan_in,
                                                Transposed ? 1 : 0, begin, end);
            if (st != FFI_OK) status.store(st);
        });
        OP_REQUIRES(ctx, status.load() == FFI_OK, ::tensorflow::errors::InvalidArgument("ffi_host_forward_f32: ", ffi_status_string(status.load())));
    }
};

template <typename Int, bool Transposed>
class FanInSparseMatmulGradCpuOp : public OpKernel {                    // register.cpp:42-72
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
        std::atomic<int> status{FFI_OK};
        const float* x = features.flat<float>().data();
        const float* w = weights.flat<float>().data();
        const float* g = out_grad.flat<float>().data();
        // weight gradient: units over the threads; input gradient: batch entries over the threads
        Pool(ctx)->ParallelFor(s.num_units, s.batch * s.fan_in * 2, [&](int64_t begin, int64_t end) {
            const int st = ffi_host_backward_f32(x, Ids<Int>(lookup), w, g, nullptr, weight_grad->flat<float>().data(), s.batch,
                                                 s.num_features, s.num_units, s.fan_in, Transposed ? 1 : 0, begin, end, 0, 0);
            if (st != FFI_OK) status.store(st);
        });
        Pool(ctx)->ParallelFor(s.batch, s.num_units * s.fan_in * 2, [&](int64_t begin, int64_t end) {
            const int st = ffi_host_backward_f32(x, Ids<Int>(lookup), w, g, feature_grad->flat<float>().data(), nullptr, s.batch,
                                                 s.num_features, s.num_units, s.fan_in, Transposed ? 1 : 0, 0, 0, begin, end);
            if (st != FFI_OK) status.store(st);
        });
        OP_REQUIRES(ctx, status.load() == FFI_OK, ::tensorflow::errors::InvalidArgument("ffi_host_backward_f32: ", ffi_status_string(status.load())));
    }
};

}  // namespace

// ---- the eight CPU kernels (register.cpp:79-80,88-89,97-98,106-107) --------------------------------------------
#define FFI_REGISTER_CPU(OP, CLASS, INT, TRANSPOSED)                                                                      \
    REGISTER_KERNEL_BUILDER(                                                                                              \
        Name(OP).Device(::tensorflow::DEVICE_CPU).TypeConstraint<float>("T").TypeConstraint<::tensorflow::INT>("I"),      \
        CLASS<::tensorflow::INT, TRANSPOSED>)

FFI_REGISTER_CPU("FanInSparseMatmul", FanInSparseMatmulCpuOp, int32, false);
FFI_REGISTER_CPU("FanInSparseMatmul", FanInSparseMatmulCpuOp, uint32, false);
FFI_REGISTER_CPU("FanInSparseMatmulTp", FanInSparseMatmulCpuOp, int32, true);
FFI_REGISTER_CPU("FanInSparseMatmulTp", FanInSparseMatmulCpuOp, uint32, true);
FFI_REGISTER_CPU("FanInSparseMatmulGrad", FanInSparseMatmulGradCpuOp, int32, false);
FFI_REGISTER_CPU("FanInSparseMatmulGrad", FanInSparseMatmulGradCpuOp, uint32, false);
FFI_REGISTER_CPU("FanInSparseMatmulGradTp", FanInSparseMatmulGradCpuOp, int32, true);
FFI_REGISTER_CPU("FanInSparseMatmulGradTp", FanInSparseMatmulGradCpuOp, uint32, true);
