// TensorFlow custom ops over the compressed allreduce schedules: the counterpart of the
// reference's src/tf_ops/tfAllreduce.cc for the three Comprex_* families (the uncompressed
// AlltooneAllreduceApply / RingAllreduceApply / BigringAllreduceApply ops of :113-114,123-124,133-134
// are transport only and stay with the reference).  Same op names, same attributes
// (`T`, `gaspi_allreduce : int` = address of the C++ object), same in-place behaviour, and
// additionally registered for DEVICE_GPU: there the tensor's device buffer goes straight into
// apply()/flush(), which run the HIP kernels on it without a copy.
//
// Build inside a TensorFlow (ROCm) installation:
//   g++ -std=c++14 -shared -fPIC tfAllreduce.cc -I<repo>/include <tf.sysconfig.get_compile_flags()>
//       <tf.sysconfig.get_link_flags()> -L<repo>/comprex_amd/lib -lcomprex_gfx950 -o libtfAllreduce.so
// Without TensorFlow's headers this file still compiles: it then only instantiates the op bodies
// (tf_op_contract.hxx), which is what the build check and the C++ contract test use.
#include <tf_op_contract.hxx>

#if defined(__has_include)
#if __has_include("tensorflow/core/framework/op_kernel.h")
#define COMPREX_HAVE_TENSORFLOW 1
#endif
#endif

#ifdef COMPREX_HAVE_TENSORFLOW

#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/shape_inference.h"

namespace {

using tensorflow::OpKernel;
using tensorflow::OpKernelConstruction;
using tensorflow::OpKernelContext;

// One kernel class for all six ops: the schedule, the element type and apply-or-flush are
// template parameters.
template <template <class> class Schedule, typename T, bool kFlush>
class ComprexAllreduceOp : public OpKernel {
public:
    explicit ComprexAllreduceOp(OpKernelConstruction* construction) : OpKernel(construction), attribute_(0) {
        tensorflow::int64 address = 0;
        OP_REQUIRES_OK(construction, construction->GetAttr("gaspi_allreduce", &address));
        attribute_ = static_cast<comprex_tf::attr_int>(address);
    }
    void Compute(OpKernelContext* context) override {
        tensorflow::Tensor tensor = context->input(0);  // shares the input's buffer
        T* buffer = tensor.flat<T>().data();
        const long long count = tensor.NumElements();
        try {
            if (kFlush) comprex_tf::compute_flush<Schedule, T>(attribute_, buffer, count);
            else comprex_tf::compute_apply<Schedule, T>(attribute_, buffer, count);
        } catch (const std::exception& e) {
            context->CtxFailure(tensorflow::errors::Internal(e.what()));
            return;
        }
        context->set_output(0, tensor);
    }
private:
    comprex_tf::attr_int attribute_;
};

}  // namespace

#define COMPREX_OP(NAME)                                                              \
    REGISTER_OP(NAME)                                                                 \
        .Attr("T: {int32, float32, float64}")                                         \
        .Attr("gaspi_allreduce : int")                                                \
        .Input("input_tensor: T")                                                     \
        .Output("output_tensor: T")                                                   \
        .SetShapeFn([](tensorflow::shape_inference::InferenceContext* c) {            \
            c->set_output(0, c->input(0));                                            \
            return tensorflow::Status();                                              \
        })                                                                            \
        .Doc("Compressed allreduce, in place on the input tensor")
#define COMPREX_KERNELS_FOR(NAME, SCHEDULE, FLUSH, TYPE)                                                  \
    REGISTER_KERNEL_BUILDER(Name(NAME).Device(tensorflow::DEVICE_CPU).TypeConstraint<TYPE>("T"),          \
                            ComprexAllreduceOp<SCHEDULE, TYPE, FLUSH>);                                   \
    REGISTER_KERNEL_BUILDER(Name(NAME).Device(tensorflow::DEVICE_GPU).TypeConstraint<TYPE>("T"),          \
                            ComprexAllreduceOp<SCHEDULE, TYPE, FLUSH>)
#define COMPREX_KERNELS(NAME, SCHEDULE, FLUSH)     \
    COMPREX_KERNELS_FOR(NAME, SCHEDULE, FLUSH, float);  \
    COMPREX_KERNELS_FOR(NAME, SCHEDULE, FLUSH, double); \
    COMPREX_KERNELS_FOR(NAME, SCHEDULE, FLUSH, int)

COMPREX_OP("ComprexAlltooneAllreduceApply");
COMPREX_KERNELS("ComprexAlltooneAllreduceApply", Comprex_AllToOneAllreduce, false);
COMPREX_OP("ComprexAlltooneAllreduceFlush");
COMPREX_KERNELS("ComprexAlltooneAllreduceFlush", Comprex_AllToOneAllreduce, true);
COMPREX_OP("ComprexRingAllreduceApply");
COMPREX_KERNELS("ComprexRingAllreduceApply", Comprex_RingAllreduce, false);
COMPREX_OP("ComprexRingAllreduceFlush");
COMPREX_KERNELS("ComprexRingAllreduceFlush", Comprex_RingAllreduce, true);
COMPREX_OP("ComprexBigringAllreduceApply");
COMPREX_KERNELS("ComprexBigringAllreduceApply", Comprex_BigRingAllreduce, false);
COMPREX_OP("ComprexBigringAllreduceFlush");
COMPREX_KERNELS("ComprexBigringAllreduceFlush", Comprex_BigRingAllreduce, true);

#else  // no TensorFlow: keep the op bodies compiled

template float* comprex_tf::compute_apply<Comprex_AllToOneAllreduce, float>(comprex_tf::attr_int, float*, long long);
template float* comprex_tf::compute_flush<Comprex_AllToOneAllreduce, float>(comprex_tf::attr_int, float*, long long);
template float* comprex_tf::compute_apply<Comprex_RingAllreduce, float>(comprex_tf::attr_int, float*, long long);
template float* comprex_tf::compute_flush<Comprex_RingAllreduce, float>(comprex_tf::attr_int, float*, long long);
template float* comprex_tf::compute_apply<Comprex_BigRingAllreduce, float>(comprex_tf::attr_int, float*, long long);
template float* comprex_tf::compute_flush<Comprex_BigRingAllreduce, float>(comprex_tf::attr_int, float*, long long);
template double* comprex_tf::compute_apply<Comprex_BigRingAllreduce, double>(comprex_tf::attr_int, double*, long long);
template int* comprex_tf::compute_flush<Comprex_RingAllreduce, int>(comprex_tf::attr_int, int*, long long);

#endif
