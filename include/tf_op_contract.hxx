// What the reference's TensorFlow ops do with an allreduce object, without TensorFlow
// (src/tf_ops/tfAllreduce.cc:24-41 and :55-72):
//   * the op's attribute `gaspi_allreduce` is a 64-bit integer that IS the address of a
//     `Schedule<T>` object built by the caller (python: ctypes c_void_p -> int);
//   * Compute() calls apply(buffer, count) or flush(buffer, count) IN PLACE on the input tensor's
//     buffer and returns that same tensor as the output.
// The op kernels of comprex_amd/tf_ops/tfAllreduce.cc and the C++ test of this contract both go
// through these functions, so the test exercises the code path of the ops although TensorFlow is
// not needed to build it.  `buffer` may be a host pointer (DEVICE_CPU kernels) or a device pointer
// (DEVICE_GPU kernels): the schedules of allreduce.hxx tell them apart themselves.
#ifndef TF_OP_CONTRACT_HXX
#define TF_OP_CONTRACT_HXX

#include <cstdint>
#include <stdexcept>

#include "allreduce.hxx"

namespace comprex_tf {

typedef long long attr_int;  // tensorflow::int64

template <template <class> class Schedule, typename T> inline attr_int attribute_of(Schedule<T>* object) {
    return static_cast<attr_int>(reinterpret_cast<std::intptr_t>(object));
}

template <template <class> class Schedule, typename T> inline Schedule<T>* object_behind(attr_int attribute) {
    Schedule<T>* object = reinterpret_cast<Schedule<T>*>(static_cast<std::intptr_t>(attribute));
    if (!object) throw std::invalid_argument("gaspi_allreduce: the attribute holds a null address");
    return object;
}

// Both return `buffer`: the op's output aliases its input.
template <template <class> class Schedule, typename T>
inline T* compute_apply(attr_int attribute, T* buffer, long long count) {
    object_behind<Schedule, T>(attribute)->apply(buffer, static_cast<int>(count));
    return buffer;
}

template <template <class> class Schedule, typename T>
inline T* compute_flush(attr_int attribute, T* buffer, long long count) {
    object_behind<Schedule, T>(attribute)->flush(buffer, static_cast<int>(count));
    return buffer;
}

}  // namespace comprex_tf

#endif  // TF_OP_CONTRACT_HXX
