// Small RAII helpers over the cx_* C ABI for the C++ classes of this directory: status ->
// exception, element type -> cx_dtype, a growable device buffer, and a view of a caller's
// pointer that stages pageable host memory through the device when needed.
//
// The reference's classes work on host pointers only.  Here every `T*` argument may be a
// host pointer (staged: copied in, and copied back when the call writes it) or a device
// pointer (used in place), so callers of the reference keep working and GPU-resident callers
// pay nothing.
#ifndef CX_DEVICE_HXX
#define CX_DEVICE_HXX

#include <cstddef>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "comprex_gfx950.h"

namespace cxx {

inline void check(int rc) {
    if (rc != CX_OK) throw std::runtime_error(cx_last_error());
}

template <class T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr cx_dtype value = CX_F32; };
template <> struct dtype_of<double> { static constexpr cx_dtype value = CX_F64; };
template <> struct dtype_of<int> { static constexpr cx_dtype value = CX_I32; };

// One handle (stream + scratch) per object, created on first use so that constructing and
// cloning threshold/compressor objects never touches the GPU.
class Handle {
public:
    Handle() : h_(nullptr) {}
    Handle(const Handle&) : h_(nullptr) {}  // clones get their own scratch
    Handle& operator=(const Handle&) { return *this; }
    ~Handle() { if (h_) cx_destroy(h_); }
    cx_handle get() {
        if (!h_) check(cx_create(&h_, nullptr));
        return h_;
    }
private:
    cx_handle h_;
};

class DeviceBuffer {
public:
    DeviceBuffer() : p_(nullptr), bytes_(0) {}
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { release(); }
    void release() {
        if (p_) cx_device_free(p_);
        p_ = nullptr;
        bytes_ = 0;
    }
    // contents are not preserved
    void* reserve(size_t bytes) {
        if (bytes > bytes_) {
            release();
            check(cx_device_alloc(&p_, bytes));
            bytes_ = bytes;
        }
        return p_;
    }
    void* data() const { return p_; }
    size_t bytes() const { return bytes_; }
private:
    void* p_;
    size_t bytes_;
};

// View of `n` elements at `p` that the GPU can dereference.  A device pointer is used as is;
// a host pointer is copied into `stage` first (when `read`) and copied back by flush() (when
// `write`).
template <class T>
class Staged {
    typedef typename std::remove_const<T>::type U;
public:
    Staged(cx_handle h, DeviceBuffer& stage, T* p, size_t n, bool read, bool write)
        : h_(h), host_(nullptr), dev_(p), staged_(nullptr), bytes_(n * sizeof(T)), write_(write) {
        if (p && n && !cx_pointer_on_device(p)) {
            host_ = p;
            staged_ = static_cast<U*>(stage.reserve(bytes_));
            dev_ = staged_;
            if (read) check(cx_copy(h_, staged_, host_, bytes_));
        }
    }
    T* get() const { return dev_; }
    void flush() {
        if (host_ && write_) check(cx_copy(h_, const_cast<U*>(host_), staged_, bytes_));
    }
private:
    cx_handle h_;
    T* host_;
    T* dev_;
    U* staged_;
    size_t bytes_;
    bool write_;
};

}  // namespace cxx

#endif
