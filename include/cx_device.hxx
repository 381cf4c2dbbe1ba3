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
#include <memory>
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

// The stream an object's GPU work runs on, and the stream its caller's vectors live on.
//
// The reference's calls are synchronous host code; here they enqueue GPU work.  Every object
// (a ComprEx with its compressor and threshold clones, or a compressor / threshold used on its
// own) has a stream of its own, so that independent channels overlap.  What keeps a caller's
// vector safe is the order between that stream and the caller's ("origin", NULL = the null stream,
// where plain hipMemcpy / framework default-stream work runs): the object's work on the vector
// runs after what the origin was given before the call and before what it is given afterwards.
// For the null stream the runtime keeps that order itself (the object's stream is created
// "blocking": null-stream work waits for it and it waits for null-stream work), which spares the
// host two event joins of 8 to 9 us per call.  For any other origin a pair of joins brackets every
// call: on entry the object's stream waits for an event recorded on the origin, on exit the
// origin waits for one recorded on the object's stream; the host never blocks.  Scopes nest (a
// ComprEx call that runs its threshold's prepare joins once).
class StreamCtx {
public:
    StreamCtx() : stream_(nullptr), owned_(false), made_(false), origin_(nullptr), ev_(nullptr), depth_(0) {}
    StreamCtx(const StreamCtx&) = delete;
    StreamCtx& operator=(const StreamCtx&) = delete;
    ~StreamCtx() {
        if (ev_) cx_event_destroy(ev_);
        if (owned_ && stream_) {
            cx_stream_synchronize(stream_);
            cx_stream_destroy(stream_);
        }
    }
    // the object's stream, created on first use
    // (a "blocking" stream: the runtime orders it with the null stream both ways, so a caller on the null
    // stream, the reference's style and a framework's default stream, needs no join; other objects'
    // streams are not ordered with it)
    void* stream() {
        if (!made_) {
            check(cx_stream_create_blocking(&stream_));
            owned_ = true;
            made_ = true;
        }
        return stream_;
    }
    // run on a stream of the caller's instead (not owned; NULL = the null stream)
    void adopt(void* hip_stream) {
        if (made_ && owned_ && stream_) {
            check(cx_stream_synchronize(stream_));
            check(cx_stream_destroy(stream_));
        }
        stream_ = hip_stream;
        owned_ = false;
        made_ = true;
    }
    void set_origin(void* hip_stream) { origin_ = hip_stream; }
    void* origin() const { return origin_; }

    // the object's own stream and the null stream order themselves
    bool ordered_by_runtime(void* s) const { return s == origin_ || (owned_ && origin_ == nullptr); }
    void enter() {
        if (depth_++ > 0) return;
        void* s = stream();
        if (ordered_by_runtime(s)) return;
        check(cx_event_record(event(), origin_));
        check(cx_stream_wait_event(s, event()));
    }
    void leave() {
        if (--depth_ > 0) return;
        void* s = stream();
        if (ordered_by_runtime(s)) return;
        if (cx_event_record(event(), s) == CX_OK) cx_stream_wait_event(origin_, event());
    }

private:
    void* event() {
        if (!ev_) check(cx_event_create(&ev_));
        return ev_;
    }
    void* stream_;
    bool owned_, made_;
    void* origin_;
    void* ev_;
    int depth_;
};

// Joins the object's stream with the caller's for the time of one call.
class Scope {
public:
    explicit Scope(StreamCtx& c) : c_(c) { c_.enter(); }
    ~Scope() { c_.leave(); }
    Scope(const Scope&) = delete;
    Scope& operator=(const Scope&) = delete;
private:
    StreamCtx& c_;
};

// Orders two streams once: everything `later` is given from now on runs after what `earlier` holds now.
class StreamOrder {
public:
    StreamOrder() : turn_(0) { ev_[0] = ev_[1] = nullptr; }
    StreamOrder(const StreamOrder&) : turn_(0) { ev_[0] = ev_[1] = nullptr; }
    StreamOrder& operator=(const StreamOrder&) { return *this; }
    ~StreamOrder() {
        for (int i = 0; i < 2; ++i)
            if (ev_[i]) cx_event_destroy(ev_[i]);
    }
    void order(void* earlier, void* later) {
        if (earlier == later) return;
        void*& ev = ev_[turn_ ^= 1];  // two events in turn: one is never recorded again while its wait is fresh
        if (!ev) check(cx_event_create(&ev));
        check(cx_event_record(ev, earlier));
        check(cx_stream_wait_event(later, ev));
    }
private:
    void* ev_[2];
    int turn_;
};

// One handle (scratch, on the object's stream) per object, created on first use so that
// constructing and cloning threshold/compressor objects never touches the GPU.
class Handle {
public:
    Handle() : ctx_(std::make_shared<StreamCtx>()), h_(nullptr) {}
    Handle(const Handle&) : ctx_(std::make_shared<StreamCtx>()), h_(nullptr) {}  // clones get their own scratch and stream
    Handle& operator=(const Handle&) { return *this; }
    ~Handle() { if (h_) cx_destroy(h_); }
    cx_handle get() {
        if (!h_) check(cx_create(&h_, ctx_->stream()));
        return h_;
    }
    StreamCtx& ctx() { return *ctx_; }
    const std::shared_ptr<StreamCtx>& ctx_ptr() const { return ctx_; }
    // share another object's stream (a ComprEx and its clones work on one stream)
    void bind(const std::shared_ptr<StreamCtx>& c) {
        ctx_ = c;
        refresh();
    }
    // the context's stream changed (StreamCtx::adopt)
    void refresh() {
        if (h_) check(cx_set_stream(h_, ctx_->stream()));
    }
private:
    std::shared_ptr<StreamCtx> ctx_;  // outlives the handle: cx_destroy waits for the stream
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
