// Compressors with the interface of the reference's src/compressor.hxx, computed on the GPU
// through the cx_* C ABI.
//
//   Compressor<T>            base: compress / compress_update / compress_add_update /
//                            decompress / add / clone          (reference src/compressor.hxx:24-76)
//   CompressorNone<T>        dense copy: int32 n, then n values (:83-151)
//   CompressorIndexPairs<T>  int32 n, int32 k, k x (int32 index, T value), ascending index
//                                                              (:538-661)
//   CompressorRLE<T>         run-length codec: values + alternating run lengths  (:158-532)
//
// Vectors and message buffers may be host or device pointers.  The reference's calls carry no
// buffer capacity; like the reference, the buffer is trusted to hold the message
// (8 + n*(4+sizeof(T)) bytes at most).  ComprEx uses the *_device entry points, which do carry
// the capacity and can take the threshold from device memory.
#ifndef COMPRESSOR_H
#define COMPRESSOR_H

#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>

#include "cx_device.hxx"
#include "threshold.hxx"

template <class VarTYPE>
class Compressor {
public:
    Compressor() {}
    Compressor(const Compressor<VarTYPE>&) {}
    virtual ~Compressor() {}

    // writes the compressed vector into targetBuffer, returns the bytes written
    virtual int compress(void* targetBuffer, const VarTYPE* data_vector, const int data_vector_size,
                         VarTYPE threshold) {
        cxx::Scope scope(handle_.ctx());
        return compression_strategy(targetBuffer, data_vector, NULL, data_vector_size, threshold);
    }
    virtual int compress_update(void* targetBuffer, VarTYPE* update_vector, const int update_vector_size,
                                VarTYPE threshold) {
        cxx::Scope scope(handle_.ctx());
        return compression_strategy(targetBuffer, NULL, update_vector, update_vector_size, threshold);
    }
    virtual int compress_add_update(void* targetBuffer, VarTYPE* update_vector, const int update_vector_size,
                                    const VarTYPE* data_vector, const int data_vector_size, VarTYPE threshold) {
        check_sizes(update_vector_size, data_vector_size);
        cxx::Scope scope(handle_.ctx());
        return compression_strategy(targetBuffer, data_vector, update_vector, update_vector_size, threshold);
    }

    // returns the bytes consumed from sourceBuffer
    virtual int decompress(VarTYPE* output, int output_size, const void* sourceBuffer) {
        cxx::Scope scope(handle_.ctx());
        return decompression_strategy(output, output_size, sourceBuffer);
    }
    virtual void add(VarTYPE* output, int output_size, const void* sourceBuffer) {
        cxx::Scope scope(handle_.ctx());
        return add_strategy(output, output_size, sourceBuffer);
    }

    virtual Compressor<VarTYPE>* clone() const = 0;

    // Not in the reference: adds `count` messages (device addresses) to `output` in the order given,
    // which is what the chief's loop over its workers does, one add() per worker
    // (src/allreduce.tpp:186-189); a compressor may do it in one pass over `output`.
    virtual void add_many(VarTYPE* output, int output_size, const void* const* d_sources, int count) {
        for (int i = 0; i < count; ++i) add(output, output_size, d_sources[i]);
    }

    // Not in the reference: the stream this object's GPU work runs on and the caller's stream it is
    // joined with around every call (cx_device.hxx).  A ComprEx binds its clones to its own.
    void bind_stream(const std::shared_ptr<cxx::StreamCtx>& ctx) { handle_.bind(ctx); }
    cxx::StreamCtx& stream_context() { return handle_.ctx(); }
    void stream_changed() { handle_.refresh(); }

    // Not in the reference: bytes of the largest message a vector of n elements can produce.
    virtual long long max_message_bytes(int n) const = 0;

    // Not in the reference: sizes this compressor's GPU scratch for vectors of up to n elements, so
    // that the exchange itself never allocates (the reference takes its memory in the constructors
    // too, src/comprEx.tpp:40-60).  `whole_vector_topk`: the one-pass exact top-k will be used.
    virtual void reserve(int n, bool whole_vector_topk) {
        cxx::check(cx_reserve(handle_.get(), cxx::dtype_of<VarTYPE>::value, n,
                              reserve_paths() | (whole_vector_topk ? (unsigned)CX_RESERVE_THRESHOLD : 0u)));
    }

    // Not in the reference: waits for this compressor's GPU work and returns (and forgets) the first
    // error a kernel recorded since the last call, CX_OK if none.  A message cut short for lack of
    // room (CX_ERR_CAPACITY) is valid as far as it goes; what it could not hold stayed in the
    // update vector.
    virtual int device_status() { return cx_synchronize(handle_.get()); }

    // Device-side entry used by ComprEx: all pointers are device pointers, `capacity` is the
    // size of d_target in bytes, the threshold comes from d_threshold (device) or, when that is
    // NULL, from `threshold`.  d_size_prefix (may be NULL) receives the message's byte count.
    // With wait == false the call only enqueues work and returns -1 instead of the byte count.
    virtual int compress_device(void* d_target, long long capacity, const VarTYPE* d_data, VarTYPE* d_update, int n,
                                const VarTYPE* d_threshold, VarTYPE threshold, int* d_size_prefix, bool wait) = 0;
    virtual int decompress_device(VarTYPE* d_output, int output_size, const void* d_source, bool wait) = 0;
    virtual void add_device(VarTYPE* d_output, int output_size, const void* d_source) = 0;

    // Not in the reference.  ThresholdTopK(rule)::prepare_with(d_update, d_data) and
    // compress_add_update as one call that only enqueues work; the threshold is left in d_thr_out.
    // Returns false, having done nothing, when the compressor has no such path.
    virtual bool write_step_device(void* d_target, long long capacity, const VarTYPE* d_data, VarTYPE* d_update, int n,
                                   const typename ThresholdFunction<VarTYPE>::TopKRule& rule, VarTYPE* d_thr_out,
                                   int* d_size_prefix) {
        return false;
    }

protected:
    virtual int compression_strategy(void* output, const VarTYPE* data_vector, VarTYPE* update_vector,
                                     const int vector_size, VarTYPE threshold) = 0;
    virtual int decompression_strategy(VarTYPE* output, int output_size, const void* input) = 0;
    virtual void add_strategy(VarTYPE* output, int output_size, const void* sourceBuffer) = 0;

    // Status of a receive: a message that an earlier SEND of this compressor had to cut short is no
    // concern of the receive (the note is dropped; flushRests sends what stayed behind).
    static int receive_status(cx_handle h) {
        const int rc = cx_synchronize(h);
        return rc == CX_ERR_CAPACITY ? cx_synchronize(h) : rc;
    }

    static void check_sizes(int update_vector_size, int data_vector_size) {
        if (data_vector_size != update_vector_size) {
            char msg[100];
            snprintf(msg, sizeof msg, "Compressor: Update vector size (%d) is not equal data vector size (%d)!",
                     update_vector_size, data_vector_size);
            throw std::runtime_error(msg);
        }
    }

    virtual unsigned reserve_paths() const { return CX_RESERVE_COMPRESS | CX_RESERVE_REDUCE; }
    cxx::Handle handle_;
    cxx::DeviceBuffer stage_msg_, stage_a_, stage_b_;
};

// ---------------------------------------------------------------------------------------
template <class VarTYPE>
class CompressorIndexPairs : public Compressor<VarTYPE> {
public:
    CompressorIndexPairs() : _topK(0) {}
    CompressorIndexPairs(float topK) : _topK(topK) {}
    CompressorIndexPairs(const CompressorIndexPairs<VarTYPE>& other) : Compressor<VarTYPE>(other), _topK(other._topK) {}

    virtual Compressor<VarTYPE>* clone() const { return new CompressorIndexPairs<VarTYPE>(*this); }

    virtual long long max_message_bytes(int n) const { return 8 + (long long)n * (4 + (long long)sizeof(VarTYPE)); }

    virtual int compress_device(void* d_target, long long capacity, const VarTYPE* d_data, VarTYPE* d_update, int n,
                                const VarTYPE* d_threshold, VarTYPE threshold, int* d_size_prefix, bool wait) {
        int bytes = -1;
        cxx::check(cx_ip_compress(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_target, capacity, d_data,
                                  d_update, n, d_threshold ? nullptr : &threshold, d_threshold, d_size_prefix,
                                  wait ? &bytes : nullptr));
        return bytes;
    }
    virtual bool write_step_device(void* d_target, long long capacity, const VarTYPE* d_data, VarTYPE* d_update, int n,
                                   const typename ThresholdFunction<VarTYPE>::TopKRule& rule, VarTYPE* d_thr_out,
                                   int* d_size_prefix) {
        cxx::check(cx_ip_write_step(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_target, capacity, d_data,
                                    d_update, n, rule.topK, rule.default_subsamples, rule.subsample_factor,
                                    rule.d_positions, rule.n_positions, d_thr_out, d_size_prefix, nullptr));
        return true;
    }
    virtual int decompress_device(VarTYPE* d_output, int output_size, const void* d_source, bool wait) {
        int bytes = -1;
        cxx::check(cx_ip_decompress(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_output, output_size,
                                    d_source, wait ? &bytes : nullptr));
        return bytes;
    }
    virtual void add_device(VarTYPE* d_output, int output_size, const void* d_source) {
        cxx::check(cx_ip_add(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_output, output_size, d_source, 1));
    }

protected:
    float _topK;

    virtual int compression_strategy(void* output, const VarTYPE* data_vector, VarTYPE* update_vector,
                                     const int vector_size, VarTYPE threshold) {
        cx_handle h = this->handle_.get();
        const long long cap = max_message_bytes(vector_size);
        cxx::Staged<const VarTYPE> d(h, this->stage_a_, data_vector, (size_t)(data_vector ? vector_size : 0), true, false);
        cxx::Staged<VarTYPE> u(h, this->stage_b_, update_vector, (size_t)(update_vector ? vector_size : 0), true, true);
        const bool host_out = !cx_pointer_on_device(output);
        void* d_out = host_out ? this->stage_msg_.reserve((size_t)cap) : output;
        const int bytes = compress_device(d_out, cap, data_vector ? d.get() : nullptr,
                                          update_vector ? u.get() : nullptr, vector_size, nullptr, threshold, nullptr,
                                          true);
        if (host_out) cxx::check(cx_copy(h, output, d_out, (size_t)bytes));
        u.flush();
        return bytes;
    }

    // message header as the host sees it
    void read_header(const void* msg, int hdr[2]) {
        cx_handle h = this->handle_.get();
        cxx::check(cx_copy(h, hdr, msg, 8));
        cxx::check(cx_synchronize(h));
    }

    // a host-resident message is staged whole (its length comes from its own header)
    const void* stage_message(const void* msg) {
        if (cx_pointer_on_device(msg)) return msg;
        int hdr[2];
        std::memcpy(hdr, msg, 8);
        const size_t bytes = 8 + (size_t)(hdr[1] < 0 ? 0 : hdr[1]) * (4 + sizeof(VarTYPE));
        void* d = this->stage_msg_.reserve(bytes);
        cxx::check(cx_copy(this->handle_.get(), d, msg, bytes));
        return d;
    }

    virtual int decompression_strategy(VarTYPE* output, int output_size, const void* input) {
        cx_handle h = this->handle_.get();
        const void* d_in = stage_message(input);
        cxx::Staged<VarTYPE> o(h, this->stage_a_, output, (size_t)output_size, false, true);
        int bytes = 0;
        const int rc = cx_ip_decompress(h, cxx::dtype_of<VarTYPE>::value, o.get(), output_size, d_in, &bytes);
        o.flush();  // the reference zeroes the output before its size check throws
        if (rc == CX_ERR_MSG_TOO_LARGE) {
            int hdr[2];
            read_header(d_in, hdr);
            char msg[100];
            snprintf(msg, sizeof msg, "Decompression vector size (%d) is bigger than output buffer (%d)!", hdr[0],
                     output_size);
            throw std::runtime_error(msg);
        }
        cxx::check(rc);
        return bytes;
    }

    virtual void add_strategy(VarTYPE* output, int output_size, const void* sourceBuffer) {
        cx_handle h = this->handle_.get();
        const void* d_in = stage_message(sourceBuffer);
        cxx::Staged<VarTYPE> o(h, this->stage_a_, output, (size_t)output_size, true, true);
        // the kernel reads the header itself: a message made for a longer vector touches nothing and
        // is reported by the one wait below (the reference throws before it touches the output)
        // (any index order, as the reference takes: the call looks at the indices first)
        int rc = cx_ip_add(h, cxx::dtype_of<VarTYPE>::value, o.get(), output_size, d_in, CX_ADD_ANY_ORDER);
        if (rc == CX_OK) rc = Compressor<VarTYPE>::receive_status(h);
        if (rc == CX_ERR_MSG_TOO_LARGE)
            throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        cxx::check(rc);
        o.flush();
    }

public:
    // one rank-ordered pass over `output` for all the messages: each element is read and written
    // once, the additions to it happen in the order of the messages, exactly as with one add() per
    // message.  The kernels check every header first: a message made for a longer vector leaves
    // `output` untouched.
    virtual void add_many(VarTYPE* output, int output_size, const void* const* d_sources, int count) {
        if (count <= 0) return;
        cxx::Scope scope(this->handle_.ctx());
        cx_handle h = this->handle_.get();
        cxx::Staged<VarTYPE> o(h, this->stage_a_, output, (size_t)output_size, true, true);
        cxx::check(cx_ip_reduce(h, cxx::dtype_of<VarTYPE>::value, o.get(), output_size, d_sources, count, 1,
                                CX_REDUCE_ANY_ORDER));
        const int rc = Compressor<VarTYPE>::receive_status(h);
        if (rc == CX_ERR_MSG_TOO_LARGE)
            throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        cxx::check(rc);
        o.flush();
    }
};

// ---------------------------------------------------------------------------------------
// Run-length codec (reference src/compressor.hxx:158-532): int32 n, int32 c, c values, int32 runs,
// int32 signum, run lengths; an element is sent when |x| >= threshold.  The sent values are
// stored densely, as the reference's decoder expects (its encoder indexes them by vector
// position, :238,277,316, and only decodes when every element is sent).  decompress returns the
// vector length the message carries, as the reference's does (:469), not a byte count.
template <class VarTYPE>
class CompressorRLE : public Compressor<VarTYPE> {
public:
    CompressorRLE() {}
    CompressorRLE(const CompressorRLE<VarTYPE>& other) : Compressor<VarTYPE>(other) {}
    virtual Compressor<VarTYPE>* clone() const { return new CompressorRLE<VarTYPE>(*this); }

    // n values, n + 1 run lengths at most
    virtual long long max_message_bytes(int n) const { return 16 + (long long)n * (long long)sizeof(VarTYPE) + 4ll * ((long long)n + 1); }

protected:
    virtual unsigned reserve_paths() const { return CX_RESERVE_RLE | CX_RESERVE_REDUCE; }
public:

    virtual int compress_device(void* d_target, long long capacity, const VarTYPE* d_data, VarTYPE* d_update, int n,
                                const VarTYPE* d_threshold, VarTYPE threshold, int* d_size_prefix, bool wait) {
        if (!d_data && !d_update) throw std::runtime_error("Compression needs a valid input vector!");
        int bytes = -1;
        cxx::check(cx_rle_compress(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_target, capacity, d_data,
                                   d_update, n, d_threshold ? nullptr : &threshold, d_threshold, d_size_prefix,
                                   wait ? &bytes : nullptr));
        return bytes;
    }
    virtual int decompress_device(VarTYPE* d_output, int output_size, const void* d_source, bool) {
        int n = 0;
        const int rc = cx_rle_decompress(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_output, output_size,
                                         d_source, &n);
        if (rc == CX_ERR_MSG_TOO_LARGE) throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        cxx::check(rc);
        return n;
    }
    virtual void add_device(VarTYPE* d_output, int output_size, const void* d_source) {
        const int rc = cx_rle_add(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, d_output, output_size, d_source);
        if (rc == CX_ERR_MSG_TOO_LARGE) throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        cxx::check(rc);
    }

protected:
    virtual int compression_strategy(void* output, const VarTYPE* data_vector, VarTYPE* update_vector,
                                     const int vector_size, VarTYPE threshold) {
        cx_handle h = this->handle_.get();
        const long long cap = max_message_bytes(vector_size);
        cxx::Staged<const VarTYPE> d(h, this->stage_a_, data_vector, (size_t)(data_vector ? vector_size : 0), true, false);
        cxx::Staged<VarTYPE> u(h, this->stage_b_, update_vector, (size_t)(update_vector ? vector_size : 0), true, true);
        const bool host_out = !cx_pointer_on_device(output);
        void* d_out = host_out ? this->stage_msg_.reserve((size_t)cap) : output;
        const int bytes = compress_device(d_out, cap, data_vector ? d.get() : nullptr,
                                          update_vector ? u.get() : nullptr, vector_size, nullptr, threshold, nullptr,
                                          true);
        if (host_out) cxx::check(cx_copy(h, output, d_out, (size_t)bytes));
        u.flush();
        cxx::check(cx_synchronize(h));
        return bytes;
    }

    // a host-resident message is staged whole: its length follows from c and, behind the values, runs
    const void* stage_message(const void* msg) {
        if (cx_pointer_on_device(msg)) return msg;
        const char* p = static_cast<const char*>(msg);
        int c = 0, runs = 0;
        std::memcpy(&c, p + 4, 4);
        if (c < 0) c = 0;
        std::memcpy(&runs, p + 8 + (size_t)c * sizeof(VarTYPE), 4);
        if (runs < 0) runs = 0;
        const size_t bytes = 16 + (size_t)c * sizeof(VarTYPE) + 4 * (size_t)runs;
        void* d = this->stage_msg_.reserve(bytes);
        cxx::check(cx_copy(this->handle_.get(), d, msg, bytes));
        return d;
    }

    virtual int decompression_strategy(VarTYPE* output, int output_size, const void* input) {
        cx_handle h = this->handle_.get();
        const void* d_in = stage_message(input);
        // only the message's n elements are written: a host vector is staged in and out
        cxx::Staged<VarTYPE> o(h, this->stage_a_, output, (size_t)output_size, true, true);
        const int n = decompress_device(o.get(), output_size, d_in, true);
        o.flush();
        cxx::check(cx_synchronize(h));
        return n;
    }
    virtual void add_strategy(VarTYPE* output, int output_size, const void* sourceBuffer) {
        cx_handle h = this->handle_.get();
        const void* d_in = stage_message(sourceBuffer);
        cxx::Staged<VarTYPE> o(h, this->stage_a_, output, (size_t)output_size, true, true);
        add_device(o.get(), output_size, d_in);
        o.flush();
        cxx::check(cx_synchronize(h));
    }
};

// ---------------------------------------------------------------------------------------
// Dense "compression": the whole vector behind an int32 length.  Composed from the library's
// streaming primitives; not a hot path.
template <class VarTYPE>
class CompressorNone : public Compressor<VarTYPE> {
public:
    CompressorNone() {}
    CompressorNone(const CompressorNone<VarTYPE>& other) : Compressor<VarTYPE>(other) {}
    virtual Compressor<VarTYPE>* clone() const { return new CompressorNone<VarTYPE>(*this); }
    virtual long long max_message_bytes(int n) const { return 4 + (long long)n * (long long)sizeof(VarTYPE); }
    virtual void reserve(int, bool) {}  // copies and adds only: no scratch

    virtual int compress_device(void* d_target, long long capacity, const VarTYPE* d_data, VarTYPE* d_update, int n,
                                const VarTYPE*, VarTYPE, int* d_size_prefix, bool) {
        if (!d_data && !d_update) throw std::runtime_error("Compression needs a valid input vector!");
        cx_handle h = this->handle_.get();
        const long long bytes = 4 + (long long)n * (long long)sizeof(VarTYPE);
        if (bytes > capacity) throw std::runtime_error("compressed message does not fit the buffer it was given");
        const cx_dtype dt = cxx::dtype_of<VarTYPE>::value;
        char* out = static_cast<char*>(d_target);
        const int n32 = n;
        cxx::check(cx_copy(h, out, &n32, 4));
        if (d_data && d_update) {
            cxx::check(cx_add_vec(h, dt, d_update, d_data, n));  // update + data, one add per element
            cxx::check(cx_copy(h, out + 4, d_update, (size_t)n * sizeof(VarTYPE)));
            cxx::check(cx_zero(h, dt, d_update, n));
        } else if (d_update) {
            cxx::check(cx_copy(h, out + 4, d_update, (size_t)n * sizeof(VarTYPE)));
            cxx::check(cx_zero(h, dt, d_update, n));
        } else {
            cxx::check(cx_copy(h, out + 4, d_data, (size_t)n * sizeof(VarTYPE)));
        }
        if (d_size_prefix) {
            const int b32 = (int)bytes;
            cxx::check(cx_copy(h, d_size_prefix, &b32, 4));
        }
        return (int)bytes;
    }
    virtual int decompress_device(VarTYPE* d_output, int output_size, const void* d_source, bool) {
        cx_handle h = this->handle_.get();
        int r_size = 0;
        cxx::check(cx_copy(h, &r_size, d_source, 4));
        cxx::check(cx_synchronize(h));
        if (r_size > output_size) throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        cxx::check(cx_copy(h, d_output, static_cast<const char*>(d_source) + 4, (size_t)r_size * sizeof(VarTYPE)));
        return 4 + r_size * (int)sizeof(VarTYPE);
    }
    virtual void add_device(VarTYPE* d_output, int output_size, const void* d_source) {
        cx_handle h = this->handle_.get();
        int r_size = 0;
        cxx::check(cx_copy(h, &r_size, d_source, 4));
        cxx::check(cx_synchronize(h));
        if (r_size > output_size) throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        // the reference adds output_size elements whatever the message holds (src/compressor.hxx:146-148);
        // only the r_size elements the message really has are added here
        cxx::check(cx_add_vec(h, cxx::dtype_of<VarTYPE>::value, d_output,
                              reinterpret_cast<const VarTYPE*>(static_cast<const char*>(d_source) + 4), r_size));
    }

protected:
    virtual int compression_strategy(void* output, const VarTYPE* data_vector, VarTYPE* update_vector,
                                     const int vector_size, VarTYPE threshold) {
        cx_handle h = this->handle_.get();
        const long long cap = 4 + (long long)vector_size * (long long)sizeof(VarTYPE);
        cxx::Staged<const VarTYPE> d(h, this->stage_a_, data_vector, (size_t)(data_vector ? vector_size : 0), true, false);
        cxx::Staged<VarTYPE> u(h, this->stage_b_, update_vector, (size_t)(update_vector ? vector_size : 0), true, true);
        const bool host_out = !cx_pointer_on_device(output);
        void* d_out = host_out ? this->stage_msg_.reserve((size_t)cap) : output;
        const int bytes = compress_device(d_out, cap, data_vector ? d.get() : nullptr,
                                          update_vector ? u.get() : nullptr, vector_size, nullptr, threshold, nullptr,
                                          true);
        if (host_out) cxx::check(cx_copy(h, output, d_out, (size_t)bytes));
        u.flush();
        cxx::check(cx_synchronize(h));
        return bytes;
    }
    virtual int decompression_strategy(VarTYPE* output, int output_size, const void* input) {
        cx_handle h = this->handle_.get();
        int r_size = 0;
        cxx::check(cx_copy(h, &r_size, input, 4));
        cxx::check(cx_synchronize(h));
        if (r_size > output_size) throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        cxx::check(cx_copy(h, output, static_cast<const char*>(input) + 4, (size_t)r_size * sizeof(VarTYPE)));
        cxx::check(cx_synchronize(h));
        return 4 + r_size * (int)sizeof(VarTYPE);
    }
    virtual void add_strategy(VarTYPE* output, int output_size, const void* sourceBuffer) {
        cx_handle h = this->handle_.get();
        int r_size = 0;
        cxx::check(cx_copy(h, &r_size, sourceBuffer, 4));
        cxx::check(cx_synchronize(h));
        if (r_size > output_size) throw std::runtime_error("Decompression vector size is bigger than output buffer!");
        const size_t bytes = 4 + (size_t)r_size * sizeof(VarTYPE);
        const void* d_in = sourceBuffer;
        if (!cx_pointer_on_device(sourceBuffer)) {
            void* d = this->stage_msg_.reserve(bytes);
            cxx::check(cx_copy(h, d, sourceBuffer, bytes));
            d_in = d;
        }
        cxx::Staged<VarTYPE> o(h, this->stage_a_, output, (size_t)output_size, true, true);
        add_device(o.get(), output_size, d_in);
        o.flush();
        cxx::check(cx_synchronize(h));
    }
};

#endif  // COMPRESSOR_H
