// ComprEx<T>: one directed, compressed point-to-point channel with an error-feedback
// residual, with the public interface of the reference's include/comprEx.hxx:69-166 and the
// behaviour of src/comprEx.tpp:30-363.  FastComprEx<T> (one-step-stale, double-buffered
// variant, include/comprEx.hxx:173-227, src/comprEx.tpp:366-514) follows below.
//
// What is different from the reference:
//   * the residual ("rests") lives in device memory, and so do the send/receive buffers;
//   * the GaspiCxx Source/TargetBuffer pair is replaced by one device buffer per directed
//     (source, target, tag) triple, owned by the GaspiEnvironment stand-in: the sender's
//     compressor writes the message where the receiver reads it.  Every object works on a HIP
//     stream of its own (shared with its compressor and threshold clones); a message's
//     hand-over is an event the sender's stream records and the receiver's stream waits for,
//     and every call joins the object's stream with the caller's (GaspiEnvironment::
//     set_user_stream, default the null stream) on entry and on exit;
//   * `vector` arguments may be host pointers (staged) or device pointers (used in place);
//   * with one thread playing all ranks a receive with no message pending throws instead of
//     blocking for ever; with one thread per rank (GaspiEnvironment::set_blocking) it waits;
//   * writeRemote only enqueues GPU work; nothing is copied to the host.
#ifndef COMPREX_H
#define COMPREX_H

#include <cstdio>
#include <memory>
#include <stdexcept>
#include <vector>

#include "compressor.hxx"
#include "gaspiEnvironment.hxx"
#include "threshold.hxx"

template <class VarTYPE>
class ComprEx {
protected:
    std::unique_ptr<Compressor<VarTYPE> > compressor;
    std::unique_ptr<ThresholdFunction<VarTYPE> > threshold;

    GaspiEnvironment* gaspiCxx_segment;

    // "rests": the error of compression accumulated locally, rests_size elements on the device
    cxx::DeviceBuffer restsVect;
    int rests_size;
    std::vector<VarTYPE> rests_mirror;  // host copy handed out by getRests_p()

    std::shared_ptr<cxx::Channel> srcBuff_data;   // messages this object sends
    std::shared_ptr<cxx::Channel> targBuff_data;  // messages this object receives

    int srcRank, targRank;
    int size;              // uncompressed vector length in elements
    long long bufferSize;  // bytes of the send/receive buffers
    float size_factor;
    bool send_sizeBytes;

    cxx::Handle handle_;
    cxx::DeviceBuffer stage_;
    cxx::DeviceBuffer forward_;  // message in transit between inbox and outbox (forward_buffer)
    cxx::StreamOrder cross_;     // for the calls that touch another object's buffers

    VarTYPE* rests() const { return static_cast<VarTYPE*>(restsVect.data()); }
    char* src_address() const { return static_cast<char*>(srcBuff_data->buffer.data()); }
    char* targ_address() const { return static_cast<char*>(targBuff_data->buffer.data()); }

    // this object's stream (its compressor and threshold clones work on it too)
    void* stream() { return handle_.ctx().stream(); }
    // joins the object's stream with the caller's for the time of a call
    cxx::StreamCtx& joined() {
        handle_.ctx().set_origin(gaspiCxx_segment ? gaspiCxx_segment->user_stream() : nullptr);
        return handle_.ctx();
    }
    void bind_clones() {
        compressor->bind_stream(handle_.ctx_ptr());
        threshold->bind_stream(handle_.ctx_ptr());
    }

    void alloc_rests() {
        restsVect.reserve((size_t)size * sizeof(VarTYPE));
        rests_size = size;
        resetRests();
    }

    // "waitForCompletion" of the reference's TargetBuffer
    void wait_for_message() {
        targBuff_data->wait_message(gaspiCxx_segment->blocking(), gaspiCxx_segment->timeout_s(), stream());
    }
    // the source buffer may be overwritten once the receiver has read the previous message
    void wait_for_room() {
        srcBuff_data->wait_consumed(gaspiCxx_segment->blocking(), gaspiCxx_segment->timeout_s(), stream());
    }

    // send-side tail shared by all write paths: data-only / update-only / fused compression
    // of `n` elements into the source buffer at byte offset `at`
    void compress_into(long long at, const VarTYPE* d_data, VarTYPE* d_update, int n, bool use_threshold) {
        const int offset = send_sizeBytes ? (int)sizeof(int) : 0;
        const VarTYPE* d_thr = use_threshold ? threshold->device_threshold() : nullptr;
        const VarTYPE thr = use_threshold && !d_thr ? threshold->get_threshold() : (VarTYPE)0;
        compressor->compress_device(src_address() + at + offset, bufferSize - at - offset, d_data, d_update, n, d_thr,
                                    thr, send_sizeBytes ? reinterpret_cast<int*>(src_address() + at) : nullptr, false);
    }

    // Sends of the whole residual.  Messages that earlier sends had to cut short for lack of room
    // are not an error (what they could not hold stayed in the residual and leaves now); other
    // errors recorded by the compressor's kernels are.
    void forgive_short_messages() {
        const int st = compressor->device_status();
        if (st != CX_OK && st != CX_ERR_CAPACITY) cxx::check(st);
    }
    // After the flush's message has been handed over: a flush that did not fit its buffer has sent
    // what fitted, the rest is still in the residual, and the caller is told (the reference writes
    // past its buffer here).
    void report_flush(int st) {
        if (st == CX_ERR_CAPACITY)
            throw std::runtime_error("flushRests: the send buffer held only part of the residual, the rest stays in the "
                                     "residual: flush again or increase size_factor!");
        cxx::check(st);
    }

    // residual += d_data with the entries above the threshold compressed into the message at
    // `d_target`: one call when the threshold is a top-k rule and the compressor has a path for
    // it, else false (nothing done) and the caller takes the two steps.
    bool fused_topk_into(void* d_target, long long capacity, const VarTYPE* d_data, int n, int* d_size_prefix) {
        typename ThresholdFunction<VarTYPE>::TopKRule rule;
        if (n != rests_size || n <= 0 || !threshold->topk_rule(&rule)) return false;
        if (rule.topK > 1.0f || rule.topK < 0.0f) return false;  // let prepare_with report it
        // a claim without a fused call is harmless: the caller's prepare_with follows and overwrites it
        VarTYPE* slot = threshold->claim_device_threshold();
        if (!slot) return false;
        return compressor->write_step_device(d_target, capacity, d_data, rests(), n, rule, slot, d_size_prefix);
    }

public:
    ComprEx()
        : compressor(new CompressorNone<VarTYPE>()), threshold(new ThresholdNone<VarTYPE>()), gaspiCxx_segment(NULL),
          rests_size(0), srcRank(-1), targRank(-1), size(0), bufferSize(0), size_factor(0), send_sizeBytes(false) {
        bind_clones();
    }

    ComprEx(GaspiEnvironment* segment, int size, float size_factor = 1.0, bool send_sizeBytes = false)
        : compressor(new CompressorNone<VarTYPE>()), threshold(new ThresholdNone<VarTYPE>()),
          gaspiCxx_segment(segment), rests_size(0), srcRank(-1), targRank(-1), size(size), size_factor(size_factor),
          send_sizeBytes(send_sizeBytes) {
        // the reference evaluates size*sizeof(T)*size_factor in fp32 and truncates to int; 64 bits here
        bufferSize = (long long)((float)((size_t)size * sizeof(VarTYPE)) * size_factor);
        bind_clones();
    }

    virtual ~ComprEx() {}

    ComprEx(const ComprEx<VarTYPE>& other) : ComprEx() { *this = other; }

    ComprEx<VarTYPE>& operator=(const ComprEx<VarTYPE>& other) {
        if (srcBuff_data || targBuff_data)
            throw std::runtime_error("ComprEx object with established connection cannot be assigned to other object!");
        gaspiCxx_segment = other.gaspiCxx_segment;
        compressor.reset(other.compressor->clone());
        threshold.reset(other.threshold->clone());
        bind_clones();
        size = other.size;
        bufferSize = other.bufferSize;
        size_factor = other.size_factor;
        send_sizeBytes = other.send_sizeBytes;
        if (other.rests_size > 0) {  // same length as the other's residual, all zero
            restsVect.reserve((size_t)other.rests_size * sizeof(VarTYPE));
            rests_size = other.rests_size;
            resetRests();
        } else {
            rests_size = 0;
        }
        reserve_scratch();  // the clones' scratch too: the exchange calls never allocate
        return *this;
    }

    // Not in the reference: run this object's GPU work (its clones' included) on a stream of the
    // caller's instead of its own (NULL = the null stream).  Waits for what the old stream holds.
    void set_stream(void* hip_stream) {
        handle_.ctx().adopt(hip_stream);
        handle_.refresh();
        compressor->stream_changed();
        threshold->stream_changed();
    }
    void* get_stream() { return stream(); }

    void setCompressor(const Compressor<VarTYPE>& c) { setCompressor(&c); }
    void setCompressor(const Compressor<VarTYPE>* c) {
        this->compressor.reset(c->clone());
        bind_clones();
        reserve_scratch();
    }
    void setThreshold(const ThresholdFunction<VarTYPE>& t) { setThreshold(&t); }
    void setThreshold(const ThresholdFunction<VarTYPE>* t) {
        this->threshold.reset(t->clone());
        bind_clones();
        reserve_scratch();
    }

    // The GPU scratch of the clones this object owns, sized for this object's vectors when the
    // clones are made: the exchange calls then never allocate.  Without a GPU (objects built only to
    // be configured) nothing is reserved.
    void reserve_scratch() {
        if (size <= 0 || cx_device_count() < 1) return;
        threshold->reserve(size);
        compressor->reserve(size, threshold->whole_vector_topk(size, nullptr));
    }

    void print_rests() {
        std::vector<VarTYPE> r = getRests();
        for (size_t it = 0; it < r.size(); ++it) printf("Rests[%d]: %g\n", (int)it, (double)r[it]);
    }

    virtual void resetRests() {
        if (rests_size > 0)
            cxx::check(cx_zero(handle_.get(), cxx::dtype_of<VarTYPE>::value, rests(), rests_size));  // (own memory, own stream)
    }

    // Sends the whole residual (no thresholding: every non-zero element) and clears it.
    virtual void flushRests() {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        forgive_short_messages();
        wait_for_room();
        // as an update: what is sent leaves the residual, what found no room stays (the reference
        // compresses the residual as data and clears it afterwards: the same message and residual)
        compress_into(0, nullptr, rests(), rests_size, false);
        const int st = compressor->device_status();
        srcBuff_data->post(stream());
        report_flush(st);
        resetRests();
    }

    std::vector<VarTYPE> getRests() const {
        std::vector<VarTYPE> out((size_t)rests_size);
        if (rests_size > 0) {
            cx_handle h = const_cast<ComprEx<VarTYPE>*>(this)->handle_.get();
            cxx::check(cx_copy(h, out.data(), rests(), out.size() * sizeof(VarTYPE)));
            cxx::check(cx_synchronize(h));
        }
        return out;
    }

    void getRests(VarTYPE* data, int size) const {
        if (size != rests_size) {
            char error_msg[100];
            snprintf(error_msg, sizeof error_msg, "Vector of size %d does not match Rests Vector of size %d!\n", size,
                     rests_size);
            throw std::runtime_error(error_msg);
        }
        cxx::Scope scope(const_cast<ComprEx<VarTYPE>*>(this)->joined());
        cx_handle h = const_cast<ComprEx<VarTYPE>*>(this)->handle_.get();
        cxx::check(cx_copy(h, data, rests(), (size_t)size * sizeof(VarTYPE)));
        cxx::check(cx_synchronize(h));
    }

    void addRests(VarTYPE* data, int size) const {
        if (size != rests_size) {
            char error_msg[100];
            snprintf(error_msg, sizeof error_msg, "Vector of size %d does not match Rests Vector of size %d!\n", size,
                     rests_size);
            throw std::runtime_error(error_msg);
        }
        ComprEx<VarTYPE>* self = const_cast<ComprEx<VarTYPE>*>(this);
        cxx::Scope scope(self->joined());
        cx_handle h = self->handle_.get();
        cxx::Staged<VarTYPE> d(h, self->stage_, data, (size_t)size, true, true);
        cxx::check(cx_add_vec(h, cxx::dtype_of<VarTYPE>::value, d.get(), rests(), size));
        d.flush();
        cxx::check(cx_synchronize(h));
    }

    // Host copy of the residual, refreshed by this call (the reference returns a pointer to its
    // own std::vector; the residual is device memory here).
    const std::vector<VarTYPE>* getRests_p() {
        rests_mirror = getRests();
        return &rests_mirror;
    }
    // Device address of the residual (rests_size elements).
    const VarTYPE* getRests_device() const { return rests(); }

    // residual += vector; entries above the threshold are sent and cleared
    virtual void writeRemote(const VarTYPE* vector, int size) {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        cxx::Scope scope(joined());
        cx_handle h = handle_.get();
        cxx::Staged<const VarTYPE> v(h, stage_, vector, (size_t)size, true, false);
        typename ThresholdFunction<VarTYPE>::TopKRule rule;
        if (size == rests_size && size > 0 && threshold->topk_rule(&rule)) {
            wait_for_room();
            const int offset = send_sizeBytes ? (int)sizeof(int) : 0;
            if (fused_topk_into(src_address() + offset, bufferSize - offset, v.get(), size,
                                send_sizeBytes ? reinterpret_cast<int*>(src_address()) : nullptr)) {
                srcBuff_data->post(stream());
                return;
            }
        }
        threshold->prepare_with(rests(), rests_size, v.get(), size);
        if (size != rests_size) {
            char msg[100];
            snprintf(msg, sizeof msg, "Compressor: Update vector size (%d) is not equal data vector size (%d)!",
                     rests_size, size);
            throw std::runtime_error(msg);
        }
        wait_for_room();
        compress_into(0, v.get(), rests(), rests_size, true);
        srcBuff_data->post(stream());
    }

    // compression only: no threshold, residual untouched
    virtual void writeRemote_compressOnly(const VarTYPE* vector, int size) {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        cxx::Scope scope(joined());
        cx_handle h = handle_.get();
        cxx::Staged<const VarTYPE> v(h, stage_, vector, (size_t)size, true, false);
        wait_for_room();
        compress_into(0, v.get(), nullptr, size, false);
        srcBuff_data->post(stream());
    }

    // threshold from the vector alone, residual untouched
    void writeRemote_NoResidual(const VarTYPE* vector, int size) {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        cxx::Scope scope(joined());
        cx_handle h = handle_.get();
        cxx::Staged<const VarTYPE> v(h, stage_, vector, (size_t)size, true, false);
        threshold->prepare(v.get(), size);
        wait_for_room();
        compress_into(0, v.get(), nullptr, size, true);
        srcBuff_data->post(stream());
    }

    // overwrites `vector` with the received message
    virtual void readRemote(VarTYPE* vector, int size) {
        if (!targBuff_data) throw std::runtime_error("Receive issued without connecting to Remote!");
        cxx::Scope scope(joined());
        wait_for_message();
        Release release(this);  // the channel is freed whatever the decoder reports
        const int offset = send_sizeBytes ? (int)sizeof(int) : 0;
        compressor->decompress(vector, size, targ_address() + offset);
    }

    // adds the received message to `vector`
    virtual void readRemote_add(VarTYPE* vector, int size) {
        if (!targBuff_data) throw std::runtime_error("Receive issued without connecting to Remote!");
        cxx::Scope scope(joined());
        wait_for_message();
        Release release(this);
        const int offset = send_sizeBytes ? (int)sizeof(int) : 0;
        compressor->add(vector, size, targ_address() + offset);
    }

protected:
    // marks the pending message consumed when the receive leaves, also by an exception
    struct Release {
        ComprEx* c;
        explicit Release(ComprEx* c) : c(c) {}
        ~Release() {
            try {
                c->targBuff_data->consumed(c->stream());
            } catch (...) {
            }
        }
    };

public:
    // Not in the reference: a receiver that takes the messages of several channels in one call (the
    // chief of the all-to-one schedule) waits for each, collects their device addresses, adds them all
    // with add_messages() of one of the objects, and releases the channels with message_done().
    // `reader`: the object whose add_messages() will read the message (its stream waits for it)
    const void* waiting_message(ComprEx<VarTYPE>* reader = nullptr) {
        if (!targBuff_data) throw std::runtime_error("Receive issued without connecting to Remote!");
        targBuff_data->wait_message(gaspiCxx_segment->blocking(), gaspiCxx_segment->timeout_s(),
                                    (reader ? reader : this)->stream());
        return targ_address() + (send_sizeBytes ? (int)sizeof(int) : 0);
    }
    void message_done(ComprEx<VarTYPE>* reader = nullptr) { targBuff_data->consumed((reader ? reader : this)->stream()); }
    void add_messages(VarTYPE* vector, int size, const void* const* messages, int count) {
        cxx::Scope scope(joined());
        compressor->add_many(vector, size, messages, count);
    }

    // receive, pass the compressed message on to this object's target, and decompress it
    void readRemote_forward(VarTYPE* vector, int size) {
        cxx::Scope scope(joined());
        wait_for_message();
        wait_for_room();
        cx_handle h = handle_.get();
        if (send_sizeBytes) {
            int sizeBytes = 0;
            cxx::check(cx_copy(h, &sizeBytes, targ_address(), sizeof(int)));
            cxx::check(cx_copy(h, src_address(), targ_address(), (size_t)sizeBytes + sizeof(int)));
            srcBuff_data->post(stream());
            compressor->decompress(vector, size, targ_address() + sizeof(int));
        } else {
            const int sizeBytes = compressor->decompress(vector, size, targ_address());
            cxx::check(cx_copy(h, src_address(), targ_address(), (size_t)sizeBytes));
            srcBuff_data->post(stream());
        }
        targBuff_data->consumed(stream());
    }

    void readRemote_forwardCopy(VarTYPE* vector, int size) {
        if (!this->send_sizeBytes)
            throw std::runtime_error("If using readRemote_forwardCopy, send_sizeBytes must be true!");
        wait_for_message();
        wait_for_room();
        cx_handle h = handle_.get();
        int sizeBytes = 0;
        cxx::check(cx_copy(h, &sizeBytes, targ_address(), sizeof(int)));
        cxx::check(cx_copy(h, src_address(), targ_address(), (size_t)sizeBytes + sizeof(int)));
        targBuff_data->consumed(stream());
    }

    void readRemote_wait() { wait_for_message(); }

    // copies the received message into the send buffer (it is sent by forward_add).  The copy
    // goes through a private buffer: the inbox is released before this object waits for room in
    // its outbox, so a ring of ranks that all forward at once cannot wait on each other in a circle
    // (the reference has separate source and target buffers and feedback tokens for this).
    void forward_buffer() {
        if (!this->send_sizeBytes) throw std::runtime_error("If using forward_buffer, send_sizeBytes must be true!");
        cx_handle h = handle_.get();
        int sizeBytes = 0;
        cxx::check(cx_copy(h, &sizeBytes, targ_address(), sizeof(int)));
        const size_t bytes = (size_t)sizeBytes + sizeof(int);
        void* hold = forward_.reserve(bytes);
        cxx::check(cx_copy(h, hold, targ_address(), bytes));
        targBuff_data->consumed(stream());
        wait_for_room();
        cxx::check(cx_copy(h, src_address(), hold, bytes));
    }

    // sends the message sitting in the send buffer and adds it to `vector`
    void forward_add(VarTYPE* vector, int size) {
        if (!this->send_sizeBytes) throw std::runtime_error("If using forward_add, send_sizeBytes must be true!");
        cxx::Scope scope(joined());
        compressor->add(vector, size, src_address() + sizeof(int));
        srcBuff_data->post(stream());
    }

    virtual void connectTx(int targRank, int tag) {
        this->targRank = targRank;
        alloc_rests();  // the residual exists only on objects that send
        srcBuff_data = gaspiCxx_segment->channel(gaspiCxx_segment->get_rank(), targRank, tag, bufferSize);
    }

    virtual void connectRx(int srcRank, int tag) {
        this->srcRank = srcRank;
        targBuff_data = gaspiCxx_segment->channel(srcRank, gaspiCxx_segment->get_rank(), tag, bufferSize);
    }

    // srcRank: receive data from this rank; targRank: send data to this rank
    virtual void connectTo(int srcRank, int targRank, int tag) {
        connectTx(targRank, tag);
        connectRx(srcRank, tag);
    }
};

// ---------------------------------------------------------------------------------------
// FastComprEx: the message compressed by one writeRemote is sent by the NEXT one (the
// reference overlaps the RDMA put of message i-1 with the compression of message i); the
// source buffer is split in two halves used alternately.
template <class VarTYPE>
class FastComprEx : public ComprEx<VarTYPE> {
protected:
    int doublebuffer_phase;
    long long doublebuffer_offset;  // bytes between the two halves
    bool is_first;
    // the half that holds the message of the previous call is what the receiver sees: it is
    // copied to the front of the channel when it is "sent"
    cxx::DeviceBuffer halves_;
    // sizeBytes of the reference, one per half, kept on the device: every compressor writes its
    // message's byte count there (int32), and sending copies exactly that many bytes without the
    // host reading it
    cxx::DeviceBuffer half_bytes_;

    using ComprEx<VarTYPE>::restsVect;
    using ComprEx<VarTYPE>::srcBuff_data;

public:
    using ComprEx<VarTYPE>::writeRemote_compressOnly;  // the const overload stays visible

protected:

    long long send_offset() const { return doublebuffer_offset * ((doublebuffer_phase + 1) % 2); }
    long long write_offset() const { return doublebuffer_offset * doublebuffer_phase; }
    void update_doublebuffer_phase() { doublebuffer_phase = (doublebuffer_phase + 1) % 2; }
    char* half(long long off) const { return static_cast<char*>(halves_.data()) + off; }
    int* half_bytes(long long off) const { return static_cast<int*>(half_bytes_.data()) + (off == 0 ? 0 : 1); }

    void ensure_halves() {
        if (!halves_.data()) halves_.reserve((size_t)(2 * doublebuffer_offset > 32 ? 2 * doublebuffer_offset : 32));
        if (!half_bytes_.data()) {
            half_bytes_.reserve(2 * sizeof(int));
            cxx::check(cx_zero(this->handle_.get(), CX_I32, half_bytes_.data(), 2));
        }
    }

    // "initTransferPart(sizeBytes, send_offset)": hand the half at `off` to the receiver
    void send_half(long long off) {
        cx_handle h = this->handle_.get();
        this->wait_for_room();
        const long long room = doublebuffer_offset < this->bufferSize ? doublebuffer_offset : this->bufferSize;
        cxx::check(cx_copy_counted(h, this->src_address(), half(off), half_bytes(off), room));
        srcBuff_data->post(this->stream());
    }

    void compress_half(long long off, const VarTYPE* d_data, VarTYPE* d_update, int n, bool use_threshold) {
        const VarTYPE* d_thr = use_threshold ? this->threshold->device_threshold() : nullptr;
        const VarTYPE thr = use_threshold && !d_thr ? this->threshold->get_threshold() : (VarTYPE)0;
        this->compressor->compress_device(half(off), doublebuffer_offset, d_data, d_update, n, d_thr, thr,
                                          half_bytes(off), false);
    }

public:
    FastComprEx() : ComprEx<VarTYPE>(), doublebuffer_phase(0), doublebuffer_offset(0), is_first(true) {}

    FastComprEx(GaspiEnvironment* segment, int size, float size_factor = 1.0)
        : ComprEx<VarTYPE>(segment, size, size_factor * 2), doublebuffer_phase(0), is_first(true) {
        // (int)(size * size_factor * sizeof(T)) in the reference; cut to a multiple of four bytes so that
        // the second half starts where a message may start
        doublebuffer_offset = (long long)((float)size * size_factor * (float)sizeof(VarTYPE)) & ~3ll;
    }

    FastComprEx(const FastComprEx<VarTYPE>& other) : ComprEx<VarTYPE>() { *this = other; }

    FastComprEx<VarTYPE>& operator=(const FastComprEx<VarTYPE>& other) {
        ComprEx<VarTYPE>::operator=(other);
        doublebuffer_offset = other.doublebuffer_offset;
        doublebuffer_phase = 0;
        is_first = true;
        return *this;
    }

    // the halves are taken when the object connects: the exchange calls never allocate
    virtual void connectTx(int targRank, int tag) {
        ComprEx<VarTYPE>::connectTx(targRank, tag);
        ensure_halves();
    }

    virtual void flushRests() {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        ensure_halves();
        this->forgive_short_messages();
        const long long so = send_offset();
        // the message that was compressed but never sent goes back into the residual (when nothing
        // waits, the reference adds whatever its buffer holds: fresh memory, or the previous flush's
        // message a second time; nothing is added here) ...
        if (!is_first) this->compressor->add_device(this->rests(), this->rests_size, half(so));
        // ... and the whole residual is sent
        compress_half(so, nullptr, this->rests(), this->rests_size, false);
        const int st = this->compressor->device_status();
        send_half(so);
        is_first = true;
        this->report_flush(st);
        ComprEx<VarTYPE>::resetRests();
    }

    virtual void resetRests() {
        ComprEx<VarTYPE>::resetRests();
        is_first = true;
    }

    virtual void writeRemote(const VarTYPE* vector, int size) {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        ensure_halves();
        cxx::Scope scope(this->joined());
        cx_handle h = this->handle_.get();
        const long long wo = write_offset(), so = send_offset();
        if (is_first) {
            // the residual is all zero at this point, so this is an (almost) empty message
            compress_half(so, nullptr, this->rests(), this->rests_size, true);
            is_first = false;
        }
        send_half(so);  // the message of the previous call
        cxx::Staged<const VarTYPE> v(h, this->stage_, vector, (size_t)size, true, false);
        if (this->fused_topk_into(half(wo), doublebuffer_offset, v.get(), size, half_bytes(wo))) {
            update_doublebuffer_phase();
            return;
        }
        this->threshold->prepare_with(this->rests(), this->rests_size, v.get(), size);
        if (size != this->rests_size) {
            char msg[100];
            snprintf(msg, sizeof msg, "Compressor: Update vector size (%d) is not equal data vector size (%d)!",
                     this->rests_size, size);
            throw std::runtime_error(msg);
        }
        compress_half(wo, v.get(), this->rests(), this->rests_size, true);
        update_doublebuffer_phase();
    }

    virtual void writeRemote_compressOnly(VarTYPE* vector, int size) {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        ensure_halves();
        cxx::Scope scope(this->joined());
        cx_handle h = this->handle_.get();
        const long long wo = write_offset(), so = send_offset();
        if (is_first) {
            compress_half(so, this->rests(), nullptr, this->rests_size, false);
            is_first = false;
        }
        send_half(so);
        cxx::Staged<const VarTYPE> v(h, this->stage_, vector, (size_t)size, true, false);
        compress_half(wo, v.get(), nullptr, size, false);
        update_doublebuffer_phase();
    }

    // Sends what `other` compressed, without compressing again (the chief's broadcast to the
    // second and later workers, reference src/allreduce.tpp:209).
    virtual void writeRemote_sameAs(const FastComprEx* other) {
        if (!srcBuff_data) throw std::runtime_error("Send issued without connecting to Remote!");
        ensure_halves();
        const_cast<FastComprEx*>(other)->ensure_halves();
        cx_handle h = this->handle_.get();
        const long long wo = write_offset(), so = send_offset();
        if (is_first) {
            compress_half(so, nullptr, this->rests(), this->rests_size, true);
            is_first = false;
        }
        send_half(so);
        if (!other->is_first) {
            // memcpy(..., other->sizeBytes) and sizeBytes = other->sizeBytes, both on the device.  The
            // other object compressed on ITS stream: this one's waits for that, and the other's next
            // compress into the same half waits for this copy.
            FastComprEx* src = const_cast<FastComprEx*>(other);
            const long long oso = other->send_offset();
            if (other->doublebuffer_offset > doublebuffer_offset)
                throw std::runtime_error("writeRemote_sameAs: this object's buffer is smaller than the other's!");
            this->cross_.order(src->stream(), this->stream());
            cxx::check(cx_copy_counted(h, half(wo), other->half(oso), other->half_bytes(oso), doublebuffer_offset));
            cxx::check(cx_copy(h, half_bytes(wo), other->half_bytes(oso), sizeof(int)));
            this->cross_.order(this->stream(), src->stream());
        } else {
            this->is_first = true;
        }
        update_doublebuffer_phase();
    }

    virtual void connectTx_sameBufferAs(int targRank, int tag, const FastComprEx<VarTYPE>* other) {
        if (!other->srcBuff_data) throw std::runtime_error("Cannot connected with buffer of unconnected communicator!");
        this->connectTx(targRank, tag);
    }
};

#endif  // COMPREX_H
