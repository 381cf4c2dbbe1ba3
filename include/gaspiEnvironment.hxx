// Stand-in for the reference's GaspiEnvironment (include/gaspiEnvironment.hxx:9-28) on ONE
// GPU: several simulated ranks live in one process and exchange messages through device
// buffers.  There is no GASPI, no RDMA and no second GPU.
//
// A directed channel is identified by (source rank, target rank, tag), as the reference's
// SourceBuffer::connectToRemoteTarget / TargetBuffer::connectToRemoteSource pair is
// (src/comprEx.tpp:341-363).  The sender's compressor writes the message straight into the
// channel's device buffer and the receiver reads it from there: the "transfer" is an event the
// sender's stream records and the receiver's stream waits for.
//
// Two ways to drive the ranks:
//   * one thread plays all ranks in turn (set_rank before each rank's calls).  A receive with
//     nothing pending throws, because nobody else could ever send.
//   * one thread per rank, each running the reference's per-rank code unchanged
//     (set_blocking(true)): a receive waits for its message, a send waits until the previous
//     message of its channel was consumed.  Waits give up after a timeout with an exception.
// The rank is a per-thread setting.
#ifndef GASPI_ENVIRONMENT_HXX
#define GASPI_ENVIRONMENT_HXX

#include <chrono>
#include <condition_variable>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <tuple>

#include "cx_device.hxx"

namespace cxx {

struct Channel {
    DeviceBuffer buffer;   // message area
    long long capacity = 0;
    std::mutex m;
    std::condition_variable cv;
    long long sent = 0, received = 0;  // messages written / consumed
    // The hand-over on the GPU: the sender records `ready` on its stream behind the kernels that
    // write the message and the receiver's stream waits for it; the receiver records `freed` behind
    // the kernels that read it and the next send's stream waits for that (the reference's
    // notification and the write that waits for it, src/comprEx.tpp:190,231,243).  The counters
    // above only order the HOST side (who may enqueue what).
    void* ready = nullptr;
    void* freed = nullptr;
    bool ready_set = false, freed_set = false;

    ~Channel() {
        if (ready) cx_event_destroy(ready);
        if (freed) cx_event_destroy(freed);
    }

    // sender: called after the kernels that write the message were enqueued on `stream`
    void post(void* stream) {
        {
            std::lock_guard<std::mutex> g(m);
            if (!ready) check(cx_event_create(&ready));
            check(cx_event_record(ready, stream));
            ready_set = true;
            sent += 1;
        }
        cv.notify_all();
    }
    // sender: do not overwrite a message nobody has read yet.  Blocking mode waits (on the host)
    // until the receiver has enqueued its reads; either way `stream` then waits for those reads.
    void wait_consumed(bool blocking, double timeout_s, void* stream) {
        std::unique_lock<std::mutex> g(m);
        if (blocking && !cv.wait_for(g, std::chrono::duration<double>(timeout_s), [&] { return received >= sent; }))
            throw std::runtime_error("Send timed out: the previous message of this channel was never received!");
        if (freed_set) check(cx_stream_wait_event(stream, freed));
    }
    // receiver: the reference's TargetBuffer::waitForCompletion; `stream` is where the message will be read
    void wait_message(bool blocking, double timeout_s, void* stream) {
        std::unique_lock<std::mutex> g(m);
        if (!blocking) {
            if (received >= sent)
                throw std::runtime_error("Receive issued with no message pending (the reference would block here)!");
        } else if (!cv.wait_for(g, std::chrono::duration<double>(timeout_s), [&] { return sent > received; })) {
            throw std::runtime_error("Receive timed out: no message arrived!");
        }
        if (ready_set) check(cx_stream_wait_event(stream, ready));
    }
    // receiver: called after the kernels that read the message were enqueued on `stream`
    void consumed(void* stream) {
        {
            std::lock_guard<std::mutex> g(m);
            if (!freed) check(cx_event_create(&freed));
            check(cx_event_record(freed, stream));
            freed_set = true;
            received = sent;
        }
        cv.notify_all();
    }
};

}  // namespace cxx

class GaspiEnvironment {
public:
    // segment_size is what the reference reserves for GASPI; device buffers are allocated per
    // channel here, so it is only remembered.
    GaspiEnvironment(unsigned long segment_size)
        : segment_size_(segment_size), rank_(0), ranks_(1), blocking_(false), timeout_s_(60.0), barrier_count_(0),
          barrier_generation_(0) {}
    ~GaspiEnvironment() {}

    int get_rank() { return tls().env == this ? tls().rank : rank_; }
    int get_ranks() { return ranks_; }
    // Not in the reference (gaspi_run fixes both there): which simulated rank the calling thread
    // acts as from now on, and how many ranks there are.
    void set_rank(int rank, int ranks) {
        if (ranks < 1 || rank < 0 || rank >= ranks) throw std::runtime_error("set_rank: rank outside [0, ranks)");
        std::lock_guard<std::mutex> g(m_);
        rank_ = rank;
        ranks_ = ranks;
        tls().env = this;
        tls().rank = rank;
    }
    // true: receives wait for a message and sends wait for the previous one to be consumed
    // (one thread per rank); false (default): a receive with nothing pending throws.
    void set_blocking(bool blocking, double timeout_s = 60.0) {
        blocking_ = blocking;
        timeout_s_ = timeout_s;
    }
    bool blocking() const { return blocking_; }
    // Not in the reference: the HIP stream on which the calling thread's vectors are produced and
    // consumed (NULL, the default, = the null stream).  Every exchange call joins its object's own
    // stream with this one on entry and on exit, so the caller needs no synchronisation of its own.
    // A per-thread setting, like the rank: each simulated rank may work on a stream of its own.
    void set_user_stream(void* hip_stream) {
        tls().stream_env = this;
        tls().user_stream = hip_stream;
    }
    void* user_stream() { return tls().stream_env == this ? tls().user_stream : nullptr; }
    double timeout_s() const { return timeout_s_; }

    // all ranks' threads meet here (blocking mode); a no-op when one thread plays every rank
    void barrier() {
        if (!blocking_) return;
        std::unique_lock<std::mutex> g(m_);
        const long long gen = barrier_generation_;
        if (++barrier_count_ == ranks_) {
            barrier_count_ = 0;
            ++barrier_generation_;
            barrier_cv_.notify_all();
        } else if (!barrier_cv_.wait_for(g, std::chrono::duration<double>(timeout_s_),
                                         [&] { return barrier_generation_ != gen; })) {
            throw std::runtime_error("barrier timed out");
        }
    }
    void flush() {}
    // what the reference hands to ComprEx as `segment`
    GaspiEnvironment* get_segment() { return this; }
    unsigned long get_segment_size() const { return segment_size_; }

    std::shared_ptr<cxx::Channel> channel(int src_rank, int targ_rank, int tag, long long bytes) {
        std::lock_guard<std::mutex> g(m_);
        auto key = std::make_tuple(src_rank, targ_rank, tag);
        auto it = channels_.find(key);
        std::shared_ptr<cxx::Channel> ch;
        if (it != channels_.end()) {
            ch = it->second;  // the other endpoint connected first
        } else {
            ch = std::make_shared<cxx::Channel>();
            channels_[key] = ch;
        }
        if (bytes > ch->capacity) {
            ch->buffer.reserve((size_t)(bytes > 16 ? bytes : 16));
            ch->capacity = bytes;
        }
        return ch;
    }

private:
    struct Tls {
        GaspiEnvironment* env = nullptr;
        int rank = 0;
        GaspiEnvironment* stream_env = nullptr;
        void* user_stream = nullptr;
    };
    static Tls& tls() {
        static thread_local Tls t;
        return t;
    }

    unsigned long segment_size_;  // kept for callers that ask; nothing is reserved up front
    int rank_, ranks_;
    bool blocking_;
    double timeout_s_;
    std::mutex m_;
    std::condition_variable barrier_cv_;
    int barrier_count_;
    long long barrier_generation_;
    std::map<std::tuple<int, int, int>, std::shared_ptr<cxx::Channel> > channels_;
};

#endif  // GASPI_ENVIRONMENT_HXX
