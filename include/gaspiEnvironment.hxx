// Stand-in for the reference's GaspiEnvironment (include/gaspiEnvironment.hxx:9-28) on ONE
// GPU: several simulated ranks live in one process and exchange messages through device
// buffers.  There is no GASPI, no RDMA and no second GPU.
//
// A directed channel is identified by (source rank, target rank, tag), as the reference's
// SourceBuffer::connectToRemoteTarget / TargetBuffer::connectToRemoteSource pair is
// (src/comprEx.tpp:341-363).  The sender's compressor writes the message straight into the
// channel's device buffer and the receiver reads it from there: the "transfer" is the
// stream order of the two kernels.
#ifndef GASPI_ENVIRONMENT_HXX
#define GASPI_ENVIRONMENT_HXX

#include <map>
#include <memory>
#include <stdexcept>
#include <tuple>

#include "cx_device.hxx"

namespace cxx {

struct Channel {
    DeviceBuffer buffer;   // message area, bufferSize bytes
    long long capacity = 0;
    bool has_sender = false, has_receiver = false;
    long long sent = 0, received = 0;  // messages written / consumed
};

}  // namespace cxx

class GaspiEnvironment {
public:
    // segment_size is what the reference reserves for GASPI; device buffers are allocated per
    // channel here, so it is only remembered.
    GaspiEnvironment(unsigned long segment_size) : segment_size_(segment_size), rank_(0), ranks_(1) {}
    ~GaspiEnvironment() {}

    int get_rank() { return rank_; }
    int get_ranks() { return ranks_; }
    // Not in the reference (gaspi_run fixes both there): which simulated rank the following
    // calls act as, and how many ranks there are.
    void set_rank(int rank, int ranks) {
        if (ranks < 1 || rank < 0 || rank >= ranks) throw std::runtime_error("set_rank: rank outside [0, ranks)");
        rank_ = rank;
        ranks_ = ranks;
    }
    void barrier() {}
    void flush() {}
    // what the reference hands to ComprEx as `segment`
    GaspiEnvironment* get_segment() { return this; }
    unsigned long get_segment_size() const { return segment_size_; }

    std::shared_ptr<cxx::Channel> channel(int src_rank, int targ_rank, int tag, long long bytes) {
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
    unsigned long segment_size_;  // kept for callers that ask; nothing is reserved up front
    int rank_, ranks_;
    std::map<std::tuple<int, int, int>, std::shared_ptr<cxx::Channel> > channels_;
};

#endif  // GASPI_ENVIRONMENT_HXX
