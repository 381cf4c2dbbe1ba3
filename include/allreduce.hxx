// The three compressed allreduce schedules of the reference (include/allreduce.hxx:64-211,
// src/allreduce.tpp:122-721) over simulated ranks on one GPU: every rank is a host thread
// that owns one object and runs the reference's per-rank sequence; messages travel through
// the device-buffer channels of the GaspiEnvironment stand-in (set_blocking(true)).
//
//   Comprex_AllToOneAllreduce  workers send to the chief, the chief adds the messages in
//                              ascending rank order and broadcasts (FastComprEx channels)
//   Comprex_RingAllreduce      segmented ring reduce + ring broadcast, one ComprEx per segment
//   Comprex_BigRingAllreduce   unsegmented ring: every message is forwarded R-2 times
//
// apply(data, size) / flush(data, size) work in place on `data` (host or device pointer), which
// is what the reference's TF ops call (src/tf_ops/tfAllreduce.cc:33-37,64-68).  The
// uncompressed variants (GaspiEx based) are transport only and are not provided.
#ifndef ALLREDUCE_HXX
#define ALLREDUCE_HXX

#include <cstdio>
#include <map>
#include <stdexcept>
#include <vector>

#include "comprEx.hxx"
#include "gaspiEnvironment.hxx"

template <typename data_t>
class Allreduce_base {
public:
    Allreduce_base(GaspiEnvironment* gaspi_env) { this->gaspi_env = gaspi_env; }
    virtual ~Allreduce_base() {}
    virtual void apply(data_t* data, int size) = 0;

protected:
    GaspiEnvironment* gaspi_env;

    static void require_size(int size, int communicated) {
        if (size < communicated) {
            char error_msg[100];
            snprintf(error_msg, sizeof error_msg, "Vector size (%d) is smaller than communicated data size (%d)!\n",
                     size, communicated);
            throw std::runtime_error(error_msg);
        }
    }
};

// ---------------------------------------------------------------------------------------
template <typename data_t>
class Comprex_AllToOneAllreduce : public Allreduce_base<data_t> {
public:
    Comprex_AllToOneAllreduce(GaspiEnvironment* gaspi_env) : Allreduce_base<data_t>(gaspi_env), comm_size(0), chiefRank(0) {}
    ~Comprex_AllToOneAllreduce() {}

    void setupConnections(int size, int tag, int chiefRank, float compression_ratio, float size_factor = 1.0) {
        const int myRank = this->gaspi_env->get_rank();
        const int numRanks = this->gaspi_env->get_ranks();
        this->chiefRank = chiefRank;
        this->comm_size = size;
        const int comprexTag = tag * 2 * numRanks;
        const int commTag = tag * 2 * numRanks + 1;

        FastComprEx<data_t> comm_proto(this->gaspi_env->get_segment(), size, size_factor);
        comm_proto.setThreshold(ThresholdTopK<data_t>(compression_ratio));
        comm_proto.setCompressor(CompressorIndexPairs<data_t>());
        for (int rank = 0; rank < numRanks; ++rank) {
            if (rank == chiefRank) continue;
            if (myRank == chiefRank) {  // the chief talks to every worker
                comm_reduce_map[rank] = comm_proto;
                comm_reduce_map[rank].connectRx(rank, comprexTag + rank);
                comm_broadcast_map[rank] = comm_proto;
                comm_broadcast_map[rank].connectTx(rank, commTag + rank);
            } else if (rank == myRank) {  // a worker talks to the chief only
                comm_reduce_map[chiefRank] = comm_proto;
                comm_reduce_map[chiefRank].connectTx(chiefRank, comprexTag + myRank);
                comm_broadcast_map[chiefRank] = comm_proto;
                comm_broadcast_map[chiefRank].connectRx(chiefRank, commTag + myRank);
            }
        }
    }

    virtual void apply(data_t* data, int size) {
        this->require_size(size, comm_size);
        const int myRank = this->gaspi_env->get_rank();
        const int numRanks = this->gaspi_env->get_ranks();
        if (myRank == chiefRank) {
            reduce_workers(data, size);
            // broadcast: compress once, hand the same buffer to the other workers
            int copy_rank = -1;
            for (int rank = 0; rank < numRanks; ++rank) {
                if (rank == chiefRank) continue;
                if (copy_rank == -1) {
                    comm_broadcast_map[rank].writeRemote(data, size);
                    copy_rank = rank;
                } else {
                    comm_broadcast_map[rank].writeRemote_sameAs(&comm_broadcast_map[copy_rank]);
                }
            }
        } else {
            comm_reduce_map[chiefRank].writeRemote(data, size);
            comm_broadcast_map[chiefRank].readRemote(data, size);
        }
    }

    // workers send their residuals, the chief adds them; nothing is broadcast; everything is reset
    virtual void flush(data_t* data, int size) {
        const int myRank = this->gaspi_env->get_rank();
        if (myRank == chiefRank) {
            reduce_workers(data, size);
        } else {
            comm_reduce_map[chiefRank].flushRests();
        }
        reset();
    }

    // The chief's loop `for rank: readRemote_add(data)` (src/allreduce.tpp:186-189) as one pass over
    // `data`: every worker's message is waited for, then all are added in ascending rank order (which
    // fixes the order of the floating-point additions, as the loop does) by one rank-ordered reduce.
    void reduce_workers(data_t* data, int size) {
        const int numRanks = this->gaspi_env->get_ranks();
        int first = -1;
        for (int rank = 0; rank < numRanks && first < 0; ++rank)
            if (rank != chiefRank) first = rank;
        if (first < 0) return;
        FastComprEx<data_t>* reader = &comm_reduce_map[first];  // its stream reads every message
        // every channel whose message was taken is released when this call leaves, also by an exception
        struct Taken {
            std::vector<FastComprEx<data_t>*> from;
            FastComprEx<data_t>* reader;
            ~Taken() {
                for (auto* c : from) {
                    try {
                        c->message_done(reader);
                    } catch (...) {
                    }
                }
            }
        } taken;
        taken.reader = reader;
        std::vector<const void*> messages;
        for (int rank = 0; rank < numRanks; ++rank) {
            if (rank == chiefRank) continue;
            messages.push_back(comm_reduce_map[rank].waiting_message(reader));
            taken.from.push_back(&comm_reduce_map[rank]);
        }
        reader->add_messages(data, size, messages.data(), (int)messages.size());
    }

    void reset() {
        for (auto& comm : comm_reduce_map) comm.second.resetRests();
        for (auto& comm : comm_broadcast_map) comm.second.resetRests();
    }

    void set_compression_ratio(float compression_ratio) {
        for (auto& comm : comm_reduce_map) comm.second.setThreshold(ThresholdTopK<data_t>(compression_ratio));
        for (auto& comm : comm_broadcast_map) comm.second.setThreshold(ThresholdTopK<data_t>(compression_ratio));
    }

protected:
    std::map<int, FastComprEx<data_t> > comm_reduce_map;
    std::map<int, FastComprEx<data_t> > comm_broadcast_map;
    int comm_size;
    int chiefRank;
};

// ---------------------------------------------------------------------------------------
template <typename data_t>
class Comprex_RingAllreduce : public Allreduce_base<data_t> {
public:
    Comprex_RingAllreduce(GaspiEnvironment* gaspi_env) : Allreduce_base<data_t>(gaspi_env), total_size(0) {}
    ~Comprex_RingAllreduce() {}

    void setupConnections(int size, int tag, float compression_ratio, float size_factor = 1.0) {
        const int myRank = this->gaspi_env->get_rank();
        const int numRanks = this->gaspi_env->get_ranks();
        this->total_size = size;
        // contiguous segments, the first size % numRanks of them one element longer
        segment_sizes.assign(numRanks, size / numRanks);
        for (int it = 0; it < size % numRanks; ++it) segment_sizes[it] += 1;
        segment_starts.assign(numRanks, 0);
        for (int it = 1; it < numRanks; ++it) segment_starts[it] = segment_starts[it - 1] + segment_sizes[it - 1];
        if (segment_starts[numRanks - 1] + segment_sizes[numRanks - 1] != total_size)
            throw std::runtime_error("Last segment should end at the total size of the data!");

        const int recv_from = (myRank - 1 + numRanks) % numRanks;
        const int send_to = (myRank + 1) % numRanks;
        const bool send_sizeBytes = true;
        // the reduce ring estimates its threshold on fewer samples (src/allreduce.tpp:402-403)
        const int thresholdTopK_subsamples = 1000 / numRanks;
        const float thresholdTopK_sampleFactor = 4.0;
        for (int chunk = 0; chunk < numRanks; ++chunk) {
            comm_reduce_map[chunk] =
                ComprEx<data_t>(this->gaspi_env->get_segment(), segment_sizes[chunk], size_factor, send_sizeBytes);
            comm_reduce_map[chunk].setThreshold(
                ThresholdTopK<data_t>(compression_ratio, thresholdTopK_subsamples, thresholdTopK_sampleFactor));
            comm_reduce_map[chunk].setCompressor(CompressorIndexPairs<data_t>());
            comm_reduce_map[chunk].connectTo(recv_from, send_to, tag + chunk);
            comm_broadcast_map[chunk] =
                ComprEx<data_t>(this->gaspi_env->get_segment(), segment_sizes[chunk], size_factor, send_sizeBytes);
            comm_broadcast_map[chunk].setThreshold(ThresholdTopK<data_t>(compression_ratio));
            comm_broadcast_map[chunk].setCompressor(CompressorIndexPairs<data_t>());
            comm_broadcast_map[chunk].connectTo(recv_from, send_to, tag + numRanks + chunk);
        }
    }

    virtual void apply(data_t* data, int size) {
        this->require_size(size, total_size);
        const int myRank = this->gaspi_env->get_rank();
        const int numRanks = this->gaspi_env->get_ranks();
        // reduce ring: in step `it` segment (myRank - it) leaves and segment (myRank - it - 1) arrives
        for (int it = 0; it < numRanks - 1; ++it) {
            const int recv_chunk = (myRank - it - 1 + numRanks) % numRanks;
            const int send_chunk = (myRank - it + numRanks) % numRanks;
            comm_reduce_map[send_chunk].writeRemote(data + segment_starts[send_chunk], segment_sizes[send_chunk]);
            comm_reduce_map[recv_chunk].readRemote_add(data + segment_starts[recv_chunk], segment_sizes[recv_chunk]);
        }
        // broadcast ring: the finished segment is thresholded once (no residual) and passed round compressed
        const int first = (myRank + 1 + numRanks) % numRanks;
        comm_broadcast_map[first].writeRemote_NoResidual(data + segment_starts[first], segment_sizes[first]);
        for (int it = 0; it < numRanks - 2; ++it) {
            const int recv_chunk = (myRank - it + numRanks) % numRanks;
            comm_broadcast_map[recv_chunk].readRemote_forward(data + segment_starts[recv_chunk],
                                                              segment_sizes[recv_chunk]);
        }
        const int last = (myRank + 2) % numRanks;
        comm_broadcast_map[last].readRemote(data + segment_starts[last], segment_sizes[last]);
    }

    // sends every residual round the reduce ring uncompressed-in-content (threshold-free) and
    // broadcasts the exact sums (src/allreduce.tpp:463-509)
    virtual void flush(data_t* data, int size) {
        const int myRank = this->gaspi_env->get_rank();
        const int numRanks = this->gaspi_env->get_ranks();
        int recv_chunk = (myRank - 1 + numRanks) % numRanks;
        int send_chunk = myRank % numRanks;
        comm_reduce_map[send_chunk].getRests(data + segment_starts[send_chunk], segment_sizes[send_chunk]);
        comm_reduce_map[send_chunk].resetRests();
        comm_reduce_map[send_chunk].writeRemote_compressOnly(data + segment_starts[send_chunk],
                                                             segment_sizes[send_chunk]);
        if (numRanks > 2)
            comm_reduce_map[recv_chunk].readRemote(data + segment_starts[recv_chunk], segment_sizes[recv_chunk]);
        else  // with two ranks the other rank already holds the reduced segment
            comm_reduce_map[recv_chunk].readRemote_add(data + segment_starts[recv_chunk], segment_sizes[recv_chunk]);
        for (int it = 1; it < numRanks - 1; ++it) {
            recv_chunk = (myRank - it - 1 + numRanks) % numRanks;
            send_chunk = (myRank - it + numRanks) % numRanks;
            comm_reduce_map[send_chunk].addRests(data + segment_starts[send_chunk], segment_sizes[send_chunk]);
            comm_reduce_map[send_chunk].resetRests();
            comm_reduce_map[send_chunk].writeRemote_compressOnly(data + segment_starts[send_chunk],
                                                                 segment_sizes[send_chunk]);
            if (it == numRanks - 2)
                comm_reduce_map[recv_chunk].readRemote_add(data + segment_starts[recv_chunk],
                                                           segment_sizes[recv_chunk]);
            else
                comm_reduce_map[recv_chunk].readRemote(data + segment_starts[recv_chunk], segment_sizes[recv_chunk]);
        }
        for (int it = 0; it < numRanks - 1; ++it) {
            recv_chunk = (myRank - it + numRanks) % numRanks;
            send_chunk = (myRank - it + 1 + numRanks) % numRanks;
            comm_broadcast_map[send_chunk].writeRemote_compressOnly(data + segment_starts[send_chunk],
                                                                    segment_sizes[send_chunk]);
            comm_broadcast_map[recv_chunk].readRemote(data + segment_starts[recv_chunk], segment_sizes[recv_chunk]);
        }
        reset();
    }

    void reset() {
        for (auto& comm : comm_reduce_map) comm.second.resetRests();
        for (auto& comm : comm_broadcast_map) comm.second.resetRests();
    }

    void set_compression_ratio(float compression_ratio) {
        for (auto& comm : comm_reduce_map) comm.second.setThreshold(ThresholdTopK<data_t>(compression_ratio));
        for (auto& comm : comm_broadcast_map) comm.second.setThreshold(ThresholdTopK<data_t>(compression_ratio));
    }

protected:
    std::map<int, ComprEx<data_t> > comm_reduce_map;
    std::map<int, ComprEx<data_t> > comm_broadcast_map;
    int total_size;
    std::vector<int> segment_sizes;
    std::vector<int> segment_starts;
};

// ---------------------------------------------------------------------------------------
template <typename data_t>
class Comprex_BigRingAllreduce : public Allreduce_base<data_t> {
public:
    Comprex_BigRingAllreduce(GaspiEnvironment* gaspi_env) : Allreduce_base<data_t>(gaspi_env), total_size(0) {}
    ~Comprex_BigRingAllreduce() {}

    void setupConnections(int size, int tag, float compression_ratio, float size_factor = 1.0) {
        const int myRank = this->gaspi_env->get_rank();
        const int numRanks = this->gaspi_env->get_ranks();
        this->total_size = size;
        const int recv_from = (myRank - 1 + numRanks) % numRanks;
        const int send_to = (myRank + 1) % numRanks;
        comm_reduce[0] = ComprEx<data_t>(this->gaspi_env->get_segment(), size, size_factor, true);
        comm_reduce[0].setThreshold(ThresholdTopK<data_t>(compression_ratio, 1000 / numRanks, 4.0));
        comm_reduce[0].setCompressor(CompressorIndexPairs<data_t>());
        comm_reduce[0].connectTo(recv_from, send_to, tag);
        // The reference's two GaspiEx<char> feedback rings (src/allreduce.tpp:640-644) only tell
        // a sender when its neighbour's buffers may be overwritten; the channels here do that
        // themselves (a send waits until the previous message was consumed).
    }

    virtual void apply(data_t* data, int size) {
        this->require_size(size, total_size);
        comm_reduce[0].writeRemote(data, size);
        hops(data, size);
    }

    virtual void flush(data_t* data, int size) {
        this->require_size(size, total_size);
        comm_reduce[0].flushRests();
        hops(data, size);
        reset();
    }

    void reset() { comm_reduce[0].resetRests(); }

    virtual void set_compression_ratio(float compression_ratio) {
        comm_reduce[0].setThreshold(ThresholdTopK<data_t>(compression_ratio));
    }

protected:
    ComprEx<data_t> comm_reduce[1];
    int total_size;

    // every message travels R-1 hops: it is forwarded (and added) R-2 times, then only added
    void hops(data_t* data, int size) {
        const int numRanks = this->gaspi_env->get_ranks();
        for (int it = 0; it < numRanks - 2; ++it) {
            comm_reduce[0].readRemote_wait();
            comm_reduce[0].forward_buffer();
            comm_reduce[0].forward_add(data, size);
        }
        comm_reduce[0].readRemote_add(data, size);
    }
};

#endif  // ALLREDUCE_HXX
