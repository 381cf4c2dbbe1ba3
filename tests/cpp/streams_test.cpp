// Streams and events of the exchange classes (reference: the asynchronous put and the receiver's
// wait, src/comprEx.tpp:190,231,243).  Every ComprEx object works on a stream of its own; a message
// is handed over by an event; every call joins the object's stream with the caller's.
//   1. the golds of test/AllToOneAllreduce.cpp, test/RingAllreduce.cpp, test/BigRingAllreduce.cpp on
//      DEVICE vectors, each simulated rank producing and consuming its vector on a stream of its own
//      without ever waiting in between;
//   2. the gold of test/comprex.cpp with the sender moved to another stream (ComprEx::set_stream ->
//      cx_set_stream) and the receiver's vector living on a third one;
//   3. a message cut short for lack of room does not disturb the receives of the same object;
//   4. messages whose indices are not sorted (the reference's add takes any order,
//      src/compressor.hxx:640-658) through add() and add_many().
#include <allreduce.hxx>

#include <atomic>
#include <functional>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "common.hxx"

static std::mutex print_mutex;

static int run_ranks(GaspiEnvironment& env, int ranks, const std::function<int(int)>& fn) {
    std::atomic<int> failed(0);
    std::vector<std::thread> threads;
    for (int r = 0; r < ranks; ++r)
        threads.emplace_back([&, r] {
            try {
                env.set_rank(r, ranks);
                if (fn(r) != 0) ++failed;
            } catch (const std::exception& e) {
                std::lock_guard<std::mutex> g(print_mutex);
                std::cout << "rank " << r << " threw: " << e.what() << std::endl;
                ++failed;
            }
        });
    for (auto& t : threads) t.join();
    return failed.load();
}

// A simulated rank's side of the GPU: a stream of its own, a handle on it for the kernels that stand
// for the framework's work on the vector, and device memory.
struct RankGpu {
    void* stream = nullptr;
    cx_handle h = nullptr;
    std::vector<void*> mem;
    RankGpu() {
        cxx::check(cx_stream_create(&stream));
        cxx::check(cx_create(&h, stream));
    }
    ~RankGpu() {
        cx_destroy(h);
        for (void* p : mem) cx_device_free(p);
        cx_stream_destroy(stream);
    }
    template <typename T> T* alloc(size_t n) {
        void* p = nullptr;
        cxx::check(cx_device_alloc(&p, n * sizeof(T)));
        mem.push_back(p);
        return static_cast<T*>(p);
    }
    template <typename T> T* upload(const std::vector<T>& v) {
        T* d = alloc<T>(v.size());
        cxx::check(cx_copy(h, d, v.data(), v.size() * sizeof(T)));  // (waits: the host vector is pageable)
        return d;
    }
    // d = src, as two kernels on the rank's stream; nothing waits
    template <typename T> void assign(T* d, const T* src, int n) {
        cxx::check(cx_zero(h, cxx::dtype_of<T>::value, d, n));
        cxx::check(cx_add_vec(h, cxx::dtype_of<T>::value, d, src, n));
    }
    template <typename T> std::vector<T> download(const T* d, size_t n) {
        std::vector<T> v(n);
        cxx::check(cx_copy(h, v.data(), d, n * sizeof(T)));
        cxx::check(cx_synchronize(h));
        return v;
    }
};

template <typename data_t> static std::vector<data_t> make_values(int size) {
    std::vector<data_t> values(size);
    for (int i = 0; i < size; ++i) values[i] = (data_t)((i % 251) * (1 - 2 * (i % 2)));
    return values;
}

template <typename data_t> static int check(int rank, const std::vector<data_t>& result, const std::vector<data_t>& gold) {
    int errors = 0;
    for (size_t i = 0; i < result.size(); ++i)
        if (result[i] != gold[i]) {
            if (errors < 3) {
                std::lock_guard<std::mutex> g(print_mutex);
                std::cout << "Rank " << rank << " Error in [" << i << "]: result: " << result[i] << " gold: " << gold[i] << std::endl;
            }
            ++errors;
        }
    return errors;
}

// kind 0: all-to-one (chief checks), 1: ring (every rank checks), 2: big ring (chief checks)
template <typename data_t> int schedule_on_streams(int kind, int numRanks, int size, int num_runs) {
    GaspiEnvironment gaspi_env(1ul << 32);
    gaspi_env.set_rank(0, numRanks);
    gaspi_env.set_blocking(true, 60.0);
    const int chiefRank = 0, tag = 0;
    const std::vector<data_t> values = make_values<data_t>(size);
    std::vector<data_t> gold(size);
    for (int i = 0; i < size; ++i) gold[i] = (data_t)((num_runs * (numRanks - 1) + 1) * values[i]);
    int failed = run_ranks(gaspi_env, numRanks, [&](int myRank) {
        RankGpu gpu;
        gaspi_env.set_user_stream(gpu.stream);  // this rank's vectors live on its own stream
        data_t* d_values = gpu.upload(values);
        data_t* d_result = gpu.upload(values);
        int errors = 0;
        if (kind == 0) {
            Comprex_AllToOneAllreduce<data_t> allreduce(&gaspi_env);
            allreduce.setupConnections(size, tag, chiefRank, 1e-2f, 3.0f);
            gaspi_env.barrier();
            for (int run = 0; run < num_runs; ++run) {
                if (myRank != chiefRank) gpu.assign(d_result, d_values, size);
                allreduce.apply(d_result, size);
            }
            allreduce.flush(d_result, size);
            if (myRank == chiefRank) errors = check(myRank, gpu.download(d_result, size), gold);
        } else if (kind == 1) {
            Comprex_RingAllreduce<data_t> allreduce(&gaspi_env);
            allreduce.setupConnections(size, tag, 1e-2f, 3.0f);
            gaspi_env.barrier();
            const int seg = size / numRanks;
            const int val_start = myRank < numRanks - 1 ? (myRank + 1) * seg : 0, val_stop = val_start + seg;
            for (int run = 0; run < num_runs; ++run) {
                gaspi_env.barrier();
                // everything but this rank's accumulating region is set back to the values
                if (val_start > 0) gpu.assign(d_result, d_values, val_start);
                if (val_stop < size) gpu.assign(d_result + val_stop, d_values + val_stop, size - val_stop);
                allreduce.apply(d_result, size);
            }
            allreduce.flush(d_result, size);
            errors = check(myRank, gpu.download(d_result, size), gold);
        } else {
            Comprex_BigRingAllreduce<data_t> allreduce(&gaspi_env);
            allreduce.setupConnections(size, tag, 1e-2f, 3.0f);
            gaspi_env.barrier();
            for (int run = 0; run < num_runs; ++run) {
                gaspi_env.barrier();
                if (myRank != chiefRank) gpu.assign(d_result, d_values, size);
                allreduce.apply(d_result, size);
            }
            allreduce.flush(d_result, size);
            if (myRank == chiefRank) errors = check(myRank, gpu.download(d_result, size), gold);
        }
        gaspi_env.barrier();
        return errors;
    });
    const char* names[3] = {"Comprex_AllToOneAllreduce", "Comprex_RingAllreduce", "Comprex_BigRingAllreduce"};
    std::cout << names[kind] << " on device vectors, one stream per rank and per object, " << numRanks << " ranks, n=" << size
              << std::endl;
    return print_pass(failed);
}

// test/comprex.cpp's conservation gold: the sender on a stream given from outside, the vectors on a third
int p2p_foreign_stream() {
    typedef float data_t;
    const int size = 300007, num_runs = 5;
    std::vector<data_t> values(size);
    unsigned x = 99u;
    for (int i = 0; i < size; ++i) {
        x = x * 1664525u + 1013904223u;
        values[i] = (data_t)((int)((x >> 8) % 2001u) - 1000);
    }
    RankGpu user;     // where the caller's vectors live
    RankGpu foreign;  // the stream the sender is moved to
    GaspiEnvironment env(1 << 28);
    env.set_user_stream(user.stream);
    std::vector<ComprEx<data_t> > cmprex;
    cmprex.reserve(2);
    for (int rank = 0; rank < 2; ++rank) {
        env.set_rank(rank, 2);
        cmprex.emplace_back(env.get_segment(), size, 3.0f, true);
        cmprex[rank].setThreshold(ThresholdTopK<data_t>(0.05f));
        cmprex[rank].setCompressor(CompressorIndexPairs<data_t>());
        cmprex[rank].connectTo((rank + 1) % 2, (rank + 1) % 2, 7);
    }
    int errors = 0;
    if (cmprex[0].get_stream() == cmprex[1].get_stream() || cmprex[0].get_stream() == nullptr) {
        std::cout << "the two objects do not have streams of their own" << std::endl;
        ++errors;
    }
    cmprex[0].set_stream(foreign.stream);
    if (cmprex[0].get_stream() != foreign.stream) ++errors;
    data_t* d_values = user.upload(values);
    data_t* d_grad = user.alloc<data_t>(size);
    data_t* d_result = user.alloc<data_t>(size);
    cxx::check(cx_zero(user.h, CX_F32, d_result, size));
    for (int run = 0; run < num_runs; ++run) {
        if (run < num_runs - 1) {
            user.assign(d_grad, d_values, size);  // the "backward pass" on the user's stream, not waited for
            cmprex[0].writeRemote(d_grad, size);
        } else {
            cmprex[0].flushRests();
        }
        cmprex[1].readRemote_add(d_result, size);
    }
    const std::vector<data_t> result = user.download(d_result, size);
    for (int i = 0; i < size; ++i)
        if (result[i] != (data_t)(num_runs - 1) * values[i]) {
            if (errors < 5) std::cout << "Error in [" << i << "]: result: " << result[i] << std::endl;
            ++errors;
        }
    for (auto e : cmprex[0].getRests()) if (e != 0) ++errors;
    std::cout << "ComprEx point to point, sender on a foreign stream (cx_set_stream), vectors on a third" << std::endl;
    return print_pass(errors);
}

// One object sends into a buffer that is too small (size_factor < 1: the message is cut short, the
// rest stays in the residual) and then receives: the receive works and frees its channel.
int short_message_then_receive() {
    typedef float data_t;
    const int size = 4096;
    std::vector<data_t> values(size), result(size, (data_t)0);
    for (int i = 0; i < size; ++i) values[i] = (data_t)(1 + i % 7);
    GaspiEnvironment env(1 << 26);
    std::vector<ComprEx<data_t> > cmprex;
    cmprex.reserve(2);
    for (int rank = 0; rank < 2; ++rank) {
        env.set_rank(rank, 2);
        cmprex.emplace_back(env.get_segment(), size, 0.25f, true);  // room for about an eighth of the pairs
        cmprex[rank].setThreshold(ThresholdConst<data_t>(0));       // everything non-zero is to be sent
        cmprex[rank].setCompressor(CompressorIndexPairs<data_t>());
        cmprex[rank].connectTo((rank + 1) % 2, (rank + 1) % 2, 11);
    }
    int errors = 0;
    try {
        // both directions: every object has sent a short message before it receives
        cmprex[0].writeRemote(values.data(), size);
        cmprex[1].writeRemote(values.data(), size);
        cmprex[0].readRemote_add(result.data(), size);
        cmprex[1].readRemote_add(result.data(), size);
        // the channels are free again: a second round goes through
        cmprex[0].writeRemote(values.data(), size);
        cmprex[1].readRemote_add(result.data(), size);
    } catch (const std::exception& e) {
        std::cout << "threw: " << e.what() << std::endl;
        ++errors;
    }
    // conservation: what arrived plus what the sender still holds is what was given
    const std::vector<data_t> r0 = cmprex[0].getRests(), r1 = cmprex[1].getRests();
    long sent = 0;
    for (int i = 0; i < size; ++i) {
        sent += result[i] != 0;
        if (result[i] + r0[i] + r1[i] != 3 * values[i]) {
            if (errors < 5) std::cout << "Error in [" << i << "]: " << result[i] << " + " << r0[i] << " + " << r1[i] << std::endl;
            ++errors;
        }
    }
    if (sent == 0 || sent >= size) ++errors;  // some, not all
    // the flush says that it could not send everything, and leaves the rest where it was
    bool told = false;
    try {
        cmprex[0].flushRests();
    } catch (const std::exception&) {
        told = true;
    }
    if (!told) {
        std::cout << "flushRests did not report the short buffer" << std::endl;
        ++errors;
    }
    std::cout << "a message cut short for lack of room, then receives on the same object" << std::endl;
    return print_pass(errors);
}

// add() and add_many() on hand-made messages whose indices are not sorted and repeat far apart:
// the reference's loop, out[index] += value in message order.
int unsorted_messages() {
    typedef float data_t;
    const int n = 5000, k = 3000;
    struct Pair { int i; float v; };
    auto make = [&](unsigned seed, bool sorted) {
        std::vector<unsigned char> msg(8 + (size_t)k * 8);
        int hdr[2] = {n, k};
        memcpy(msg.data(), hdr, 8);
        unsigned x = seed;
        std::vector<Pair> pairs(k);
        for (int j = 0; j < k; ++j) {
            x = x * 1664525u + 1013904223u;
            pairs[j].i = sorted ? (int)((long long)j * n / k) : (int)((x >> 8) % (unsigned)(n / 4));  // many repeats
            x = x * 1664525u + 1013904223u;
            pairs[j].v = (float)((int)((x >> 8) % 2001u) - 1000) * 1.0009765625f;  // sums depend on their order
        }
        memcpy(msg.data() + 8, pairs.data(), (size_t)k * 8);
        return msg;
    };
    auto apply = [&](std::vector<data_t>& out, const std::vector<unsigned char>& msg) {
        const Pair* p = reinterpret_cast<const Pair*>(msg.data() + 8);
        for (int j = 0; j < k; ++j) out[p[j].i] += p[j].v;
    };
    int errors = 0;
    CompressorIndexPairs<data_t> comp;
    std::vector<std::vector<unsigned char> > msgs = {make(1, false), make(2, true), make(3, false), make(4, false)};
    // add(): one message at a time
    std::vector<data_t> want(n), got(n);
    for (int i = 0; i < n; ++i) want[i] = got[i] = (data_t)(i % 13) * 0.37f;
    for (auto& m : msgs) {
        apply(want, m);
        comp.add(got.data(), n, m.data());
    }
    if (memcmp(want.data(), got.data(), n * sizeof(data_t)) != 0) {
        std::cout << "add() of unsorted messages differs from the sequential loop" << std::endl;
        ++errors;
    }
    // add_many(): all at once, device-resident messages
    RankGpu gpu;
    std::vector<const void*> d_msgs;
    for (auto& m : msgs) d_msgs.push_back(gpu.upload(m));
    std::vector<data_t> got2(n);
    for (int i = 0; i < n; ++i) got2[i] = (data_t)(i % 13) * 0.37f;
    comp.add_many(got2.data(), n, d_msgs.data(), (int)d_msgs.size());
    if (memcmp(want.data(), got2.data(), n * sizeof(data_t)) != 0) {
        std::cout << "add_many() of unsorted messages differs from the sequential loop" << std::endl;
        ++errors;
    }
    // the calls that do not wait report the disorder instead of adding something else
    data_t* d_out = gpu.alloc<data_t>(n);
    cxx::check(cx_zero(gpu.h, CX_F32, d_out, n));
    cxx::check(cx_ip_add(gpu.h, CX_F32, d_out, n, d_msgs[0], 0));
    if (cx_synchronize(gpu.h) != CX_ERR_INDEX) {
        std::cout << "cx_ip_add without a wait did not report the unsorted message" << std::endl;
        ++errors;
    }
    cxx::check(cx_ip_reduce(gpu.h, CX_F32, d_out, n, d_msgs.data(), (int)d_msgs.size(), 0, 0));
    if (cx_synchronize(gpu.h) != CX_ERR_INDEX) {
        std::cout << "cx_ip_reduce without the any-order flag did not report the unsorted messages" << std::endl;
        ++errors;
    }
    // with the flag: from zeros, equal to the loop
    std::vector<data_t> want0(n, (data_t)0);
    for (auto& m : msgs) apply(want0, m);
    cxx::check(cx_ip_reduce(gpu.h, CX_F32, d_out, n, d_msgs.data(), (int)d_msgs.size(), 0, CX_REDUCE_ANY_ORDER));
    cxx::check(cx_synchronize(gpu.h));
    if (gpu.download(d_out, n) != want0) {
        std::cout << "cx_ip_reduce with CX_REDUCE_ANY_ORDER differs from the sequential loop" << std::endl;
        ++errors;
    }
    std::cout << "messages in any index order through add / add_many / cx_ip_reduce" << std::endl;
    return print_pass(errors);
}

int main() {
    if (!need_gpu()) return 77;
    int failed = 0;
    failed += schedule_on_streams<int>(0, 4, 100000, 10);
    failed += schedule_on_streams<float>(0, 3, 1000000, 5);
    failed += schedule_on_streams<int>(1, 4, 1000, 10);
    failed += schedule_on_streams<float>(1, 5, 100000, 5);
    failed += schedule_on_streams<int>(2, 4, 50, 50);
    failed += schedule_on_streams<float>(2, 3, 100000, 5);
    failed += p2p_foreign_stream();
    failed += short_message_then_receive();
    failed += unsorted_messages();
    return failed ? 1 : 0;
}
