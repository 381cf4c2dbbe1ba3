// The contract of the reference's TensorFlow ops (src/tf_ops/tfAllreduce.cc:24-41,55-72), driven
// the way an op kernel drives it: the object's address travels as a 64-bit integer attribute, and
// apply / flush run in place on a buffer in DEVICE memory (what a DEVICE_GPU kernel gets from its
// input tensor).  One host thread per simulated rank runs the per-rank program of the reference's
// Python op tests (test/AllToOneAllreduce.py, RingAllreduce.py, BigRingAllreduce.py); gold after
// `runs` x apply + flush: (runs * (ranks - 1) + 1) * values at the ranks those tests check.
// The calls go through tf_op_contract.hxx, the same functions comprex_amd/tf_ops/tfAllreduce.cc
// puts into its kernels' Compute().
#include <tf_op_contract.hxx>

#include <atomic>
#include <functional>
#include <mutex>
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

// a tensor's buffer in device memory
struct DeviceTensor {
    cxx::Handle handle;
    cxx::DeviceBuffer buffer;
    int count;
    explicit DeviceTensor(int n) : count(n) { buffer.reserve((size_t)n * sizeof(float)); }
    float* data() { return static_cast<float*>(buffer.data()); }
    void upload(const std::vector<float>& v) { cxx::check(cx_copy(handle.get(), data(), v.data(), v.size() * sizeof(float))); }
    void upload_range(const std::vector<float>& v, int lo, int hi) {
        if (hi > lo) cxx::check(cx_copy(handle.get(), data() + lo, v.data() + lo, (size_t)(hi - lo) * sizeof(float)));
    }
    std::vector<float> download() {
        std::vector<float> v(count);
        cxx::check(cx_copy(handle.get(), v.data(), data(), v.size() * sizeof(float)));
        return v;
    }
};

static int compare(int rank, const std::vector<float>& got, const std::vector<float>& gold) {
    int errors = 0;
    for (size_t i = 0; i < got.size(); ++i)
        if (got[i] != gold[i]) {
            if (errors < 3) {
                std::lock_guard<std::mutex> g(print_mutex);
                std::cout << "rank " << rank << " [" << i << "]: " << got[i] << " gold " << gold[i] << std::endl;
            }
            ++errors;
        }
    return errors;
}

enum Family { ALL_TO_ONE, RING, BIG_RING };

template <template <class> class Schedule> static void connect(Schedule<float>& s, int size);
template <> void connect<Comprex_AllToOneAllreduce>(Comprex_AllToOneAllreduce<float>& s, int size) {
    s.setupConnections(size, 0, 0, 1e-2f, 3.0f);
}
template <> void connect<Comprex_RingAllreduce>(Comprex_RingAllreduce<float>& s, int size) {
    s.setupConnections(size, 0, 1e-2f, 3.0f);
}
template <> void connect<Comprex_BigRingAllreduce>(Comprex_BigRingAllreduce<float>& s, int size) {
    s.setupConnections(size, 0, 1e-2f, 3.0f);
}

template <template <class> class Schedule> static int op_contract(const char* name, Family family, int ranks, int size, int runs) {
    GaspiEnvironment env(1ul << 32);
    env.set_rank(0, ranks);
    env.set_blocking(true, 60.0);
    std::vector<float> values(size), gold(size);
    for (int i = 0; i < size; ++i) {
        values[i] = (float)((i % 251) * (1 - 2 * (i % 2)));
        gold[i] = (float)(runs * (ranks - 1) + 1) * values[i];
    }
    int failed = run_ranks(env, ranks, [&](int rank) {
        Schedule<float> schedule(&env);
        connect<Schedule>(schedule, size);
        // python: ctypes.c_void_p(obj).value -> the op's integer attribute
        const comprex_tf::attr_int attribute = comprex_tf::attribute_of<Schedule, float>(&schedule);
        DeviceTensor tensor(size);
        tensor.upload(values);
        if (!cx_pointer_on_device(tensor.data())) return 1;
        env.barrier();
        int errors = 0;
        for (int run = 0; run < runs; ++run) {
            env.barrier();
            if (family == RING) {
                // the segment this rank finishes keeps accumulating; everything else starts from the values
                const int seg = size / ranks, lo = ((rank + 1) % ranks) * seg;
                tensor.upload_range(values, 0, lo);
                tensor.upload_range(values, lo + seg, size);
            } else if (rank != 0) {
                tensor.upload(values);
            }
            float* out = comprex_tf::compute_apply<Schedule, float>(attribute, tensor.data(), size);
            if (out != tensor.data()) ++errors;  // the output aliases the input
        }
        float* out = comprex_tf::compute_flush<Schedule, float>(attribute, tensor.data(), size);
        if (out != tensor.data()) ++errors;
        if (family == RING || rank == 0) errors += compare(rank, tensor.download(), gold);
        env.barrier();
        return errors;
    });
    std::cout << name << " through the op contract, " << ranks << " ranks, device buffer of " << size << std::endl;
    return print_pass(failed);
}

static int null_attribute_is_refused() {
    int errors = 1;
    float x = 0;
    try {
        comprex_tf::compute_apply<Comprex_BigRingAllreduce, float>(0, &x, 1);
    } catch (const std::invalid_argument&) {
        errors = 0;
    }
    std::cout << "null attribute" << std::endl;
    return print_pass(errors);
}

int main() {
    if (!need_gpu()) return 0;
    int errors = 0;
    errors += op_contract<Comprex_AllToOneAllreduce>("ComprexAlltooneAllreduceApply/Flush", ALL_TO_ONE, 3, 30000, 4);
    errors += op_contract<Comprex_RingAllreduce>("ComprexRingAllreduceApply/Flush", RING, 3, 30000, 4);
    errors += op_contract<Comprex_BigRingAllreduce>("ComprexBigringAllreduceApply/Flush", BIG_RING, 3, 30000, 4);
    errors += op_contract<Comprex_BigRingAllreduce>("ComprexBigringAllreduceApply/Flush", BIG_RING, 4, 100003, 3);
    errors += null_attribute_is_refused();
    return errors ? 1 : 0;
}
