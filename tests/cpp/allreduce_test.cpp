// Mirrors the reference's allreduce tests with one host thread per simulated rank, each running
// the per-rank program of the reference test unchanged:
//   test/AllToOneAllreduce.cpp, test/RingAllreduce.cpp, test/BigRingAllreduce.cpp
// gold at the checked ranks after `num_runs` x apply + flush: (num_runs*(numRanks-1)+1)*values.
#include <allreduce.hxx>

#include <atomic>
#include <functional>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "common.hxx"

static std::mutex print_mutex;

// runs fn(rank) on `ranks` threads; returns the number of ranks that reported errors or threw
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

// test/AllToOneAllreduce.cpp:30-103
template <typename data_t> int all_to_one(const char* name, int numRanks, int size, int num_runs) {
    GaspiEnvironment gaspi_env(1ul << 32);
    gaspi_env.set_rank(0, numRanks);
    gaspi_env.set_blocking(true, 60.0);
    const int chiefRank = 0, tag = 0;
    const std::vector<data_t> values = make_values<data_t>(size);
    std::vector<data_t> gold(size);
    for (int i = 0; i < size; ++i) gold[i] = (data_t)((num_runs * (numRanks - 1) + 1) * values[i]);
    int failed = run_ranks(gaspi_env, numRanks, [&](int myRank) {
        std::vector<data_t> result(values);
        Comprex_AllToOneAllreduce<data_t> allreduce(&gaspi_env);
        allreduce.setupConnections(size, tag, chiefRank, 1e-2f, 3.0f);
        gaspi_env.barrier();
        for (int run = 0; run < num_runs; ++run) {
            if (myRank != chiefRank) result = values;
            allreduce.apply(result.data(), size);
        }
        allreduce.flush(result.data(), size);
        int errors = myRank == chiefRank ? check(myRank, result, gold) : 0;
        gaspi_env.barrier();
        return errors;
    });
    std::cout << "Comprex_AllToOneAllreduce, " << numRanks << " ranks (" << name << ", n=" << size << ")" << std::endl;
    return print_pass(failed);
}

// test/RingAllreduce.cpp:30-118: every rank keeps one region of its vector accumulating over the runs
template <typename data_t> int ring(const char* name, int numRanks, int size, int num_runs) {
    GaspiEnvironment gaspi_env(1ul << 32);
    gaspi_env.set_rank(0, numRanks);
    gaspi_env.set_blocking(true, 60.0);
    const int tag = 0;
    const std::vector<data_t> values = make_values<data_t>(size);
    std::vector<data_t> gold(size);
    for (int i = 0; i < size; ++i) gold[i] = (data_t)((num_runs * (numRanks - 1) + 1) * values[i]);
    int failed = run_ranks(gaspi_env, numRanks, [&](int myRank) {
        std::vector<data_t> result(values);
        Comprex_RingAllreduce<data_t> allreduce(&gaspi_env);
        allreduce.setupConnections(size, tag, 1e-2f, 3.0f);
        gaspi_env.barrier();
        for (int run = 0; run < num_runs; ++run) {
            gaspi_env.barrier();
            int val_start, val_stop;
            if (myRank < numRanks - 1) {
                val_start = (myRank + 1) * (size / numRanks);
                val_stop = (myRank + 2) * (size / numRanks);
            } else {
                val_start = 0;
                val_stop = size / numRanks;
            }
            for (int it = 0; it < size; ++it) {
                if (it >= val_start && it < val_stop) continue;
                result[it] = values[it];
            }
            allreduce.apply(result.data(), size);
        }
        allreduce.flush(result.data(), size);
        int errors = check(myRank, result, gold);  // every rank holds the exact sum
        gaspi_env.barrier();
        return errors;
    });
    std::cout << "Comprex_RingAllreduce, " << numRanks << " ranks (" << name << ", n=" << size << ")" << std::endl;
    return print_pass(failed);
}

// test/BigRingAllreduce.cpp:30-108
template <typename data_t> int big_ring(const char* name, int numRanks, int size, int num_runs) {
    GaspiEnvironment gaspi_env(1ul << 32);
    gaspi_env.set_rank(0, numRanks);
    gaspi_env.set_blocking(true, 60.0);
    const int chiefRank = 0, tag = 0;
    const std::vector<data_t> values = make_values<data_t>(size);
    std::vector<data_t> gold(size);
    for (int i = 0; i < size; ++i) gold[i] = (data_t)((num_runs * (numRanks - 1) + 1) * values[i]);
    int failed = run_ranks(gaspi_env, numRanks, [&](int myRank) {
        std::vector<data_t> result(values);
        Comprex_BigRingAllreduce<data_t> allreduce(&gaspi_env);
        allreduce.setupConnections(size, tag, 1e-2f, 3.0f);
        gaspi_env.barrier();
        for (int run = 0; run < num_runs; ++run) {
            gaspi_env.barrier();
            if (myRank != chiefRank) result = values;
            allreduce.apply(result.data(), size);
        }
        allreduce.flush(result.data(), size);
        int errors = myRank == chiefRank ? check(myRank, result, gold) : 0;
        gaspi_env.barrier();
        return errors;
    });
    std::cout << "Comprex_BigRingAllreduce, " << numRanks << " ranks (" << name << ", n=" << size << ")" << std::endl;
    return print_pass(failed);
}

int main() {
    if (!need_gpu()) return 77;
    int failed = 0;
    failed += all_to_one<int>("int", 2, 100000, 10);
    failed += all_to_one<int>("int", 4, 100000, 10);
    failed += all_to_one<float>("float", 3, 1000000, 5);
    failed += ring<int>("int", 2, 1000, 10);
    failed += ring<int>("int", 4, 1000, 10);
    failed += ring<float>("float", 5, 100000, 5);
    failed += big_ring<int>("int", 2, 50, 50);
    failed += big_ring<int>("int", 4, 50, 50);
    failed += big_ring<float>("float", 3, 100000, 5);
    return failed ? 1 : 0;
}
