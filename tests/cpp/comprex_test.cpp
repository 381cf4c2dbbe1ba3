// Mirrors the reference's integration tests with simulated ranks in one process:
//   test/comprex.cpp           2 ranks, 3 x writeRemote + flushRests, gold (num_runs-1)*values
//   test/AllToOneAllreduce.cpp R ranks, chief reduces in rank order then broadcasts,
//                              gold (num_runs*(numRanks-1)+1)*values at the chief after flush
// The rank a call acts as is chosen with GaspiEnvironment::set_rank (the reference gets it from
// gaspi_run).
#include <comprEx.hxx>

#include <map>
#include <vector>

#include "common.hxx"

template <typename data_t> int comprex_p2p(const char* name) {
    const int size = 50;
    const int num_runs = 4;
    const int size_factor = 3;
    const float threshold = 0.1;
    std::vector<data_t> values(size), gold_result(size), result(size, (data_t)0);
    for (int i = 0; i < size; ++i) values[i] = (data_t)(i * (1 - 2 * (i % 2)));
    for (int i = 0; i < size; ++i) gold_result[i] = (data_t)((num_runs - 1) * values[i]);

    GaspiEnvironment env(1 << 28);
    const int tag = 1;
    std::vector<ComprEx<data_t> > cmprex;  // index = rank
    cmprex.reserve(2);
    for (int rank = 0; rank < 2; ++rank) {
        env.set_rank(rank, 2);
        cmprex.emplace_back(env.get_segment(), size, size_factor, true);
        cmprex[rank].setThreshold(ThresholdTopK<data_t>(threshold));
        cmprex[rank].setCompressor(CompressorIndexPairs<data_t>());
        cmprex[rank].connectTo((rank + 1) % 2, (rank + 1) % 2, tag);
    }
    for (int run = 0; run < num_runs; ++run) {
        if (run < num_runs - 1) cmprex[0].writeRemote(values.data(), (int)values.size());
        else cmprex[0].flushRests();
        cmprex[1].readRemote_add(result.data(), (int)result.size());
    }
    int errors = 0;
    for (int i = 0; i < size; ++i)
        if (result[i] != gold_result[i]) {
            std::cout << "Error in [" << i << "]: result: " << result[i] << " gold: " << gold_result[i] << std::endl;
            ++errors;
        }
    std::vector<data_t> rests = cmprex[0].getRests();
    for (auto e : rests) if (e != 0) ++errors;
    std::cout << "ComprEx point to point (" << name << ")" << std::endl;
    return print_pass(errors);
}

// The same conservation gold on a vector large enough for the single-pass whole-vector top-k
// (threshold and message from one pass over residual and data): ThresholdTopK with more
// sub-samples than elements, integer-valued data so that every sum is exact.
int comprex_p2p_large() {
    typedef float data_t;
    const int size = (1 << 23) + 3;
    const int num_runs = 4;
    std::vector<data_t> values(size), result(size, (data_t)0);
    unsigned x = 12345u;
    for (int i = 0; i < size; ++i) {
        x = x * 1664525u + 1013904223u;
        values[i] = (data_t)((int)((x >> 8) % 2000001u) - 1000000);
    }
    GaspiEnvironment env(1 << 30);
    std::vector<ComprEx<data_t> > cmprex;
    cmprex.reserve(2);
    for (int rank = 0; rank < 2; ++rank) {
        env.set_rank(rank, 2);
        cmprex.emplace_back(env.get_segment(), size, 3.0f, true);
        cmprex[rank].setThreshold(ThresholdTopK<data_t>(0.01f, 1 << 24));
        cmprex[rank].setCompressor(CompressorIndexPairs<data_t>());
        cmprex[rank].connectTo((rank + 1) % 2, (rank + 1) % 2, 3);
    }
    int errors = 0;
    for (int run = 0; run < num_runs; ++run) {
        if (run < num_runs - 1) cmprex[0].writeRemote(values.data(), size);
        else cmprex[0].flushRests();
        cmprex[1].readRemote_add(result.data(), size);
        if (run == 0) {  // about one percent of the elements went out (ties at the threshold stay behind)
            long sent = 0;
            for (int i = 0; i < size; ++i) sent += result[i] != 0;
            if (sent < size / 100 - 100 || sent > size / 100) {
                std::cout << "first message carried " << sent << " elements" << std::endl;
                ++errors;
            }
        }
    }
    for (int i = 0; i < size; ++i)
        if (result[i] != (data_t)(num_runs - 1) * values[i]) {
            if (errors < 5) std::cout << "Error in [" << i << "]: result: " << result[i] << std::endl;
            ++errors;
        }
    std::vector<data_t> rests = cmprex[0].getRests();
    for (auto e : rests) if (e != 0) ++errors;
    std::cout << "ComprEx point to point, 8M elements, whole-vector top-k" << std::endl;
    return print_pass(errors);
}

// Conservation gold with a ThresholdTopK that samples caller-chosen positions (cloned into the
// communicator by setThreshold), device-resident gradient.
int comprex_p2p_sample_positions() {
    typedef float data_t;
    const int size = 200003, m = 5000, num_runs = 5;
    std::vector<data_t> values(size), result(size, (data_t)0);
    std::vector<int> pos(m);
    unsigned x = 4242u;
    for (int i = 0; i < size; ++i) {
        x = x * 1664525u + 1013904223u;
        values[i] = (data_t)((int)((x >> 8) % 20001u) - 10000);
    }
    for (int i = 0; i < m; ++i) {
        x = x * 1664525u + 1013904223u;
        pos[i] = (int)((x >> 8) % (unsigned)size);
    }
    GaspiEnvironment env(1 << 28);
    ThresholdTopK<data_t> threshold(0.02f);
    threshold.set_sample_positions(pos.data(), m);
    std::vector<ComprEx<data_t> > cmprex;
    cmprex.reserve(2);
    for (int rank = 0; rank < 2; ++rank) {
        env.set_rank(rank, 2);
        cmprex.emplace_back(env.get_segment(), size, 3.0f, true);
        cmprex[rank].setThreshold(threshold);
        cmprex[rank].setCompressor(CompressorIndexPairs<data_t>());
        cmprex[rank].connectTo((rank + 1) % 2, (rank + 1) % 2, 5);
    }
    void* d_values = nullptr;
    cxx::check(cx_device_alloc(&d_values, (size_t)size * sizeof(data_t)));
    cxx::Handle h;
    cxx::check(cx_copy(h.get(), d_values, values.data(), (size_t)size * sizeof(data_t)));
    int errors = 0;
    for (int run = 0; run < num_runs; ++run) {
        if (run < num_runs - 1) cmprex[0].writeRemote(static_cast<const data_t*>(d_values), size);
        else cmprex[0].flushRests();
        cmprex[1].readRemote_add(result.data(), size);
        if (run == 0) {  // about two percent of the elements went out (the sample decides, not the vector)
            long sent = 0;
            for (int i = 0; i < size; ++i) sent += result[i] != 0;
            if (sent < size / 100 || sent > size / 25) {
                std::cout << "first message carried " << sent << " elements" << std::endl;
                ++errors;
            }
        }
    }
    for (int i = 0; i < size; ++i)
        if (result[i] != (data_t)(num_runs - 1) * values[i]) ++errors;
    cx_device_free(d_values);
    std::cout << "ComprEx point to point, caller-chosen sample positions, device gradient" << std::endl;
    return print_pass(errors);
}

// Comprex_AllToOneAllreduce::apply / flush (reference src/allreduce.tpp:172-237), every rank's
// part executed in the order the data dependencies impose.
template <typename data_t> int all_to_one(const char* name, int numRanks, int size, int num_runs, float ratio) {
    const int chief = 0, tag = 1;
    const int comprexTag = tag * 2 * numRanks, commTag = tag * 2 * numRanks + 1;
    std::vector<data_t> values(size), gold(size);
    for (int i = 0; i < size; ++i) values[i] = (data_t)((i % 97) * (1 - 2 * (i % 2)));
    for (int i = 0; i < size; ++i) gold[i] = (data_t)((num_runs * (numRanks - 1) + 1) * values[i]);

    GaspiEnvironment env(1 << 28);
    FastComprEx<data_t> proto(env.get_segment(), size, 3.0f);
    proto.setThreshold(ThresholdTopK<data_t>(ratio));
    proto.setCompressor(CompressorIndexPairs<data_t>());
    // per rank: its reduce and broadcast communicators, keyed by peer (src/allreduce.tpp:147-170)
    std::vector<std::map<int, FastComprEx<data_t> > > reduce(numRanks), bcast(numRanks);
    for (int rank = 0; rank < numRanks; ++rank) {
        env.set_rank(rank, numRanks);
        if (rank == chief) {
            for (int r = 0; r < numRanks; ++r) {
                if (r == chief) continue;
                reduce[rank][r] = proto;
                reduce[rank][r].connectRx(r, comprexTag + r);
                bcast[rank][r] = proto;
                bcast[rank][r].connectTx(r, commTag + r);
            }
        } else {
            reduce[rank][chief] = proto;
            reduce[rank][chief].connectTx(chief, comprexTag + rank);
            bcast[rank][chief] = proto;
            bcast[rank][chief].connectRx(chief, commTag + rank);
        }
    }
    // test/AllToOneAllreduce.cpp:72-90: the chief's vector accumulates over the runs, the workers
    // start every run from `values`
    std::vector<std::vector<data_t> > result(numRanks, values);
    for (int run = 0; run < num_runs; ++run) {
        for (int rank = 0; rank < numRanks; ++rank)
            if (rank != chief) result[rank] = values;
        // apply(), workers' first half: send own data
        for (int rank = 0; rank < numRanks; ++rank)
            if (rank != chief) reduce[rank][chief].writeRemote(result[rank].data(), size);
        // apply(), chief: reduce in ascending rank order ...
        for (int r = 0; r < numRanks; ++r)
            if (r != chief) reduce[chief][r].readRemote_add(result[chief].data(), size);
        // ... and broadcast: compress once, re-send the same buffer to the others
        int copy_rank = -1;
        for (int r = 0; r < numRanks; ++r) {
            if (r == chief) continue;
            if (copy_rank == -1) { bcast[chief][r].writeRemote(result[chief].data(), size); copy_rank = r; }
            else bcast[chief][r].writeRemote_sameAs(&bcast[chief][copy_rank]);
        }
        // apply(), workers' second half: receive the broadcast
        for (int rank = 0; rank < numRanks; ++rank)
            if (rank != chief) bcast[rank][chief].readRemote(result[rank].data(), size);
    }
    // flush(): workers send their residuals, the chief adds them; no broadcast; everything is reset
    for (int rank = 0; rank < numRanks; ++rank)
        if (rank != chief) reduce[rank][chief].flushRests();
    for (int r = 0; r < numRanks; ++r)
        if (r != chief) reduce[chief][r].readRemote_add(result[chief].data(), size);
    for (int rank = 0; rank < numRanks; ++rank) {
        for (auto& c : reduce[rank]) c.second.resetRests();
        for (auto& c : bcast[rank]) c.second.resetRests();
    }
    const std::vector<data_t>& total = result[chief];
    int errors = 0;
    for (int i = 0; i < size; ++i)
        if (total[i] != gold[i]) {
            if (errors < 5) std::cout << "Error in [" << i << "]: result: " << total[i] << " gold: " << gold[i] << std::endl;
            ++errors;
        }
    std::cout << "All-to-one allreduce over " << numRanks << " simulated ranks (" << name << ", n=" << size << ")" << std::endl;
    return print_pass(errors);
}

// The send variants that leave the residual alone (src/comprEx.tpp:193-222) and the forwarders
// of the ring schedules (:248-301), on a 3-rank chain 0 -> 1 -> 2 with the sizeBytes prefix on.
template <typename data_t> int variants_and_forwarders(const char* name) {
    const int size = 4000;
    int errors = 0;
    std::vector<data_t> values(size);
    for (int i = 0; i < size; ++i) values[i] = (data_t)(((i * 37) % 201 - 100) * ((i % 3) ? 1 : 0));
    GaspiEnvironment env(1 << 20);
    std::vector<ComprEx<data_t> > c;
    c.reserve(3);
    for (int rank = 0; rank < 3; ++rank) {
        env.set_rank(rank, 3);
        c.emplace_back(env.get_segment(), size, 3.0f, true);
        c[rank].setThreshold(ThresholdTopK<data_t>(0.05f, 1 << 13));  // exact top-k
        c[rank].setCompressor(CompressorIndexPairs<data_t>());
        c[rank].connectTo((rank + 2) % 3, (rank + 1) % 3, 5);  // receive from the left, send to the right
    }
    // writeRemote_compressOnly: every non-zero element arrives, residual stays zero
    c[0].writeRemote_compressOnly(values.data(), size);
    std::vector<data_t> got(size, (data_t)9);
    c[1].readRemote(got.data(), size);
    for (int i = 0; i < size; ++i) if (got[i] != values[i]) ++errors;
    for (auto e : c[0].getRests()) if (e != 0) ++errors;
    // writeRemote_NoResidual: threshold from the vector alone; |v| > thr arrives; residual untouched
    ThresholdTopK<data_t> probe(0.05f, 1 << 13);
    probe.prepare(values.data(), size);
    const data_t thr = probe.get_threshold();
    c[0].writeRemote_NoResidual(values.data(), size);
    // rank 1 forwards the compressed message to rank 2 and decompresses it for itself
    std::vector<data_t> at1(size, (data_t)9), at2(size, (data_t)9);
    c[1].readRemote_forward(at1.data(), size);
    c[2].readRemote(at2.data(), size);
    int kept = 0;
    for (int i = 0; i < size; ++i) {
        const data_t want = std::abs(values[i]) > thr ? values[i] : (data_t)0;
        if (want != 0) ++kept;
        if (at1[i] != want || at2[i] != want) ++errors;
    }
    if (kept == 0 || kept > size / 10) ++errors;
    for (auto e : c[0].getRests()) if (e != 0) ++errors;
    // forward_buffer + forward_add (the big ring's hop, src/allreduce.tpp:663-675): rank 1 copies what it
    // received into its own send buffer, sends it on and adds it to its vector
    c[0].writeRemote(values.data(), size);  // residual += values, top 5 % sent
    c[1].readRemote_wait();
    c[1].forward_buffer();
    std::vector<data_t> acc1(size, (data_t)1), acc2(size, (data_t)2);
    c[1].forward_add(acc1.data(), size);
    c[2].readRemote_add(acc2.data(), size);
    std::vector<data_t> rests0 = c[0].getRests();
    for (int i = 0; i < size; ++i) {
        const data_t sent = values[i] - rests0[i];  // what left rank 0
        if (acc1[i] != (data_t)1 + sent || acc2[i] != (data_t)2 + sent) ++errors;
    }
    // addRests / getRests(ptr) / resetRests
    std::vector<data_t> plus(size, (data_t)3), copy(size);
    c[0].addRests(plus.data(), size);
    c[0].getRests(copy.data(), size);
    for (int i = 0; i < size; ++i) if (plus[i] != (data_t)3 + rests0[i] || copy[i] != rests0[i]) ++errors;
    c[0].resetRests();
    for (auto e : c[0].getRests()) if (e != 0) ++errors;
    std::cout << "send variants and forwarders (" << name << ")" << std::endl;
    return print_pass(errors);
}

int error_paths() {
    int errors = 0;
    GaspiEnvironment env(1 << 20);
    env.set_rank(0, 2);
    ComprEx<float> c(env.get_segment(), 16);
    std::vector<float> v(16, 1.0f);
    try { c.writeRemote(v.data(), 16); ++errors; } catch (const std::runtime_error&) {}   // not connected
    try { c.readRemote(v.data(), 16); ++errors; } catch (const std::runtime_error&) {}
    try { c.flushRests(); ++errors; } catch (const std::runtime_error&) {}
    c.setThreshold(ThresholdTopK<float>(0.5f));
    c.setCompressor(CompressorIndexPairs<float>());
    c.connectTo(1, 1, 7);
    try { c.writeRemote(v.data(), 15); ++errors; } catch (const std::runtime_error&) {}   // size mismatch
    try { c.getRests(v.data(), 15); ++errors; } catch (const std::runtime_error&) {}
    try { c.addRests(v.data(), 15); ++errors; } catch (const std::runtime_error&) {}
    try { c.readRemote(v.data(), 16); ++errors; } catch (const std::runtime_error&) {}    // nothing pending
    ComprEx<float> d(env.get_segment(), 16);
    try { c = d; ++errors; } catch (const std::runtime_error&) {}                          // connected object
    std::cout << "ComprEx error paths" << std::endl;
    return print_pass(errors);
}

int main() {
    if (!need_gpu()) return 77;
    int failed = 0;
    failed += comprex_p2p<int>("int");
    failed += comprex_p2p<float>("float");
    failed += comprex_p2p<double>("double");
    failed += comprex_p2p_large();
    failed += comprex_p2p_sample_positions();
    failed += all_to_one<int>("int", 4, 1000, 10, 0.01f);
    failed += all_to_one<float>("float", 3, 100000, 5, 0.001f);
    failed += variants_and_forwarders<int>("int");
    failed += variants_and_forwarders<float>("float");
    failed += error_paths();
    return failed ? 1 : 0;
}
