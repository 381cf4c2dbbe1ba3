// FastComprEx (reference src/comprEx.tpp:366-493) and the forwarders (:248-301) on the GPU against the
// CPU checker (oracle/, test infrastructure): every message that ARRIVES is compared byte for byte,
// and the sender's residual after every call, for the IndexPairs, run-length and dense codecs.
// What the checker's state machine is pinned against: tests/test_oracle_pin.py.
#include <comprEx.hxx>

#include <cstring>
#include <string>
#include <vector>

#include "../../oracle/comprex_oracle.h"
#include "common.hxx"

namespace {

// the protected ends of a channel, for looking at the bytes in flight
template <typename T> struct PeekComprEx : ComprEx<T> {
    using ComprEx<T>::ComprEx;
    std::vector<unsigned char> inbox(size_t bytes) {
        std::vector<unsigned char> out(bytes);
        this->wait_for_message();
        cxx::check(cx_copy(this->handle_.get(), out.data(), this->targ_address(), bytes));
        cxx::check(cx_synchronize(this->handle_.get()));
        return out;
    }
    void drop() { this->targBuff_data->consumed(this->stream()); }
};

struct Lcg {
    unsigned x;
    explicit Lcg(unsigned seed) : x(seed) {}
    int next(int span) { x = x * 1664525u + 1013904223u; return (int)((x >> 8) % (unsigned)span); }
};

// checker-side sender state (see cxo_fast_write_remote_f32)
struct CheckerFast {
    int codec, n, half_bytes;
    std::vector<float> rests;
    std::vector<unsigned char> halves, sent;
    int st[3];
    float thr;
    CheckerFast(int codec, int n) : codec(codec), n(n), half_bytes(64 + n * 16), rests(n, 0.f),
                                    halves(2 * (size_t)half_bytes), sent(half_bytes), thr(0.f) { st[0] = 0; st[1] = 0; st[2] = 1; }
    int write(const std::vector<float>& v, float topK) {
        return cxo_fast_write_remote_f32(codec, rests.data(), n, v.data(), halves.data(), half_bytes, st, &thr, topK, 1000,
                                         10.0f, sent.data());
    }
    int flush() { return cxo_fast_flush_rests_f32(codec, rests.data(), n, halves.data(), half_bytes, st, sent.data()); }
    int same_as(const CheckerFast& o) {
        return cxo_fast_write_remote_same_as_f32(codec, rests.data(), n, halves.data(), half_bytes, st, thr, o.halves.data(),
                                                 o.st, sent.data());
    }
};

int compare(const char* what, int step, const std::vector<unsigned char>& got, const unsigned char* want, int bytes) {
    if (memcmp(got.data(), want, (size_t)bytes) == 0) return 0;
    std::cout << what << ": message of call " << step << " differs (" << bytes << " bytes expected)" << std::endl;
    return 1;
}

template <class Codec> int fast_against_checker(const char* name, int codec) {
    const int n = 5003;
    const float topK = 0.02f;
    int errors = 0;
    GaspiEnvironment env(1 << 24);
    env.set_rank(0, 3);
    FastComprEx<float> a(env.get_segment(), n, 5.0f), b(env.get_segment(), n, 5.0f);
    a.setThreshold(ThresholdTopK<float>(topK)); a.setCompressor(Codec()); a.connectTx(1, 11);
    b.setThreshold(ThresholdTopK<float>(topK)); b.setCompressor(Codec()); b.connectTx(2, 12);
    env.set_rank(1, 3);
    PeekComprEx<float> ra(env.get_segment(), n, 10.0f);
    ra.setCompressor(Codec()); ra.connectRx(0, 11);
    env.set_rank(2, 3);
    PeekComprEx<float> rb(env.get_segment(), n, 10.0f);
    rb.setCompressor(Codec()); rb.connectRx(0, 12);
    env.set_rank(0, 3);

    CheckerFast ca(codec, n), cb(codec, n);
    Lcg rng(77u + (unsigned)codec);
    std::vector<float> v(n), total(n, 0.f), arrived(n, 0.f);
    const std::string script = "WWSWFWSFFWWF";  // W writeRemote, S b.writeRemote_sameAs(a), F flushRests
    for (size_t step = 0; step < script.size(); ++step) {
        const char op = script[step];
        if (op == 'W') {
            for (int i = 0; i < n; ++i) { v[i] = (float)(rng.next(2001) - 1000); total[i] += v[i]; }
            const int bytes = ca.write(v, topK);
            a.writeRemote(v.data(), n);
            errors += compare(name, (int)step, ra.inbox((size_t)bytes), ca.sent.data(), bytes);
            if (step == 0 && codec == 0 && bytes != 8) { std::cout << "first message is not empty" << std::endl; ++errors; }
            ra.readRemote_add(arrived.data(), n);
        } else if (op == 'S') {
            const int bytes = cb.same_as(ca);
            b.writeRemote_sameAs(&a);
            errors += compare(name, (int)step, rb.inbox((size_t)bytes), cb.sent.data(), bytes);
            rb.drop();
        } else {
            const int bytes = ca.flush();
            a.flushRests();
            errors += compare(name, (int)step, ra.inbox((size_t)bytes), ca.sent.data(), bytes);
            ra.readRemote_add(arrived.data(), n);
            for (int i = 0; i < n; ++i)  // conservation (test/comprex.cpp:73-75): everything given so far has arrived
                if (arrived[i] != total[i]) { ++errors; break; }
        }
        const std::vector<float> r = a.getRests();
        if (memcmp(r.data(), ca.rests.data(), (size_t)n * sizeof(float)) != 0) {
            std::cout << name << ": residual after call " << step << " differs" << std::endl;
            ++errors;
        }
    }
    std::cout << "FastComprEx against the checker, every message and the residual (" << name << ")" << std::endl;
    return print_pass(errors);
}

// Forwarders (src/comprEx.tpp:248-301): what rank 1 passes on and what ranks 1 and 2 end up with, all
// expected values from the checker's writeRemote on the same inputs.
int forwarders_against_checker() {
    const int n = 4000;
    const float topK = 0.05f;
    int errors = 0;
    GaspiEnvironment env(1 << 22);
    std::vector<PeekComprEx<float> > c;
    c.reserve(3);
    for (int rank = 0; rank < 3; ++rank) {
        env.set_rank(rank, 3);
        c.emplace_back(env.get_segment(), n, 3.0f, true);
        c[rank].setThreshold(ThresholdTopK<float>(topK));
        c[rank].setCompressor(CompressorIndexPairs<float>());
        c[rank].connectTo((rank + 2) % 3, (rank + 1) % 3, 5);
    }
    Lcg rng(5u);
    std::vector<float> values(n), rests(n, 0.f), sent_dense(n);
    std::vector<unsigned char> buf(4 + 8 + (size_t)n * 8);
    for (int round = 0; round < 3; ++round) {
        for (int i = 0; i < n; ++i) values[i] = (float)(rng.next(401) - 200);
        float thr = 0.f;
        const int bytes = cxo_write_remote_f32(buf.data(), 1, rests.data(), values.data(), n, topK, 1000, 10.0f, &thr);
        std::fill(sent_dense.begin(), sent_dense.end(), 0.f);
        cxo_ip_add_f32(sent_dense.data(), n, buf.data() + 4);
        c[0].writeRemote(values.data(), n);
        std::vector<float> at1(n, 1.f), at2(n, 2.f);
        if (round == 0) {  // receive, pass the compressed message on, decompress
            c[1].readRemote_forward(at1.data(), n);
            errors += compare("readRemote_forward", round, c[2].inbox((size_t)bytes + 4), buf.data(), bytes + 4);
            c[2].readRemote(at2.data(), n);
            for (int i = 0; i < n; ++i) if (at1[i] != sent_dense[i] || at2[i] != sent_dense[i]) { ++errors; break; }
        } else {  // the big ring's hop: copy into the own send buffer, send on, add
            c[1].readRemote_wait();
            c[1].forward_buffer();
            c[1].forward_add(at1.data(), n);
            errors += compare("forward_buffer/forward_add", round, c[2].inbox((size_t)bytes + 4), buf.data(), bytes + 4);
            c[2].readRemote_add(at2.data(), n);
            for (int i = 0; i < n; ++i) if (at1[i] != 1.f + sent_dense[i] || at2[i] != 2.f + sent_dense[i]) { ++errors; break; }
        }
        const std::vector<float> r0 = c[0].getRests();
        if (memcmp(r0.data(), rests.data(), (size_t)n * 4) != 0) ++errors;
    }
    std::cout << "forwarders against the checker's writeRemote" << std::endl;
    return print_pass(errors);
}

// A flush that does not fit its buffer (size_factor 1: 4n bytes for up to 8 + 8n): what fits is sent,
// the rest stays in the residual, the caller is told; a second flush delivers the rest.
int flush_too_large_for_its_buffer() {
    const int n = 3000;
    int errors = 0;
    GaspiEnvironment env(1 << 22);
    env.set_rank(0, 2);
    ComprEx<float> s(env.get_segment(), n, 1.0f);
    s.setThreshold(ThresholdTopK<float>(0.01f)); s.setCompressor(CompressorIndexPairs<float>()); s.connectTx(1, 3);
    FastComprEx<float> f(env.get_segment(), n, 1.0f);
    f.setThreshold(ThresholdTopK<float>(0.01f)); f.setCompressor(CompressorIndexPairs<float>()); f.connectTx(1, 4);
    env.set_rank(1, 2);
    ComprEx<float> r(env.get_segment(), n, 1.0f), rf(env.get_segment(), n, 2.0f);
    r.setCompressor(CompressorIndexPairs<float>()); r.connectRx(0, 3);
    rf.setCompressor(CompressorIndexPairs<float>()); rf.connectRx(0, 4);
    std::vector<float> v(n), got(n, 0.f), gotf(n, 0.f);
    for (int i = 0; i < n; ++i) v[i] = (float)(i % 7 + 1);  // dense: a flush needs 8 + 8n bytes
    s.writeRemote(v.data(), n); r.readRemote_add(got.data(), n);
    f.writeRemote(v.data(), n); rf.readRemote_add(gotf.data(), n);
    int told = 0;
    for (int round = 0; round < 4; ++round) {
        try { s.flushRests(); } catch (const std::runtime_error& e) { ++told; if (!strstr(e.what(), "size_factor")) ++errors; }
        r.readRemote_add(got.data(), n);
    }
    if (told < 1 || told > 3) { std::cout << "ComprEx flush reported " << told << " short messages" << std::endl; ++errors; }
    for (int i = 0; i < n; ++i) if (got[i] != v[i]) { ++errors; break; }
    for (auto e : s.getRests()) if (e != 0) { ++errors; break; }
    told = 0;
    for (int round = 0; round < 4; ++round) {
        try { f.flushRests(); } catch (const std::runtime_error&) { ++told; }
        rf.readRemote_add(gotf.data(), n);
    }
    if (told < 1 || told > 3) { std::cout << "FastComprEx flush reported " << told << " short messages" << std::endl; ++errors; }
    for (int i = 0; i < n; ++i) if (gotf[i] != v[i]) { ++errors; break; }
    for (auto e : f.getRests()) if (e != 0) { ++errors; break; }
    std::cout << "a flush larger than its buffer sends what fits, keeps the rest and says so" << std::endl;
    return print_pass(errors);
}

}  // namespace

int main() {
    if (!need_gpu()) return 77;
    int failed = 0;
    failed += fast_against_checker<CompressorIndexPairs<float> >("IndexPairs", 0);
    failed += fast_against_checker<CompressorRLE<float> >("run-length", 1);
    failed += fast_against_checker<CompressorNone<float> >("dense", 2);
    failed += forwarders_against_checker();
    failed += flush_too_large_for_its_buffer();
    return failed ? 1 : 0;
}
