// Mirrors the reference's test/compressor.cpp for CompressorRLE and CompressorIndexPairs:
// compress(threshold 0) then decompress reproduces the input; plus add(), the fused
// compress_add_update and the error paths of src/compressor.hxx:44-51,620-624,645-647.
#include <compressor.hxx>

#include <cstdlib>
#include <vector>

#include "common.hxx"

template <typename data_t> int run(const char* name) {
    int failed = 0;
    const int size = 100;
    std::vector<data_t> values(size);
    for (int i = 0; i < size; ++i) values[i] = (data_t)(i * ((i % 4) / 3) * (1 - 2 * ((i % 6) / 5)));
    int nelem = 0;
    for (auto e : values)
        if (e != 0) ++nelem;
    char buffer[16 * size];

    {  // run-length codec: round trip at threshold 0 (test/compressor.cpp:43-68), then a real threshold
        int errors = 0;
        std::vector<data_t> myValues(values);
        CompressorRLE<data_t> compressor;
        std::cout << "Test CompressorRLE class (" << name << ")." << std::endl;
        const int bytes = compressor.compress(reinterpret_cast<void*>(buffer), myValues.data(), (int)myValues.size(), 0);
        if (bytes != 16 + size * (int)sizeof(data_t) + 4) ++errors;  // every element sent: one run
        std::vector<data_t> out_vec(size, (data_t)7);
        if (compressor.decompress(out_vec.data(), (int)out_vec.size(), reinterpret_cast<void*>(buffer)) != size) ++errors;
        for (int i = 0; i < size; ++i)
            if (out_vec[i] != values[i]) ++errors;
        // |x| >= 50 sent, residual keeps the rest; decompress + residual == input
        std::vector<data_t> rest(values);
        compressor.compress_update(reinterpret_cast<void*>(buffer), rest.data(), size, (data_t)50);
        std::vector<data_t> sent(size + 3, (data_t)7);
        compressor.decompress(sent.data(), size + 3, reinterpret_cast<void*>(buffer));
        for (int i = 0; i < size; ++i) {
            const bool big = std::abs(values[i]) >= (data_t)50;
            if (sent[i] != (big ? values[i] : (data_t)0) || rest[i] != (big ? (data_t)0 : values[i])) ++errors;
        }
        for (int i = size; i < size + 3; ++i)
            if (sent[i] != (data_t)7) ++errors;  // nothing beyond the message's vector is written
        std::vector<data_t> acc(size, (data_t)1);
        compressor.add(acc.data(), size, reinterpret_cast<void*>(buffer));
        for (int i = 0; i < size; ++i)
            if (acc[i] != (data_t)(1 + sent[i])) ++errors;
        try { compressor.decompress(sent.data(), size - 1, reinterpret_cast<void*>(buffer)); ++errors; } catch (const std::runtime_error&) {}
        failed += print_pass(errors);
    }
    {  // round trip  (test/compressor.cpp:70-94)
        int errors = 0;
        std::vector<data_t> myValues(values);
        CompressorIndexPairs<data_t> compressor(0.01);
        std::cout << "Test CompressorIndexPairs class (" << name << "), " << nelem << " non-zeros." << std::endl;
        const int bytes = compressor.compress(reinterpret_cast<void*>(buffer), myValues.data(), (int)myValues.size(), 0);
        if (bytes != 8 + nelem * (4 + (int)sizeof(data_t))) ++errors;
        if (nelem != 25) ++errors;
        std::vector<data_t> out_vec(size, (data_t)7);
        const int consumed = compressor.decompress(out_vec.data(), (int)out_vec.size(), reinterpret_cast<void*>(buffer));
        if (consumed != bytes) ++errors;
        for (int i = 0; i < size; ++i)
            if (out_vec[i] != values[i]) ++errors;
        failed += print_pass(errors);
    }
    {  // add: out += message
        int errors = 0;
        CompressorIndexPairs<data_t> compressor;
        std::vector<data_t> acc(size, (data_t)1);
        compressor.add(acc.data(), size, buffer);
        compressor.add(acc.data(), size, buffer);
        for (int i = 0; i < size; ++i)
            if (acc[i] != (data_t)(1 + 2 * values[i])) ++errors;
        failed += print_pass(errors);
    }
    {  // fused: update += data; |update| > thr emitted and zeroed  (src/compressor.hxx:568-581)
        int errors = 0;
        CompressorIndexPairs<data_t> compressor;
        std::vector<data_t> update(size), data(size);
        for (int i = 0; i < size; ++i) { update[i] = (data_t)(i % 7); data[i] = (data_t)(i % 5 - 2); }
        std::vector<data_t> expect_u(size);
        int k = 0;
        for (int i = 0; i < size; ++i) {
            data_t s = update[i] + data[i];
            if (std::abs(s) > (data_t)4) { ++k; expect_u[i] = 0; } else expect_u[i] = s;
        }
        const int bytes = compressor.compress_add_update(buffer, update.data(), size, data.data(), size, (data_t)4);
        if (bytes != 8 + k * (4 + (int)sizeof(data_t))) ++errors;
        for (int i = 0; i < size; ++i)
            if (update[i] != expect_u[i]) ++errors;
        std::vector<data_t> dec(size);
        compressor.decompress(dec.data(), size, buffer);
        for (int i = 0; i < size; ++i) {
            data_t s = (data_t)(i % 7) + (data_t)(i % 5 - 2);
            if (dec[i] != (std::abs(s) > (data_t)4 ? s : (data_t)0)) ++errors;
        }
        failed += print_pass(errors);
    }
    {  // errors
        int errors = 0;
        CompressorIndexPairs<data_t> compressor;
        std::vector<data_t> a(size), b(size - 1);
        try { compressor.compress_add_update(buffer, a.data(), size, b.data(), size - 1, 0); ++errors; } catch (const std::runtime_error&) {}
        compressor.compress(buffer, values.data(), size, 0);
        std::vector<data_t> small(size - 1, (data_t)5);
        try { compressor.decompress(small.data(), size - 1, buffer); ++errors; } catch (const std::runtime_error&) {}
        for (auto e : small) if (e != 0) ++errors;  // zeroed before the size check
        std::vector<data_t> small2(size - 1, (data_t)5);
        try { compressor.add(small2.data(), size - 1, buffer); ++errors; } catch (const std::runtime_error&) {}
        for (auto e : small2) if (e != 5) ++errors;  // untouched
        failed += print_pass(errors);
    }
    {  // add_many: one pass for several messages == one add() per message, in order
        int errors = 0;
        CompressorIndexPairs<data_t> compressor;
        cxx::Handle copier;
        cxx::DeviceBuffer on_device[3];
        const void* messages[3];
        std::vector<data_t> one_by_one(size), at_once(size);
        for (int i = 0; i < size; ++i) one_by_one[i] = at_once[i] = (data_t)(3 * i - 50);
        for (int m = 0; m < 3; ++m) {
            const int bytes = compressor.compress(buffer, values.data(), size, (data_t)(2 * m));
            cxx::check(cx_copy(copier.get(), on_device[m].reserve((size_t)bytes), buffer, (size_t)bytes));
            messages[m] = on_device[m].data();
            compressor.add(one_by_one.data(), size, buffer);
        }
        compressor.add_many(at_once.data(), size, messages, 3);
        for (int i = 0; i < size; ++i) if (one_by_one[i] != at_once[i]) ++errors;
        std::vector<data_t> small(size - 1, (data_t)5);
        try { compressor.add_many(small.data(), size - 1, messages, 3); ++errors; } catch (const std::runtime_error&) {}
        for (auto e : small) if (e != 5) ++errors;  // untouched
        compressor.add_many(at_once.data(), size, messages, 0);  // nothing to add
        for (int i = 0; i < size; ++i) if (one_by_one[i] != at_once[i]) ++errors;
        std::cout << "add_many (" << name << ")" << std::endl;
        failed += print_pass(errors);
    }
    {  // clones are independent objects that give the same bytes
        int errors = 0;
        CompressorIndexPairs<data_t> compressor;
        Compressor<data_t>* c2 = compressor.clone();
        char buffer2[16 * size];
        const int b1 = compressor.compress(buffer, values.data(), size, 0);
        const int b2 = c2->compress(buffer2, values.data(), size, 0);
        if (b1 != b2 || memcmp(buffer, buffer2, b1) != 0) ++errors;
        delete c2;
        failed += print_pass(errors);
    }
    return failed;
}

int main() {
    if (!need_gpu()) return 77;
    int failed = run<int>("int");
    failed += run<float>("float");
    failed += run<double>("double");
    return failed ? 1 : 0;
}
