// Mirrors the reference's test/threshold.cpp (same data formula, same checks) on this
// library's ThresholdConst / ThresholdTopK, for int (as the reference) and float.
#include <threshold.hxx>

#include <cmath>
#include <cstdlib>
#include <vector>

#include "common.hxx"

template <typename data_t> int run(const char* name) {
    int failed = 0;
    const int size = 100;
    std::vector<data_t> values(size);
    for (int i = 0; i < size; ++i) values[i] = (data_t)(i * (1 - 2 * (i % 2)));

    {  // ThresholdConst(20): mask == |v| >= 20  (test/threshold.cpp:36-55)
        int errors = 0;
        ThresholdConst<data_t> threshold(20);
        std::cout << "Test ThresholdConst class (" << name << "). threshold: " << threshold.get_threshold() << std::endl;
        std::vector<data_t> out_vec(size);
        threshold.apply(out_vec.data(), (int)out_vec.size(), values.data(), (int)values.size());
        for (int i = 0; i < size; ++i)
            if ((out_vec[i] != 0) != (std::abs(values[i]) >= threshold.get_threshold())) ++errors;
        failed += print_pass(errors);
    }
    {  // ThresholdTopK(0.10): threshold 90, 10 elements  (test/threshold.cpp:58-85)
        int errors = 0;
        ThresholdTopK<data_t> threshold(0.10);
        std::cout << "Test ThresholdTopK class (" << name << ")." << std::endl;
        std::vector<data_t> out_vec(size);
        threshold.apply(out_vec.data(), (int)out_vec.size(), values.data(), (int)values.size());
        int nelem = 0;
        for (auto e : out_vec)
            if (e != 0) ++nelem;
        std::cout << "threshold: " << threshold.get_threshold() << " #elements: " << nelem << std::endl;
        if (threshold.get_threshold() != (data_t)90) ++errors;
        if (nelem != 10) ++errors;
        for (int i = 0; i < size; ++i)
            if ((out_vec[i] != 0) != (std::abs(values[i]) >= threshold.get_threshold())) ++errors;
        failed += print_pass(errors);
    }
    {  // apply_split: high + low == input, high holds the |v| >= thr part  (src/threshold.hxx:30-50)
        int errors = 0;
        ThresholdConst<data_t> threshold(33);
        std::vector<data_t> hi(size), lo(size);
        threshold.apply_split(hi.data(), size, lo.data(), size, values.data(), size);
        for (int i = 0; i < size; ++i) {
            const bool keep = std::abs(values[i]) >= (data_t)33;
            if (hi[i] != (keep ? values[i] : (data_t)0) || lo[i] != (keep ? (data_t)0 : values[i])) ++errors;
        }
        failed += print_pass(errors);
    }
    {  // error behaviour: target smaller than source, bad topK, negative constant
        int errors = 0;
        ThresholdConst<data_t> threshold(1);
        std::vector<data_t> small(size - 1);
        try { threshold.apply(small.data(), (int)small.size(), values.data(), size); ++errors; } catch (const std::runtime_error&) {}
        try { ThresholdTopK<data_t> t(1.5f); ++errors; } catch (const std::runtime_error&) {}
        try { ThresholdTopK<data_t> t(-0.1f); ++errors; } catch (const std::runtime_error&) {}
        try { ThresholdConst<data_t> t((data_t)-1); ++errors; } catch (const std::runtime_error&) {}
        ThresholdTopK<data_t> t(0.1f);
        try { t.prepare_with(values.data(), size, values.data(), size - 1); ++errors; } catch (const std::runtime_error&) {}
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
