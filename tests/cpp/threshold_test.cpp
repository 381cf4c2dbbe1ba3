// Mirrors the reference's test/threshold.cpp (same data formula, same checks) on this
// library's ThresholdConst / ThresholdTopK, for int (as the reference) and float.
#include <threshold.hxx>

#include <algorithm>
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
    {  // caller-chosen sample positions: the order statistic of |v[p] + a[p]| over them, also in a clone
        int errors = 0;
        const int n = 5000, m = 700;
        const float topK = 0.05f;
        std::vector<data_t> v(n), a(n);
        std::vector<int> pos(m);
        unsigned x = 99u;
        for (int i = 0; i < n; ++i) {
            x = x * 1664525u + 1013904223u;
            v[i] = (data_t)((int)((x >> 9) % 20001u) - 10000);
            a[i] = (data_t)((int)((x >> 3) % 11u) - 5);
        }
        for (int i = 0; i < m; ++i) {
            x = x * 1664525u + 1013904223u;
            pos[i] = (int)((x >> 8) % (unsigned)n);
        }
        std::vector<data_t> mags(m);
        for (int i = 0; i < m; ++i) mags[i] = (data_t)std::abs((data_t)(v[pos[i]] + a[pos[i]]));
        std::sort(mags.begin(), mags.end(), [](data_t l, data_t r) { return l > r; });
        const data_t gold = mags[(int)(std::ceil((float)m * topK) - 1.0f)];
        ThresholdTopK<data_t> t(topK);
        t.set_sample_positions(pos.data(), m);
        t.prepare_with(v.data(), n, a.data(), n);
        if (t.get_threshold() != gold) ++errors;
        ThresholdFunction<data_t>* c = t.clone();
        c->prepare_with(v.data(), n, a.data(), n);
        if (c->get_threshold() != gold) ++errors;
        delete c;
        t.set_sample_positions(nullptr, 0);  // back to the strided rule: 1000 samples of 5000
        t.prepare_with(v.data(), n, a.data(), n);
        std::vector<data_t> strided(1000);
        const float stepsize = (float)n / 1000.0f;
        for (int i = 0; i < 1000; ++i) {
            const int p = (int)((float)i * stepsize);
            strided[i] = (data_t)std::abs((data_t)(v[p] + a[p]));
        }
        std::sort(strided.begin(), strided.end(), [](data_t l, data_t r) { return l > r; });
        if (t.get_threshold() != strided[(int)(std::ceil(1000.0f * topK) - 1.0f)]) ++errors;
        std::cout << "ThresholdTopK over caller-chosen positions (" << name << ")" << std::endl;
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
