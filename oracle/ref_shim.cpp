/*
 * ref_shim.cpp -- extern "C" doorway onto the REAL reference headers.
 * TEST INFRASTRUCTURE ONLY.  Compiled only where the reference tree is present
 * (g++ -std=c++14 -O3 -DNDEBUG -I$REF/src), output to oracle/_ref/.  It includes
 * the reference's src/threshold.hxx and src/compressor.hxx where they lie; no
 * reference source is copied.  The exported cxr_* functions take the same
 * arguments as the oracle's cxo_* functions so a test can call both and compare.
 *
 * -DNDEBUG is required: the reference's RLE codec has an inverted assert
 * (src/compressor.hxx:368); IndexPairs does not depend on it.
 */
#include <compressor.hxx>
#include <threshold.hxx>

#include <cstdint>
#include <cstring>
#include <stdexcept>

namespace {

// Opens the protected sub-sample count for inspection (threshold.hxx:182-186).
template <class T>
struct TopKProbe : ThresholdTopK<T> {
    using ThresholdTopK<T>::ThresholdTopK;
    int subsamples_probe() { return this->calc_subsamples(); }
    T threshold_of(std::vector<T>& v) { return this->calc_threshold(v); }
};

} // namespace

extern "C" {

int cxr_calc_subsamples(float topK, int default_subsamples, float subsample_factor) {
    TopKProbe<float> t(topK, default_subsamples, subsample_factor);
    return t.subsamples_probe();
}

#define CXR_DEFINE(SFX, T)                                                                        \
    T cxr_calc_threshold_##SFX(T* vec_copy, size_t m, float topK) {                               \
        TopKProbe<T> t(topK);                                                                     \
        std::vector<T> v(vec_copy, vec_copy + m);                                                 \
        return t.threshold_of(v);                                                                 \
    }                                                                                             \
    T cxr_topk_prepare_##SFX(const T* vec, int n, float topK, int ds, float sf) {                 \
        ThresholdTopK<T> t(topK, ds, sf);                                                         \
        t.prepare(vec, n);                                                                        \
        return t.get_threshold();                                                                 \
    }                                                                                             \
    T cxr_topk_prepare_with_##SFX(const T* vec, int n, const T* add_vec, int add_n, float topK,   \
                                  int ds, float sf, int* err) {                                   \
        if (err) *err = 0;                                                                        \
        ThresholdTopK<T> t(topK, ds, sf);                                                         \
        try { t.prepare_with(vec, n, add_vec, add_n); }                                           \
        catch (const std::runtime_error&) { if (err) *err = 1; return (T)0; }                     \
        return t.get_threshold();                                                                 \
    }                                                                                             \
    /* ThresholdFunction::apply with a constant threshold (ThresholdConst, >=) */                 \
    void cxr_threshold_apply_##SFX(T* out, const T* in, int n, T thr) {                           \
        ThresholdConst<T> t(thr);                                                                 \
        t.apply(out, n, in, n);                                                                   \
    }                                                                                             \
    void cxr_threshold_apply_split_##SFX(T* high, T* low, const T* in, int n, T thr) {            \
        ThresholdConst<T> t(thr);                                                                 \
        t.apply_split(high, n, low, n, in, n);                                                    \
    }                                                                                             \
    /* ThresholdTopK::apply: prepare + >= mask; returns the threshold it used */                  \
    T cxr_topk_apply_##SFX(T* out, const T* in, int n, float topK) {                              \
        ThresholdTopK<T> t(topK);                                                                 \
        t.apply(out, n, in, n);                                                                   \
        return t.get_threshold();                                                                 \
    }                                                                                             \
    int cxr_ip_compress_##SFX(void* out, const T* data, T* update, int n, T thr) {                \
        CompressorIndexPairs<T> c;                                                                \
        if (data && update) return c.compress_add_update(out, update, n, data, n, thr);           \
        if (update) return c.compress_update(out, update, n, thr);                                \
        return c.compress(out, data, n, thr);                                                     \
    }                                                                                             \
    int cxr_ip_compress_add_update_##SFX(void* out, T* update, int un, const T* data, int dn,     \
                                         T thr) {                                                 \
        CompressorIndexPairs<T> c;                                                                \
        try { return c.compress_add_update(out, update, un, data, dn, thr); }                     \
        catch (const std::runtime_error&) { return -2; }                                          \
    }                                                                                             \
    int cxr_ip_decompress_##SFX(T* out, int out_n, const void* in) {                              \
        CompressorIndexPairs<T> c;                                                                \
        try { return c.decompress(out, out_n, in); }                                              \
        catch (const std::runtime_error&) { return -1; }                                          \
    }                                                                                             \
    int cxr_ip_add_##SFX(T* out, int out_n, const void* in) {                                     \
        CompressorIndexPairs<T> c;                                                                \
        try { c.add(out, out_n, in); }                                                            \
        catch (const std::runtime_error&) { return -1; }                                          \
        return 0;                                                                                 \
    }

/* the reference's run-length codec: its decoder and adder on any message, its encoder only
 * where it is sound (every element sent) */
#define CXR_DEFINE_RLE(SFX, T)                                                                    \
    int cxr_rle_compress_##SFX(void* out, const T* data, T* update, int n, T thr) {               \
        CompressorRLE<T> c;                                                                       \
        if (data && update) return c.compress_add_update(out, update, n, data, n, thr);           \
        if (update) return c.compress_update(out, update, n, thr);                                \
        return c.compress(out, data, n, thr);                                                     \
    }                                                                                             \
    int cxr_rle_decompress_##SFX(T* out, int out_n, const void* in) {                             \
        CompressorRLE<T> c;                                                                       \
        try { return c.decompress(out, out_n, in); }                                              \
        catch (const std::runtime_error&) { return -1; }                                          \
    }                                                                                             \
    int cxr_rle_add_##SFX(T* out, int out_n, const void* in) {                                    \
        CompressorRLE<T> c;                                                                       \
        try { c.add(out, out_n, in); }                                                            \
        catch (const std::runtime_error&) { return -1; }                                          \
        return 0;                                                                                 \
    }
/* the reference's dense codec (compressor.hxx:83-151) */
#define CXR_DEFINE_NONE(SFX, T)                                                                   \
    int cxr_none_compress_##SFX(void* out, const T* data, T* update, int n) {                     \
        CompressorNone<T> c;                                                                      \
        try {                                                                                     \
            if (data && update) return c.compress_add_update(out, update, n, data, n, (T)0);      \
            if (update) return c.compress_update(out, update, n, (T)0);                           \
            return c.compress(out, data, n, (T)0);                                                \
        } catch (const std::runtime_error&) { return -1; }                                        \
    }                                                                                             \
    int cxr_none_decompress_##SFX(T* out, int out_n, const void* in) {                            \
        CompressorNone<T> c;                                                                      \
        try { return c.decompress(out, out_n, in); }                                              \
        catch (const std::runtime_error&) { return -1; }                                          \
    }                                                                                             \
    int cxr_none_add_##SFX(T* out, int out_n, const void* in) {                                   \
        CompressorNone<T> c;                                                                      \
        try { c.add(out, out_n, in); }                                                            \
        catch (const std::runtime_error&) { return -1; }                                          \
        return 0;                                                                                 \
    }
CXR_DEFINE_NONE(f32, float)
CXR_DEFINE_NONE(f64, double)
CXR_DEFINE_NONE(i32, int)

CXR_DEFINE_RLE(f32, float)
CXR_DEFINE_RLE(f64, double)
CXR_DEFINE_RLE(i32, int)

CXR_DEFINE(f32, float)
CXR_DEFINE(f64, double)
CXR_DEFINE(i32, int)

/* 1 when the constructor rejects topK (threshold.hxx:131-133), else 0 */
int cxr_topk_ctor_throws(float topK) {
    try { ThresholdTopK<float> t(topK); } catch (const std::runtime_error&) { return 1; }
    return 0;
}
int cxr_const_ctor_throws(float thr) {
    try { ThresholdConst<float> t(thr); } catch (const std::runtime_error&) { return 1; }
    return 0;
}

} // extern "C"
