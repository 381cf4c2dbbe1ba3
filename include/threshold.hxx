// Threshold functions with the interface of the reference's src/threshold.hxx, computed on
// the GPU through the cx_* C ABI.
//
//   ThresholdFunction<T>  base: apply / apply_split / clone / get_threshold / prepare /
//                         prepare_with                       (reference src/threshold.hxx:15-65)
//   ThresholdNone<T>      passes everything, threshold 0      (:72-88)
//   ThresholdConst<T>     constant threshold, rejects < 0     (:96-119)
//   ThresholdTopK<T>      threshold = the (ceil(m*topK)-1)-th largest magnitude of a strided
//                         sub-sample of vec (+ add_vec)        (:127-242)
//
// Vectors may be host or device pointers.  After prepare*/prepare_with the threshold stays on
// the device (device_threshold()) so that a compressor can consume it without a host round
// trip; get_threshold() fetches it when the caller wants the number.
#ifndef THRESHOLD_H
#define THRESHOLD_H

#include <cmath>
#include <memory>
#include <stdexcept>

#include "cx_device.hxx"

template <class VarTYPE>
class ThresholdFunction {
public:
    virtual ~ThresholdFunction() {}

    // out = |in| >= threshold ? in : 0, after prepare(in)
    virtual void apply(VarTYPE* out_vec, int out_vec_size, const VarTYPE* in_vec, int in_vec_size) {
        if (out_vec_size < in_vec_size)
            throw std::runtime_error("Thresholding target buffer is smaller than source buffer!");
        cxx::Scope scope(handle_.ctx());
        prepare(in_vec, in_vec_size);
        run_apply(out_vec, nullptr, in_vec, in_vec_size);
    }

    // high = values at or above the threshold, low = the rest
    virtual void apply_split(VarTYPE* high_vec, int high_vec_size, VarTYPE* low_vec, int low_vec_size,
                             const VarTYPE* in_vec, int in_vec_size) {
        if (high_vec_size < in_vec_size || low_vec_size < in_vec_size)
            throw std::runtime_error("Thresholding target buffer is smaller than source buffer!");
        cxx::Scope scope(handle_.ctx());
        prepare(in_vec, in_vec_size);
        run_apply(high_vec, low_vec, in_vec, in_vec_size);
    }

    virtual ThresholdFunction<VarTYPE>* clone() const = 0;

    virtual VarTYPE get_threshold() = 0;

    virtual void prepare(const VarTYPE* vec, int vec_size) {}

    virtual void prepare_with(const VarTYPE* vec, int vec_size, const VarTYPE* add_vec, int add_vec_size) {}

    // Device address of the current threshold, or nullptr when only the host value exists.
    virtual const VarTYPE* device_threshold() { return nullptr; }
    // Not in the reference: sizes the GPU scratch of this threshold for vectors of up to n elements.
    virtual void reserve(int n) {}
    // Not in the reference: the stream this object's GPU work runs on and the caller's stream it is
    // joined with around every call (cx_device.hxx).  A ComprEx binds its clones to its own.
    void bind_stream(const std::shared_ptr<cxx::StreamCtx>& ctx) { handle_.bind(ctx); }
    cxx::StreamCtx& stream_context() { return handle_.ctx(); }
    void stream_changed() { handle_.refresh(); }

    // Not in the reference.  True when prepare_with on n elements would apply the top-k rule to
    // every element (no sub-sampling); the fraction is returned.  ComprEx then computes threshold
    // and message in one fused call and leaves the threshold where claim_device_threshold() says.
    virtual bool whole_vector_topk(int n, float* topK_out) const { return false; }
    virtual VarTYPE* claim_device_threshold() { return nullptr; }
    // Not in the reference.  The parameters of a top-k threshold (fraction, sub-sampling rule, optional
    // caller-chosen sample positions on the device), for a caller that runs prepare_with and the
    // compression as one call; false for every other kind of threshold.
    struct TopKRule {
        float topK;
        int default_subsamples;
        float subsample_factor;
        const int* d_positions;
        int n_positions;
    };
    virtual bool topk_rule(TopKRule*) const { return false; }

protected:
    virtual bool is_aboveThreshold(const VarTYPE& target) = 0;

    // the masking loop of apply / apply_split on the GPU, '>=' semantics
    virtual void run_apply(VarTYPE* high, VarTYPE* low, const VarTYPE* in, int n) {
        cx_handle h = handle_.get();
        cxx::Staged<const VarTYPE> s_in(h, stage_in_, in, (size_t)n, true, false);
        cxx::Staged<VarTYPE> s_hi(h, stage_hi_, high, (size_t)n, false, true);
        cxx::Staged<VarTYPE> s_lo(h, stage_lo_, low, (size_t)(low ? n : 0), false, true);
        const VarTYPE thr = get_threshold();
        cxx::check(cx_threshold_apply(h, cxx::dtype_of<VarTYPE>::value, s_hi.get(), low ? s_lo.get() : nullptr,
                                      s_in.get(), n, &thr, nullptr));
        s_hi.flush();
        s_lo.flush();
        cxx::check(cx_synchronize(h));
    }

    cxx::Handle handle_;
    cxx::DeviceBuffer stage_in_, stage_hi_, stage_lo_;
};

template <class VarTYPE>
class ThresholdNone : public ThresholdFunction<VarTYPE> {
public:
    ThresholdNone() {}
    ThresholdNone(const ThresholdNone<VarTYPE>&) {}
    virtual ThresholdFunction<VarTYPE>* clone() const { return new ThresholdNone<VarTYPE>(*this); }
    virtual VarTYPE get_threshold() { return 0; }

protected:
    virtual bool is_aboveThreshold(const VarTYPE&) { return true; }
    // everything passes, NaN included: a plain copy (and an all-zero low part)
    virtual void run_apply(VarTYPE* high, VarTYPE* low, const VarTYPE* in, int n) {
        cx_handle h = this->handle_.get();
        cxx::check(cx_copy(h, high, in, (size_t)n * sizeof(VarTYPE)));
        if (low) {
            cxx::Staged<VarTYPE> s_lo(h, this->stage_lo_, low, (size_t)n, false, true);
            cxx::check(cx_zero(h, cxx::dtype_of<VarTYPE>::value, s_lo.get(), n));
            s_lo.flush();
        }
        cxx::check(cx_synchronize(h));
    }
};

template <class VarTYPE>
class ThresholdConst : public ThresholdFunction<VarTYPE> {
public:
    ThresholdConst(VarTYPE threshold) : _threshold(threshold) {
        if (_threshold < 0) throw std::runtime_error("Threshold of ThresholdConst is <0!");
    }
    ThresholdConst(const ThresholdConst<VarTYPE>& other) : _threshold(other._threshold) {}
    virtual ThresholdFunction<VarTYPE>* clone() const { return new ThresholdConst<VarTYPE>(*this); }
    virtual VarTYPE get_threshold() { return _threshold; }

protected:
    VarTYPE _threshold;
    virtual bool is_aboveThreshold(const VarTYPE& target) { return std::abs(target) >= _threshold; }
};

template <class VarTYPE>
class ThresholdTopK : public ThresholdFunction<VarTYPE> {
public:
    ThresholdTopK(float topK, int default_subsamples = 1000, float subsample_factor = 10.0)
        : _threshold(0), on_device_(false), host_valid_(true), sample_m_(0) {
        if (topK > 1.0 || topK < 0.0) throw std::runtime_error("topK value must be between 0.0 and 1.0!");
        this->topK = topK;
        this->default_subsamples = default_subsamples;
        this->subsamples_factor = subsample_factor;
    }

    // a clone carries the configuration (sample positions included) and the last host-visible
    // threshold, with scratch of its own
    ThresholdTopK(const ThresholdTopK<VarTYPE>& other)
        : topK(other.topK), default_subsamples(other.default_subsamples), subsamples_factor(other.subsamples_factor),
          _threshold(const_cast<ThresholdTopK<VarTYPE>&>(other).get_threshold()), on_device_(false),
          host_valid_(true), sample_m_(0) {
        if (other.sample_m_ > 0) set_sample_positions(static_cast<const int*>(other.sample_idx_.data()), other.sample_m_);
    }

    // Not in the reference: prepare / prepare_with take the order statistic over these positions
    // (int32 indices into the vector; host or device pointer, copied) instead of the strided
    // sub-sample; m == 0 returns to the reference's rule.
    void set_sample_positions(const int* idx, int m) {
        sample_m_ = 0;
        if (m <= 0) return;
        if (!idx) throw std::runtime_error("sample positions: null pointer");
        cxx::Scope scope(this->handle_.ctx());
        cx_handle h = this->handle_.get();
        cxx::check(cx_copy(h, sample_idx_.reserve((size_t)m * sizeof(int)), idx, (size_t)m * sizeof(int)));
        cxx::check(cx_synchronize(h));
        sample_m_ = m;
    }

    float getTopK() const { return topK; }

    virtual ThresholdFunction<VarTYPE>* clone() const { return new ThresholdTopK<VarTYPE>(*this); }

    virtual VarTYPE get_threshold() {
        if (!host_valid_) {
            cx_handle h = this->handle_.get();
            cxx::check(cx_copy(h, &_threshold, cx_threshold_slot(h), sizeof(VarTYPE)));
            cxx::check(cx_synchronize(h));
            host_valid_ = true;
        }
        return _threshold;
    }

    virtual const VarTYPE* device_threshold() {
        return on_device_ ? static_cast<const VarTYPE*>(cx_threshold_slot(this->handle_.get())) : nullptr;
    }

    virtual void reserve(int n) {
        cxx::check(cx_reserve(this->handle_.get(), cxx::dtype_of<VarTYPE>::value, n, CX_RESERVE_THRESHOLD));
    }

    // n < subsamples is the reference's test for using the whole vector (src/threshold.hxx:224-231)
    virtual bool whole_vector_topk(int n, float* topK_out) const {
        if (sample_m_ > 0) return false;
        const int subsamples = cx_topk_subsamples(topK, default_subsamples, subsamples_factor);
        if (topK_out) *topK_out = topK;
        return subsamples < 0 || n < subsamples;
    }
    virtual bool topk_rule(typename ThresholdFunction<VarTYPE>::TopKRule* rule) const {
        rule->topK = topK;
        rule->default_subsamples = default_subsamples;
        rule->subsample_factor = subsamples_factor;
        rule->d_positions = sample_m_ > 0 ? static_cast<const int*>(sample_idx_.data()) : nullptr;
        rule->n_positions = sample_m_;
        return true;
    }
    // the slot will hold the threshold once the caller's fused call has run
    virtual VarTYPE* claim_device_threshold() {
        on_device_ = true;
        host_valid_ = false;
        return static_cast<VarTYPE*>(cx_threshold_slot(this->handle_.get()));
    }

    virtual void prepare(const VarTYPE* vec, int vec_size) {
        if (sample_m_ > 0) {
            prepare_indexed(vec, vec_size, nullptr, static_cast<const int*>(sample_idx_.data()), sample_m_);
            return;
        }
        cxx::Scope scope(this->handle_.ctx());
        cx_handle h = this->handle_.get();
        cxx::Staged<const VarTYPE> v(h, this->stage_in_, vec, (size_t)vec_size, true, false);
        cxx::check(cx_topk_threshold(h, cxx::dtype_of<VarTYPE>::value, v.get(), nullptr, vec_size, 0, topK,
                                     default_subsamples, subsamples_factor, nullptr, nullptr));
        on_device_ = true;
        host_valid_ = false;
    }

    virtual void prepare_with(const VarTYPE* vec, int vec_size, const VarTYPE* add_vec, int add_vec_size) {
        if (vec_size != add_vec_size) throw std::runtime_error("vector sizes must be the same!");
        if (sample_m_ > 0) {
            prepare_indexed(vec, vec_size, add_vec, static_cast<const int*>(sample_idx_.data()), sample_m_);
            return;
        }
        cxx::Scope scope(this->handle_.ctx());
        cx_handle h = this->handle_.get();
        cxx::Staged<const VarTYPE> v(h, this->stage_in_, vec, (size_t)vec_size, true, false);
        cxx::Staged<const VarTYPE> a(h, this->stage_hi_, add_vec, (size_t)add_vec_size, true, false);
        cxx::check(cx_topk_threshold(h, cxx::dtype_of<VarTYPE>::value, v.get(), a.get(), vec_size, add_vec_size, topK,
                                     default_subsamples, subsamples_factor, nullptr, nullptr));
        on_device_ = true;
        host_valid_ = false;
    }

    // Not in the reference: the same order statistic over caller-chosen sample positions
    // (device int32 indices).
    void prepare_indexed(const VarTYPE* vec, int vec_size, const VarTYPE* add_vec, const int* d_idx, int m) {
        cxx::Scope scope(this->handle_.ctx());
        cx_handle h = this->handle_.get();
        cxx::Staged<const VarTYPE> v(h, this->stage_in_, vec, (size_t)vec_size, true, false);
        cxx::Staged<const VarTYPE> a(h, this->stage_hi_, add_vec, (size_t)(add_vec ? vec_size : 0), true, false);
        cxx::check(cx_topk_threshold_indexed(h, cxx::dtype_of<VarTYPE>::value, v.get(), add_vec ? a.get() : nullptr,
                                             vec_size, d_idx, m, topK, nullptr, nullptr));
        on_device_ = true;
        host_valid_ = false;
    }

protected:
    float topK;
    int default_subsamples;
    float subsamples_factor;
    VarTYPE _threshold;
    bool on_device_;   // the handle's slot holds the current threshold
    bool host_valid_;  // _threshold mirrors it
    cxx::DeviceBuffer sample_idx_;  // caller-chosen sample positions (device copy), sample_m_ of them
    int sample_m_;

    virtual bool is_aboveThreshold(const VarTYPE& target) { return std::abs(target) >= get_threshold(); }
};

#endif  // THRESHOLD_H
