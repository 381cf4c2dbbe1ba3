// Exact order statistic of magnitudes on the GPU: the threshold of
// ThresholdTopK<T>::calc_threshold (reference src/threshold.hxx:189-205), i.e. the
// (topk_pos+1)-th largest |x| of the (sub)sampled vector, or max|x| + 1 when topk_pos <= 0.
//
// std::nth_element's result is an order statistic, so any exact selection gives the same
// bits.  Here: most-significant-digit radix select on the magnitude's bit pattern (for
// non-negative IEEE numbers and for |int| the unsigned bit pattern orders like the value),
// 11 bits per pass, digit histograms accumulated in LDS and merged into a global
// histogram with one atomic per non-empty bin and block.
//
// Keys are produced on the fly from the sampling rule of prep_vec / prep_add_vec
// (src/threshold.hxx:208-240): the whole vector, `subsamples` strided positions
// (int)(i * stepsize) with the product in fp32, or a caller-supplied index list; with a
// second vector the key is |vec[p] + add_vec[p]| (one IEEE add, the same bits the
// compressor's `update[i] += data[i]` produces later).
#include "cx_common.hpp"

namespace cx {

namespace {

constexpr int kBlock = 256;

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T x[V]; };

__device__ __forceinline__ uint32_t key_of(float v) { return __float_as_uint(v) & 0x7fffffffu; }
__device__ __forceinline__ uint64_t key_of(double v) {
    return (uint64_t)__double_as_longlong(v) & 0x7fffffffffffffffull;
}
__device__ __forceinline__ uint32_t key_of(int v) { return (uint32_t)(v < 0 ? -v : v); }

__device__ __forceinline__ float value_of(uint32_t k, float) { return __uint_as_float(k); }
__device__ __forceinline__ double value_of(uint64_t k, double) { return __longlong_as_double((long long)k); }
__device__ __forceinline__ int value_of(uint32_t k, int) { return (int)k; }

__global__ __launch_bounds__(kBlock) void select_init_kernel(SelectState* st, unsigned long long rank) {
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) st->hist[b] = 0u;
    if (threadIdx.x == 0) {
        st->prefix = 0ull;
        st->mask = 0ull;
        st->rank = rank;
    }
}

// One histogram pass.  SMODE: 0 whole vector, 1 strided, 2 indexed.
template <typename T, int SMODE, bool HAS_ADD, int VEC>
__global__ __launch_bounds__(kBlock) void select_hist_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                             const int* __restrict__ idx, long long m, int n,
                                                             float stepsize, SelectState* __restrict__ st, int shift,
                                                             int bits) {
    using key_t = typename Elem<T>::key_t;
    __shared__ unsigned lds_hist[kRadixBins];
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) lds_hist[b] = 0u;
    __syncthreads();

    const key_t prefix = (key_t)st->prefix;
    const key_t mask = (key_t)st->mask;
    const unsigned digit_mask = (1u << bits) - 1u;
    const long long stride = (long long)gridDim.x * kBlock;

    if (SMODE == 0 && VEC > 1) {
        const long long nvec = m / VEC;
        for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += stride) {
            Pack<T, VEC> a = reinterpret_cast<const Pack<T, VEC>*>(vec)[i];
            if (HAS_ADD) {
                Pack<T, VEC> b = reinterpret_cast<const Pack<T, VEC>*>(add)[i];
#pragma unroll
                for (int c = 0; c < VEC; ++c) a.x[c] = (T)(a.x[c] + b.x[c]);
            }
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                const key_t k = key_of(a.x[c]);
                if ((k & mask) == prefix) atomicAdd(&lds_hist[(unsigned)(k >> shift) & digit_mask], 1u);
            }
        }
        // tail elements
        for (long long i = nvec * VEC + (long long)blockIdx.x * kBlock + threadIdx.x; i < m; i += stride) {
            T v = vec[i];
            if (HAS_ADD) v = (T)(v + add[i]);
            const key_t k = key_of(v);
            if ((k & mask) == prefix) atomicAdd(&lds_hist[(unsigned)(k >> shift) & digit_mask], 1u);
        }
    } else {
        for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < m; i += stride) {
            long long p;
            if (SMODE == 0) {
                p = i;
            } else if (SMODE == 1) {
                // (int)(i * stepsize), product rounded to fp32 (threshold.hxx:217,236)
                p = (long long)(int)__fmul_rn((float)(int)i, stepsize);
                if (p > (long long)n - 1) p = (long long)n - 1;  // the reference would read out of bounds
                if (p < 0) p = 0;
            } else {
                p = idx[i];
                if (p < 0 || p >= (long long)n) continue;  // ignore positions outside the vector
            }
            T v = vec[p];
            if (HAS_ADD) v = (T)(v + add[p]);
            const key_t k = key_of(v);
            if ((k & mask) == prefix) atomicAdd(&lds_hist[(unsigned)(k >> shift) & digit_mask], 1u);
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) {
        const unsigned c = lds_hist[b];
        if (c) atomicAdd(&st->hist[b], c);
    }
}

// Picks the digit that holds the wanted descending rank, narrows the state, clears the
// histogram for the next pass.  After the last pass the key is complete and the
// threshold is written.  One block.
template <typename T>
__global__ __launch_bounds__(kBlock) void select_pick_kernel(SelectState* st, int shift, int bits, int last,
                                                             int plus_one, T* __restrict__ thr_out) {
    constexpr int kPer = kRadixBins / kBlock;  // bins per thread
    __shared__ unsigned long long s_sum[kBlock];
    __shared__ unsigned s_digit;
    __shared__ unsigned long long s_above;
    const int t = threadIdx.x;
    // thread t owns bins [hi - kPer + 1, hi], walking from the top digit down
    const int hi = kRadixBins - 1 - t * kPer;
    unsigned cnt[kPer];
    unsigned long long local = 0;
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        cnt[q] = st->hist[hi - q];
        local += cnt[q];
    }
    s_sum[t] = local;
    if (t == 0) {
        s_digit = 0u;
        s_above = 0ull;
    }
    __syncthreads();
    // exclusive scan over threads (256 values; serial per thread is cheap enough: one block, once per pass)
    unsigned long long before = 0;
    for (int q = 0; q < t; ++q) before += s_sum[q];
    const unsigned long long rank = st->rank;
    if (rank >= before && rank < before + local) {
        unsigned long long acc = before;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            if (rank < acc + cnt[q]) {
                s_digit = (unsigned)(hi - q);
                s_above = acc;
                break;
            }
            acc += cnt[q];
        }
    }
    __syncthreads();
    for (int b = t; b < kRadixBins; b += kBlock) st->hist[b] = 0u;
    if (t == 0) {
        const unsigned long long digit_mask = ((1ull << bits) - 1ull) << shift;
        const unsigned long long prefix = st->prefix | ((unsigned long long)s_digit << shift);
        st->prefix = prefix;
        st->mask = st->mask | digit_mask;
        st->rank = rank - s_above;
        if (last) {
            using key_t = typename Elem<T>::key_t;
            T v = value_of((key_t)prefix, T());
            if (plus_one) v = (T)(v + 1);
            *thr_out = v;
        }
    }
}

template <typename T> __global__ void set_scalar_kernel(T* out, T v) { *out = v; }

template <typename T, int SMODE, bool HAS_ADD, int VEC>
void launch_hist(cx_handle h, const T* vec, const T* add, const int* idx, long long m, int n, float stepsize, int shift,
                 int bits) {
    const long long per_block = (long long)kBlock * VEC * 8;
    long long blocks = (m + per_block - 1) / per_block;
    if (blocks < 1) blocks = 1;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL((select_hist_kernel<T, SMODE, HAS_ADD, VEC>), dim3((unsigned)blocks), dim3(kBlock), 0, h->stream,
                       vec, add, idx, m, n, stepsize, h->sel, shift, bits);
}

template <typename T, bool HAS_ADD>
void dispatch_hist(cx_handle h, int smode, bool vec_ok, const T* vec, const T* add, const int* idx, long long m, int n,
                   float stepsize, int shift, int bits) {
    constexpr int kVec = 16 / (int)sizeof(T);
    if (smode == kSampleFull) {
        if (vec_ok) launch_hist<T, 0, HAS_ADD, kVec>(h, vec, add, idx, m, n, stepsize, shift, bits);
        else launch_hist<T, 0, HAS_ADD, 1>(h, vec, add, idx, m, n, stepsize, shift, bits);
    } else if (smode == kSampleStrided) {
        launch_hist<T, 1, HAS_ADD, 1>(h, vec, add, idx, m, n, stepsize, shift, bits);
    } else {
        launch_hist<T, 2, HAS_ADD, 1>(h, vec, add, idx, m, n, stepsize, shift, bits);
    }
}

}  // namespace

template <typename T>
int launch_topk_threshold(cx_handle h, const T* vec, const T* add_vec, int n, const int* d_idx, int m, int sample_mode,
                          float stepsize, float topK, T* d_thr_out) {
    if (!d_thr_out) d_thr_out = static_cast<T*>(h->d_thr);
    if (m <= 0) {
        // empty input: undefined in the reference (dereferences end()); defined here as 1
        hipLaunchKernelGGL(set_scalar_kernel<T>, dim3(1), dim3(1), 0, h->stream, d_thr_out, (T)1);
        CX_HIP(hipGetLastError());
        return CX_OK;
    }
    const int pos = cx_topk_pos((size_t)m, topK);
    const int plus_one = pos <= 0 ? 1 : 0;
    unsigned long long rank = plus_one ? 0ull : (unsigned long long)pos;
    if (rank > (unsigned long long)(m - 1)) rank = (unsigned long long)(m - 1);

    const bool vec_ok =
        ((reinterpret_cast<uintptr_t>(vec) | reinterpret_cast<uintptr_t>(add_vec)) & 15u) == 0;  // null add is aligned
    constexpr int kKeyBits = Elem<T>::key_bits;
    constexpr int kPasses = (kKeyBits + kRadixBits - 1) / kRadixBits;

    hipLaunchKernelGGL(select_init_kernel, dim3(1), dim3(kBlock), 0, h->stream, h->sel, rank);
    for (int p = 0; p < kPasses; ++p) {
        int shift = kKeyBits - kRadixBits * (p + 1);
        int bits = kRadixBits;
        if (shift < 0) {
            bits += shift;
            shift = 0;
        }
        if (add_vec)
            dispatch_hist<T, true>(h, sample_mode, vec_ok, vec, add_vec, d_idx, (long long)m, n, stepsize, shift, bits);
        else
            dispatch_hist<T, false>(h, sample_mode, vec_ok, vec, add_vec, d_idx, (long long)m, n, stepsize, shift, bits);
        hipLaunchKernelGGL(select_pick_kernel<T>, dim3(1), dim3(kBlock), 0, h->stream, h->sel, shift, bits,
                           p == kPasses - 1 ? 1 : 0, plus_one, d_thr_out);
    }
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template int launch_topk_threshold<float>(cx_handle, const float*, const float*, int, const int*, int, int, float, float, float*);
template int launch_topk_threshold<double>(cx_handle, const double*, const double*, int, const int*, int, int, float, float, double*);
template int launch_topk_threshold<int>(cx_handle, const int*, const int*, int, const int*, int, int, float, float, int*);

}  // namespace cx
