// Device-side pieces of the radix select shared by the selection kernels (k_select.hip) and by the
// kernels that consume a selection's last histogram themselves (k_compact.hip).
#pragma once

#include "cx_common.hpp"

namespace cx {
namespace {

// magnitude bit patterns: for non-negative IEEE numbers and for |int| the unsigned pattern orders
// like the value
__device__ __forceinline__ uint32_t key_of(float v) { return __float_as_uint(v) & 0x7fffffffu; }
__device__ __forceinline__ uint64_t key_of(double v) {
    return (uint64_t)__double_as_longlong(v) & 0x7fffffffffffffffull;
}
__device__ __forceinline__ uint32_t key_of(int v) { return (uint32_t)(v < 0 ? -v : v); }

__device__ __forceinline__ float value_of(uint32_t k, float) { return __uint_as_float(k); }
__device__ __forceinline__ double value_of(uint64_t k, double) { return __longlong_as_double((long long)k); }
__device__ __forceinline__ int value_of(uint32_t k, int) { return (int)k; }


// Block-wide: digit holding descending rank `rank` in hist[0..kRadixBins), and how many keys
// lie above that digit.  All threads get the result.  A rank beyond the total gives digit 0.
template <int BLOCK>
__device__ __forceinline__ void block_pick(const unsigned* hist, unsigned long long rank, unsigned long long* s_sum,
                                           unsigned* s_digit, unsigned long long* s_above, unsigned& digit,
                                           unsigned long long& above) {
    constexpr int kPer = kRadixBins / BLOCK;  // bins per thread
    const int t = threadIdx.x;
    const int hi = kRadixBins - 1 - t * kPer;  // thread t owns bins [hi - kPer + 1, hi], top digits first
    // a vector holds fewer than 2^31 keys: 32-bit sums are exact, and half the cross-lane traffic
    const unsigned want = rank > 0xffffffffull ? 0xffffffffu : (unsigned)rank;
    unsigned cnt[kPer];
    unsigned local = 0;
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        cnt[q] = hist[hi - q];
        local += cnt[q];
    }
    unsigned incl = local;  // inclusive scan over threads
    const int lane = t & 63, wave = t >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) s_sum[wave] = incl;
    if (t == 0) {
        *s_digit = 0u;
        *s_above = 0ull;
    }
    __syncthreads();
    unsigned before = incl - local;
#pragma unroll
    for (int w = 0; w < BLOCK / 64; ++w) {  // every wavefront reads all the sums at once, not one after the other
        const unsigned sw = (unsigned)s_sum[w];
        before += w < wave ? sw : 0u;
    }
    if (want >= before && want - before < local) {
        unsigned acc = before;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            if (want - acc < cnt[q]) {
                *s_digit = (unsigned)(hi - q);
                *s_above = acc;
                break;
            }
            acc += cnt[q];
        }
    }
    __syncthreads();
    digit = *s_digit;
    above = *s_above;
    __syncthreads();
}


// Shift and width of the digit that radix pass p looks at.
template <typename T> __device__ __forceinline__ void pass_digits_dev(int p, int& shift, int& bits) {
    shift = Elem<T>::key_bits - kRadixBits * (p + 1);
    bits = kRadixBits;
    if (shift < 0) {
        bits += shift;
        shift = 0;
    }
}

// Chained passes without a pick launch in between: pass p leaves its histogram in
// st->pass_hist[p]; every block of the NEXT kernel redoes the cheap pick over it on its own
// (a complete histogram is visible to all of them: it was finished by the previous kernel), so
// no block ever waits for another and no launch is spent on a one-block kernel.
// Returns the state entering pass p (p >= 1): the digits of passes 0..p-1 fixed.  `prev_hist`
// replaces pass p-1's histogram when those counts were made elsewhere.
template <typename T, int BLOCK>
__device__ __forceinline__ PickState state_entering_pass(const SelectState* __restrict__ st, int p,
                                                         unsigned long long rank0,
                                                         unsigned long long* s_sum, unsigned* s_digit,
                                                         unsigned long long* s_above,
                                                         const unsigned* __restrict__ prev_hist = nullptr) {
    PickState s;
    if (p == 1) {
        s.prefix = 0ull;
        s.mask = 0ull;
        s.rank = rank0;
    } else {
        s = st->pass_state[p - 1];
    }
    // every thread reads its own bins straight from the global histogram (through LDS first: 0.3 us more per pick)
    const unsigned* counts = prev_hist ? prev_hist : st->pass_hist[p - 1];
    unsigned digit;
    unsigned long long above;
    block_pick<BLOCK>(counts, s.rank, s_sum, s_digit, s_above, digit, above);
    int shift, bits;
    pass_digits_dev<T>(p - 1, shift, bits);
    s.prefix |= (unsigned long long)digit << shift;
    s.mask |= ((1ull << bits) - 1ull) << shift;
    s.rank -= above;
    return s;
}

}  // namespace
}  // namespace cx
