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
#include "cx_select_dev.hpp"

#include <cmath>

namespace cx {

namespace {

constexpr int kBlock = 256;

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T x[V]; };

// ---- pieces shared by the selection kernels ------------------------------------------------
// Digit count into an LDS histogram.  The keys a wavefront looks at together often share one
// digit (candidates just above a bound, samples of one exponent): those are counted with ONE
// atomic.  Must be called by whole wavefronts.
__device__ __forceinline__ void hist_add(unsigned* lds_hist, bool active, unsigned digit) {
    const unsigned long long act = __ballot(active);
    if (act == 0ull) return;
    const int leader = __ffsll((long long)act) - 1;
    const unsigned d0 = __shfl(digit, leader, 64);
    const unsigned long long same = __ballot(active && digit == d0);
    if ((int)(threadIdx.x & 63) == leader) atomicAdd(&lds_hist[d0], (unsigned)__popcll(same));
    if (active && digit != d0) atomicAdd(&lds_hist[digit], 1u);
}

// Adds a block's LDS digit counts to the global histogram.
template <int BLOCK> __device__ __forceinline__ void merge_hist(const unsigned* lds_hist, SelectState* st) {
    __syncthreads();
    for (int b = threadIdx.x; b < kRadixBins; b += BLOCK) {
        const unsigned c = lds_hist[b];
        if (c) atomicAdd(&st->hist[b], c);
    }
}

// Last step of the chained passes: the pick over the last pass's histogram completes the key; the
// threshold is written and the passes' histograms are cleared for the next run.  One block.
// (Folding a pick into the histogram kernel, with the block that arrives last doing it, was measured
// slower on this GPU: the device-scope fences that make the other blocks' counts visible inside one
// kernel cost more than a launch.  Chaining does without: see state_entering_pass.)
template <typename T>
__global__ __launch_bounds__(kBlock) void select_final_kernel(SelectState* st, unsigned long long rank0, int plus_one,
                                                              T* __restrict__ thr_out) {
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    using key_t = typename Elem<T>::key_t;
    __shared__ unsigned s_digit;
    __shared__ unsigned long long s_above, s_sum[kBlock / 64];
    const PickState done = state_entering_pass<T, kBlock>(st, kPasses, rank0, s_sum, &s_digit, &s_above);
    if (threadIdx.x == 0) {
        T v = value_of((key_t)done.prefix, T());
        if (plus_one) v = (T)(v + 1);
        *thr_out = v;
    }
    for (int b = threadIdx.x; b < (kPasses + 1) * kRadixBins; b += kBlock) (&st->pass_hist[0][0])[b] = 0u;
}

// One histogram pass over the keys described by (vec, add, idx).  SMODE: 0 whole vector,
// 1 strided, 2 indexed.  The first `nblocks` blocks of the grid share the keys; the others leave.
// Keys into the block's histogram.  Zero keys are counted in a register and go in once per wavefront:
// the zeros of a sparse gradient would otherwise queue up 64 deep on one LDS address (three passes over
// 2^20 zeros: 37 us against 22 us for normal data; over 10^8: 1.0 ms against 0.48 ms; with this 21 us and
// 0.23 ms, and vectors of 90 % zeros 20 us and 0.23 ms against 25 us and 0.47 ms).  It costs normal data
// 1.2 us per selection of 2^20 keys.  Measured alternatives on 2^20 normal keys: a wavefront's equal
// digits put together with ballots +4 us per selection, a thread's equal digits in a row as one atomic
// +2.5 us.
struct DigitCounter {
    unsigned zeros = 0u;
    template <typename KEY>
    __device__ __forceinline__ void count(unsigned* lds_hist, bool counted, KEY key, unsigned digit) {
        zeros += (counted && key == (KEY)0) ? 1u : 0u;
        if (counted && key != (KEY)0) atomicAdd(&lds_hist[digit], 1u);
    }
    // every lane of the wavefront must call this
    __device__ __forceinline__ void flush(unsigned* lds_hist) {
        unsigned z = zeros;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) z += __shfl_xor(z, off, 64);
        if ((threadIdx.x & 63) == 0 && z) atomicAdd(&lds_hist[0], z);
        zeros = 0u;
    }
};

// Loads in flight per thread and threads per block of select_hist_kernel.  Measured as three chained passes
// over r + g, normal data, 2^18 / 2^20 / 2^22 / 10^8 keys: one load at a time, 256 threads 19.3 / 26.4 / 40.9 /
// 464 us; four loads, 256 threads 19.7 / 23.9 / 36.0 / 489; four loads, 512 threads 19.0 / 22.3 / 32.8 / 469;
// four loads, 1024 threads 18.1 / 21.6 / 30.4 / 439 (a pass with about 128 blocks leaves a SIMD one wavefront of
// 256-thread blocks, and its arithmetic between the LDS atomics is then exposed); eight loads: no better.
constexpr int kHistUnroll = 4;
constexpr int kHistBlock = 1024;

template <typename T, int SMODE, bool HAS_ADD, int VEC, int BLOCK>
__device__ __forceinline__ void hist_pass(const T* __restrict__ vec, const T* __restrict__ add,
                                          const int* __restrict__ idx, long long m, int n, float stepsize,
                                          SelectState* __restrict__ st, int p, unsigned long long rank0,
                                          unsigned nblocks, const unsigned* __restrict__ prev_hist = nullptr,
                                          typename Elem<T>::key_t* __restrict__ keys_out = nullptr) {
    using key_t = typename Elem<T>::key_t;
    __shared__ unsigned lds_hist[kRadixBins];
    __shared__ unsigned s_digit;
    __shared__ unsigned long long s_above, s_sum[BLOCK / 64];
    if (blockIdx.x >= nblocks) return;
    // chained passes: every block redoes the cheap pick over the previous pass's complete histogram
    // (issuing the first round of loads before the pick was measured: 0.1 to 0.2 us per step on 61 706 and
    // on 2^20 elements, not kept)
    PickState s;
    s.prefix = 0ull;
    s.mask = 0ull;
    s.rank = rank0;
    if (p > 0) {
        s = state_entering_pass<T, BLOCK>(st, p, rank0, s_sum, &s_digit, &s_above, prev_hist);
        if (blockIdx.x == 0 && threadIdx.x == 0) st->pass_state[p] = s;
    }
    for (int b = threadIdx.x; b < kRadixBins; b += BLOCK) lds_hist[b] = 0u;
    __syncthreads();

    const key_t prefix = (key_t)s.prefix;
    const key_t mask = (key_t)s.mask;
    int shift, bits;
    pass_digits_dev<T>(p, shift, bits);
    const unsigned digit_mask = (1u << bits) - 1u;
    const long long stride = (long long)nblocks * BLOCK;
    DigitCounter run;

    if (SMODE == 0 && VEC > 1) {
        const long long nvec = m / VEC;
        long long i = (long long)blockIdx.x * BLOCK + threadIdx.x;
        // kHistUnroll rounds of loads in flight per thread
        for (; i + (kHistUnroll - 1) * stride < nvec; i += kHistUnroll * stride) {
            Pack<T, VEC> x[kHistUnroll], y[kHistUnroll];
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u) {
                x[u] = reinterpret_cast<const Pack<T, VEC>*>(vec)[i + u * stride];
                if (HAS_ADD) y[u] = reinterpret_cast<const Pack<T, VEC>*>(add)[i + u * stride];
            }
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u) {
#pragma unroll
                for (int c = 0; c < VEC; ++c) {
                    const T v = HAS_ADD ? (T)(x[u].x[c] + y[u].x[c]) : x[u].x[c];
                    const key_t k = key_of(v);
                    run.count(lds_hist, (k & mask) == prefix, k, (unsigned)(k >> shift) & digit_mask);
                }
            }
        }
        for (; i < nvec; i += stride) {
            Pack<T, VEC> x = reinterpret_cast<const Pack<T, VEC>*>(vec)[i];
            if (HAS_ADD) {
                Pack<T, VEC> y = reinterpret_cast<const Pack<T, VEC>*>(add)[i];
#pragma unroll
                for (int c = 0; c < VEC; ++c) x.x[c] = (T)(x.x[c] + y.x[c]);
            }
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                const key_t k = key_of(x.x[c]);
                run.count(lds_hist, (k & mask) == prefix, k, (unsigned)(k >> shift) & digit_mask);
            }
        }
        // tail elements
        for (long long i = nvec * VEC + (long long)blockIdx.x * BLOCK + threadIdx.x; i < m; i += stride) {
            T v = vec[i];
            if (HAS_ADD) v = (T)(v + add[i]);
            const key_t k = key_of(v);
            run.count(lds_hist, (k & mask) == prefix, k, (unsigned)(k >> shift) & digit_mask);
        }
    } else {
        // where key i is read from
        auto position = [&](long long i, bool& ok) -> long long {
            long long p;
            ok = true;
            if (SMODE == 0) {
                p = i;
            } else if (SMODE == 1) {
                // (int)(i * stepsize), product rounded to fp32 (threshold.hxx:217,236)
                p = (long long)(int)__fmul_rn((float)(int)i, stepsize);
                if (p > (long long)n - 1) p = (long long)n - 1;  // the reference would read out of bounds
                if (p < 0) p = 0;
            } else {
                p = idx[i];
                ok = p >= 0 && p < (long long)n;  // positions outside the vector count as magnitude 0
                if (!ok) p = 0;
            }
            return p;
        };
        long long i = (long long)blockIdx.x * BLOCK + threadIdx.x;
        // kHistUnroll keys' dependent loads (position, then the values there) in flight per thread
        for (; i + (kHistUnroll - 1) * stride < m; i += kHistUnroll * stride) {
            long long p[kHistUnroll];
            bool ok[kHistUnroll];
            T v[kHistUnroll];
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u) p[u] = position(i + u * stride, ok[u]);
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u) {
                v[u] = vec[p[u]];
                if (HAS_ADD) v[u] = (T)(v[u] + add[p[u]]);
            }
#pragma unroll
            for (int u = 0; u < kHistUnroll; ++u) {
                const key_t k = ok[u] ? key_of(v[u]) : (key_t)0;
                if (keys_out) keys_out[i + u * stride] = k;
                run.count(lds_hist, (k & mask) == prefix, k, (unsigned)(k >> shift) & digit_mask);
            }
        }
        for (; i < m; i += stride) {
            bool ok;
            const long long p = position(i, ok);
            T v = vec[p];
            if (HAS_ADD) v = (T)(v + add[p]);
            const key_t k = ok ? key_of(v) : (key_t)0;
            if (keys_out) keys_out[i] = k;
            run.count(lds_hist, (k & mask) == prefix, k, (unsigned)(k >> shift) & digit_mask);
        }
    }
    run.flush(lds_hist);
    __syncthreads();
    for (int b = threadIdx.x; b < kRadixBins; b += BLOCK) {
        const unsigned c = lds_hist[b];
        if (c) atomicAdd(&st->pass_hist[p][b], c);
    }
}

template <typename T, int SMODE, bool HAS_ADD, int VEC>
__global__ __launch_bounds__(kHistBlock) void select_hist_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                                 const int* __restrict__ idx, long long m, int n,
                                                                 float stepsize, SelectState* __restrict__ st, int p,
                                                                 unsigned long long rank0,
                                                                 typename Elem<T>::key_t* __restrict__ keys_out) {
    hist_pass<T, SMODE, HAS_ADD, VEC, kHistBlock>(vec, add, idx, m, n, stepsize, st, p, rank0, gridDim.x, nullptr, keys_out);
}

// The same pass where the DEVICE decides what is counted: the *cand_count candidate keys (magnitude bit
// patterns, i.e. a vector of |x|) when they hold the wanted rank and all fit their buffer, the whole
// vector(s) otherwise.  Every pass of a selection reads the same count and decides alike, so the
// host launches the passes without knowing which way they go.  The grid is sized for the whole
// vector; over the candidates only the blocks they need stay, and pass 0 has nothing to do: the
// kernel that collected them left their top-digit counts behind the last pass's histogram.
// Threads of a block of select_hist_either_kernel and 16-byte loads per thread over the candidates.  Measured as
// the whole threshold call on 12 M / 32 Mi / 10^8 elements at 1 %: 256 x 8 loads 56 / 79 / 156 us, 256 x 4: 54 / 79 /
// 159, 512 x 4: 54 / 78 / 156, 1024 x 2: 54 / 79 / 157, 1024 x 8: 58 / 82 / 157 (nothing to choose between them).
constexpr int kEitherBlock = 256;
constexpr unsigned kEitherLoads = 8u;

template <typename T, bool HAS_ADD, int VEC>
__global__ __launch_bounds__(kEitherBlock) void select_hist_either_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                                    long long m,
                                                                    const typename Elem<T>::key_t* __restrict__ cand,
                                                                    unsigned cap, const unsigned* __restrict__ cand_count,
                                                                    SelectState* __restrict__ st, int p,
                                                                    unsigned long long rank0) {
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    const unsigned count = *cand_count;
    if ((unsigned long long)count > rank0 && count <= cap) {
        if (p == 0) return;
        constexpr unsigned kPerBlock = (unsigned)kEitherBlock * VEC * kEitherLoads;
        unsigned need = (count + kPerBlock - 1u) / kPerBlock;
        if (need > gridDim.x) need = gridDim.x;
        hist_pass<T, 0, false, VEC, kEitherBlock>(reinterpret_cast<const T*>(cand), nullptr, nullptr, (long long)count, (int)count, 1.0f,
                                    st, p, rank0, need, p == 1 ? st->pass_hist[kPasses] : nullptr);
    } else {
        hist_pass<T, 0, HAS_ADD, VEC, kEitherBlock>(vec, add, nullptr, m, (int)m, 1.0f, st, p, rank0, gridDim.x);
    }
}

// One histogram pass over the values of an IndexPairs message (int32 n | int32 k | k pairs), whose
// pair count is only known on the device; at most `cap` pairs are looked at.
template <typename T> __device__ __forceinline__ typename Elem<T>::key_t pair_key(const unsigned* w);
template <> __device__ __forceinline__ uint32_t pair_key<float>(const unsigned* w) { return w[1] & 0x7fffffffu; }
template <> __device__ __forceinline__ uint32_t pair_key<int>(const unsigned* w) { return key_of((int)w[1]); }
template <> __device__ __forceinline__ uint64_t pair_key<double>(const unsigned* w) {
    return ((uint64_t)w[1] | ((uint64_t)w[2] << 32)) & 0x7fffffffffffffffull;
}

// Threads and blocks of select_hist_pairs_kernel: every block merges its histogram with global atomics, so few
// large blocks.  Measured as the whole single-pass call on 25.6 M elements at 0.1 % / 1 % and on 10^8 at 1 %:
// 256 x 256 threads 113.4 / 121.9 / 276.4 us, 64 x 1024 110.1 / 117.5 / 270.6, 128 x 1024 109.3 / 115.5 / 265.3,
// 128 x 512 109.2 / 117.7 / 271.9, 32 x 1024 110.1 / 121.2 / 287.0.
constexpr int kPairsBlock = 1024;
constexpr int kPairsBlocks = 128;

template <typename T>
__global__ __launch_bounds__(kPairsBlock) void select_hist_pairs_kernel(const unsigned* __restrict__ msg_words, unsigned cap,
                                                                   SelectState* __restrict__ st, int p,
                                                                   unsigned long long rank0) {
    using key_t = typename Elem<T>::key_t;
    constexpr int PW = Elem<T>::pair_words;
    __shared__ unsigned lds_hist[kRadixBins];
    __shared__ unsigned s_digit;
    __shared__ unsigned long long s_above, s_sum[kPairsBlock / 64];
    PickState s;
    s.prefix = 0ull;
    s.mask = 0ull;
    s.rank = rank0;
    if (p > 0) {
        s = state_entering_pass<T, kPairsBlock>(st, p, rank0, s_sum, &s_digit, &s_above);
        if (blockIdx.x == 0 && threadIdx.x == 0) st->pass_state[p] = s;
    }
    for (int b = threadIdx.x; b < kRadixBins; b += kPairsBlock) lds_hist[b] = 0u;
    __syncthreads();
    const key_t prefix = (key_t)s.prefix;
    const key_t mask = (key_t)s.mask;
    int shift, bits;
    pass_digits_dev<T>(p, shift, bits);
    const unsigned digit_mask = (1u << bits) - 1u;
    unsigned m = msg_words[1];
    if (m > cap) m = cap;
    const unsigned stride = gridDim.x * kPairsBlock;
    // whole wavefronts stay in the loop together (hist_add is a cross-lane operation); four
    // independent loads per lane are in flight before the first count
    for (unsigned i0 = blockIdx.x * kPairsBlock; i0 < m; i0 += 4u * stride) {
        key_t k[4];
        bool in[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const unsigned i = i0 + (unsigned)q * stride + threadIdx.x;
            in[q] = i < m;  // m <= cap < 2^31 / 4: the index cannot wrap
            k[q] = in[q] ? pair_key<T>(msg_words + 2 + (size_t)i * PW) : (key_t)0;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
            hist_add(lds_hist, in[q] && (k[q] & mask) == prefix, (unsigned)(k[q] >> shift) & digit_mask);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < kRadixBins; b += kPairsBlock) {
        const unsigned c = lds_hist[b];
        if (c) atomicAdd(&st->pass_hist[p][b], c);
    }
}

// ---- up to 2^18 keys: two launches --------------------------------------------------------
// First launch: every block gathers one key per thread, stores it to `keys` and counts its top
// digit in LDS.  Second launch, one block: picks the digits alone, in LDS as soon as the keys
// still in play fit there.
//
// One block has the instruction throughput and the memory bandwidth of one compute unit
// (measured: about 50 GB/s, 7 us per 100 000 four-byte keys), so the second launch must not read
// every key.  When the wanted key is near the top, each block of the first launch passes on a
// SHORT LIST: its keys from the top digit of its own short_k-th largest key upwards (all its keys
// when it has fewer), and the largest such digit over all blocks is recorded.  The list holds
// EVERY key whose top digit is at least that one, so when more such keys exist than the wanted
// rank, the answer is found from the list alone.  Otherwise (large keys clustered in a few
// blocks, ties, keys that all share their top digit so that the list overflows) the second launch
// starts from the top-digit counts of ALL keys, which every block of the first launch adds to the
// global histogram either way (leaving that out made the first launch 0.7 us faster and this
// case 60 us slower: the one block would have to count every key again), and reads the key array.
//
// One launch, with the block that finishes last doing the second launch's work, was measured
// slower (30 us against 25): making the other blocks' keys visible inside one kernel takes a
// device-wide release per block and an acquire in the last one, and on this GPU those write back
// and invalidate the L2 of the block's XCD (0.5 to 1.2 us and 2.5 us; 30 us more with a fence in
// every thread), which is what the launch boundary does anyway.
// threads per block of the first launch, one key each.  Measured, threshold + compress: 256 / 512 / 1024
// threads give 0.213 / 0.207 / 0.208 ms on 100 M elements with 100 000 sampled positions and 39 / 44 / 42 us
// on all of 61 706 elements.
constexpr int kFirstBlock = 1024;
constexpr int kFinishBlock = 1024;
constexpr int kListBytes = 49152;           // LDS list of the last block
constexpr int kShortGlobalKeys = 1 << 16;   // capacity of the short list in device memory
// Largest key count of this path.  Four keys per thread and 2^20 keys were measured too: no faster
// than three histogram passes over the vector (63 vs 68 us at 2^20 keys), and the last block's
// worst case (no usable short list: it reads every key, up to three times) grows with the key count.
constexpr int kSmallSelect = 1 << 18;

// One block walks `count` keys that start on a 16-byte boundary and hands every key that still
// matches the fixed digits to `hit`.  Written for one compute unit: sixteen 16-byte loads per lane
// are in flight per round (a round trip to memory per round, not per key), and the test costs two
// instructions per key.
template <typename KEY, typename HIT>
__device__ __forceinline__ void scan_matching(const KEY* src, unsigned count, KEY prefix, KEY mask, HIT hit) {
    constexpr int KV = 16 / (int)sizeof(KEY);  // keys per 16-byte load
    constexpr int kLoads = 16;
    const int t = threadIdx.x;
    const Pack<KEY, KV>* kv = reinterpret_cast<const Pack<KEY, KV>*>(src);
    const int nfull = (int)(count / KV);
    for (int v0 = 0; v0 < nfull; v0 += kFinishBlock * kLoads) {
        Pack<KEY, KV> kk[kLoads];
#pragma unroll
        for (int q = 0; q < kLoads; ++q) {
            const int v = v0 + q * kFinishBlock + t;
            if (v < nfull) {
                kk[q] = kv[v];
            } else {
#pragma unroll
                for (int c = 0; c < KV; ++c) kk[q].x[c] = (KEY)0;
            }
        }
#pragma unroll
        for (int q = 0; q < kLoads; ++q) {
            bool any = false;
#pragma unroll
            for (int c = 0; c < KV; ++c) any |= (kk[q].x[c] & mask) == prefix;
            if (any && v0 + q * kFinishBlock + t < nfull) {  // (an empty mask matches the padding too)
#pragma unroll
                for (int c = 0; c < KV; ++c)
                    if ((kk[q].x[c] & mask) == prefix) hit(kk[q].x[c]);
            }
        }
    }
    for (unsigned i = (unsigned)nfull * KV + t; i < count; i += kFinishBlock) {  // fewer than KV keys
        const KEY k1 = src[i];
        if ((k1 & mask) == prefix) hit(k1);
    }
}

template <typename T, int SMODE, bool HAS_ADD>
__global__ __launch_bounds__(kFirstBlock) void select_first_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                              const int* __restrict__ idx, int m, int n, float stepsize,
                                                              typename Elem<T>::key_t* __restrict__ keys,
                                                              SelectState* __restrict__ st, int short_k,
                                                              typename Elem<T>::key_t* __restrict__ short_keys,
                                                              unsigned short_cap) {
    using key_t = typename Elem<T>::key_t;
    constexpr int shift0 = Elem<T>::key_bits - kRadixBits;
    constexpr int shift1 = Elem<T>::key_bits - 2 * kRadixBits;
    constexpr unsigned kDigitMask = (1u << kRadixBits) - 1u;
    __shared__ unsigned lds_hist[kRadixBins];
    __shared__ unsigned s_digit, s_base, s_wave[kFirstBlock / 64];
    __shared__ unsigned long long s_above, s_sum[kFirstBlock / 64];
    const int t = threadIdx.x;
    const bool short_on = short_k > 0;

    // ---- every block: gather, count, pass on
    for (int b = t; b < kRadixBins; b += kFirstBlock) lds_hist[b] = 0u;
    __syncthreads();
    // the grid covers m; whole wavefronts take every step together (hist_add is a cross-lane operation)
    // The keys are dealt out to the blocks 64 at a time, in turn (wavefront w of block b takes keys
    // [(w * blocks + b) * 64, + 64)): a block that took 1024 consecutive keys or samples would see one stretch
    // of the vector, and where stretches differ in scale (the layers of a network) the blocks' short lists,
    // sized for an even share of the large keys, could not decide (25.6 M elements in layers, 65 536 strided
    // samples: the second launch 12.1 us, with the keys dealt out 5.9 us).  A wavefront's keys, positions
    // and stores stay consecutive.
    const long long i = ((long long)(t >> 6) * gridDim.x + blockIdx.x) * 64 + (t & 63);
    key_t mine = 0;
    const bool have = i < m;
    if (have) {
        long long p;
        bool ok = true;
        if (SMODE == 0) {
            p = i;
        } else if (SMODE == 1) {
            p = (long long)(int)__fmul_rn((float)(int)i, stepsize);  // (int)(i * stepsize), product in fp32
            if (p > (long long)n - 1) p = (long long)n - 1;          // the reference would read out of bounds
            if (p < 0) p = 0;
        } else {
            p = idx[i];
            ok = p >= 0 && p < (long long)n;  // positions outside the vector count as magnitude 0
            if (!ok) p = 0;
        }
        T v = vec[p];
        if (HAS_ADD) v = (T)(v + add[p]);
        mine = ok ? key_of(v) : (key_t)0;
        keys[i] = mine;
    }
    hist_add(lds_hist, have, (unsigned)(mine >> shift0) & kDigitMask);
    // (the global histogram is only read when the short list cannot decide; adding to it costs
    // this launch under a microsecond, counting every key again in the second launch would cost 7)
    merge_hist<kFirstBlock>(lds_hist, st);
    if (short_on) {
        __syncthreads();
        unsigned digit;
        unsigned long long above;
        block_pick<kFirstBlock>(lds_hist, (unsigned long long)(short_k - 1), s_sum, &s_digit, &s_above, digit, above);
        // the cut is refined by the second digit: a top digit alone can be as coarse as a whole
        // binade (64-bit keys: it is the exponent), and a block would pass on every key of it
        for (int b = t; b < kRadixBins; b += kFirstBlock) lds_hist[b] = 0u;
        __syncthreads();
        const unsigned first_digit = (unsigned)(mine >> shift0) & kDigitMask;
        const unsigned second_digit = (unsigned)(mine >> shift1) & kDigitMask;
        hist_add(lds_hist, have && first_digit == digit, second_digit);
        __syncthreads();
        unsigned digit2;
        unsigned long long above2;
        block_pick<kFirstBlock>(lds_hist, (unsigned long long)(short_k - 1) - above, s_sum, &s_digit, &s_above, digit2,
                                above2);
        const unsigned cut = (digit << kRadixBits) | digit2;  // leading 2 * kRadixBits bits of the block's short_k-th key
        const bool out = have && ((first_digit << kRadixBits) | second_digit) >= cut;
        const unsigned long long outs = __ballot(out);
        const int lane = t & 63, wave = t >> 6;
        if (lane == 0) s_wave[wave] = (unsigned)__popcll(outs);
        __syncthreads();
        if (t == 0) {
            unsigned total = 0;
            for (int w = 0; w < kFirstBlock / 64; ++w) total += s_wave[w];
            s_base = atomicAdd(&st->short_count, total);
            atomicMax(&st->short_digit, cut);
        }
        __syncthreads();
        unsigned at = s_base + (unsigned)__popcll(outs & ((1ull << lane) - 1ull));
        for (int w = 0; w < wave; ++w) at += s_wave[w];
        if (out && at < short_cap) short_keys[at] = mine;  // an overflowing list is seen from its count
    }

}

// Bitwise AND and OR over the wavefront.
template <typename KEY> __device__ __forceinline__ void wave_and_or(KEY& a, KEY& o) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        a &= (KEY)__shfl_xor(a, off, 64);
        o |= (KEY)__shfl_xor(o, off, 64);
    }
}

// The second launch.  The short list's keys from the digit on from which the list is complete move
// to LDS (a round trip to memory per kListKeys listed keys).  Those keys share their leading bits
// (they are the largest few percent): the digits are taken from the first bit in which they differ,
// so that ONE histogram spreads them over the bins, and as soon as at most kDirect keys are left the
// wanted one is found by counting, for each, the keys above it.  Everything else (no short list,
// more such keys than LDS holds, a rank the list does not reach) starts from the first launch's
// top-digit counts of all keys and walks the fixed digits from the top over the key array, as the
// whole-vector passes do.
constexpr int kDirect = 256;

template <typename T>
__global__ __launch_bounds__(kFinishBlock) void select_finish_kernel(const typename Elem<T>::key_t* __restrict__ keys,
                                                                     int m, SelectState* __restrict__ st,
                                                                     unsigned long long rank, int plus_one,
                                                                     T* __restrict__ thr_out, int short_on,
                                                                     const typename Elem<T>::key_t* __restrict__ short_keys,
                                                                     unsigned short_cap, unsigned* __restrict__ zero_word) {
    using key_t = typename Elem<T>::key_t;
    constexpr int kKeyBits = Elem<T>::key_bits;
    constexpr int kListKeys = kListBytes / (int)sizeof(key_t);
    constexpr int shift1 = kKeyBits - 2 * kRadixBits;
    constexpr key_t kAllBits = (key_t)(~(key_t)0) >> (8 * (int)sizeof(key_t) - kKeyBits);
    static_assert(kDirect * sizeof(key_t) <= kRadixBins * sizeof(unsigned), "the candidates reuse the histogram");
    __shared__ __align__(8) unsigned lds_hist[kRadixBins];
    __shared__ key_t s_list[kListKeys];
    __shared__ key_t s_and, s_or, s_answer;
    __shared__ unsigned s_digit, s_fill;
    __shared__ unsigned long long s_above, s_sum[kFinishBlock / 64];
    const int t = threadIdx.x;
    const int lane = t & 63;

    // what the first launch's blocks passed on
    const unsigned short_count = short_on ? st->short_count : 0u;
    const unsigned short_cut = short_on ? st->short_digit : 0u;  // leading 2 * kRadixBits bits
    for (int b = t; b < kRadixBins; b += kFinishBlock) lds_hist[b] = 0u;
    if (t == 0) {
        s_fill = 0u;
        s_and = kAllBits;
        s_or = (key_t)0;
    }
    __syncthreads();
    if (short_on && t == 0) {  // clean for the next run
        st->short_count = 0u;
        st->short_digit = 0u;
    }
    if (zero_word && t == 0) *zero_word = 0u;  // a counter the kernels after this one start from
    key_t prefix = 0, mask = 0;
    int lo = kKeyBits;  // the bits below this one are still open
    // where the keys still in play are read from: the key array, the short list, or (listed) LDS
    const key_t* src = keys;
    unsigned src_n = (unsigned)m;
    bool listed = false, counted = false;
    unsigned list_n = 0;
    if (short_on && short_count <= short_cap) {
        // the listed keys from the digit on from which the list is complete move to LDS, a round
        // trip to memory per kListKeys of them (one, usually); their order does not matter
        constexpr int kPer = kListKeys / kFinishBlock;
        key_t all_and = kAllBits, all_or = (key_t)0;
        for (unsigned first = 0; first < short_count; first += (unsigned)(kPer * kFinishBlock)) {
            key_t kk[kPer];
#pragma unroll
            for (int q = 0; q < kPer; ++q) {
                const unsigned j = first + (unsigned)(q * kFinishBlock + t);
                kk[q] = j < short_count ? short_keys[j] : (key_t)0;
            }
#pragma unroll
            for (int q = 0; q < kPer; ++q) {
                if (first + (unsigned)(q * kFinishBlock) < short_count) {  // the same for the whole block
                    const unsigned j = first + (unsigned)(q * kFinishBlock + t);
                    const bool in = j < short_count && (unsigned)(kk[q] >> shift1) >= short_cut;
                    const unsigned long long ins = __ballot(in);
                    unsigned base = 0;
                    if (lane == 0 && ins) base = atomicAdd(&s_fill, (unsigned)__popcll(ins));
                    base = __shfl(base, 0, 64);
                    const unsigned at = base + (unsigned)__popcll(ins & ((1ull << lane) - 1ull));
                    if (in && at < (unsigned)kListKeys) {  // (more than fit: seen from the count)
                        s_list[at] = kk[q];
                        all_and &= kk[q];
                        all_or |= kk[q];
                    }
                }
            }
        }
        wave_and_or<key_t>(all_and, all_or);
        if (lane == 0) {
            atomicAnd(&s_and, all_and);
            atomicOr(&s_or, all_or);
        }
        __syncthreads();
        const unsigned complete = s_fill;
        if (complete <= (unsigned)kListKeys && rank < (unsigned long long)complete) {  // the wanted key is one of these
            counted = true;
            listed = true;
            list_n = complete;
            const key_t differ = s_and ^ s_or;
            lo = differ ? 64 - __clzll((unsigned long long)differ) : 0;
            const key_t open_bits = lo >= 8 * (int)sizeof(key_t) ? (key_t)~(key_t)0 : (key_t)(((key_t)1 << lo) - 1);
            mask = kAllBits & ~open_bits;
            prefix = s_and & mask;
        }
    }
    __syncthreads();
    bool hist_ready = false;
    // top digit of every key, counted by the first launch: used when the short list did not decide
    for (int b = t; b < kRadixBins; b += kFinishBlock) {
        if (!counted) lds_hist[b] = st->hist[b];
        st->hist[b] = 0u;  // leave it clean for the next run
    }
    if (!counted) {
        hist_ready = true;
        __syncthreads();
    }
    while (lo > 0) {
        const int bits = lo < kRadixBits ? lo : kRadixBits;
        const int shift = lo - bits;
        const unsigned digit_mask = (1u << bits) - 1u;
        if (!hist_ready) {
            for (int b = t; b < kRadixBins; b += kFinishBlock) lds_hist[b] = 0u;
            __syncthreads();
            if (listed) {
                for (unsigned j = t; j < list_n; j += kFinishBlock) {
                    const key_t k1 = s_list[j];
                    if ((k1 & mask) == prefix) atomicAdd(&lds_hist[(unsigned)(k1 >> shift) & digit_mask], 1u);
                }
            } else {
                // zero keys are counted in a register and go in once per wavefront: a vector of (mostly) zeros
                // would otherwise queue every key up on one LDS address (61 706 zeros: 134 us)
                unsigned zeros = 0u;
                scan_matching<key_t>(src, src_n, prefix, mask, [&](key_t k1) {
                    if (k1 == (key_t)0) ++zeros;
                    else atomicAdd(&lds_hist[(unsigned)(k1 >> shift) & digit_mask], 1u);
                });
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) zeros += __shfl_xor(zeros, off, 64);
                if (lane == 0 && zeros) atomicAdd(&lds_hist[0], zeros);
            }
            __syncthreads();
        }
        hist_ready = false;
        unsigned digit;
        unsigned long long above;
        block_pick<kFinishBlock>(lds_hist, rank, s_sum, &s_digit, &s_above, digit, above);
        const unsigned in_digit = lds_hist[digit];
        prefix |= (key_t)digit << shift;
        mask |= (key_t)((1ull << bits) - 1ull) << shift;
        rank -= above;
        lo = shift;
        if (lo == 0) break;
        if (!listed && in_digit <= (unsigned)kListKeys) {
            // collect the keys still in play; their order does not matter
            if (t == 0) s_fill = 0u;
            __syncthreads();
            scan_matching<key_t>(src, src_n, prefix, mask, [&](key_t k1) { s_list[atomicAdd(&s_fill, 1u)] = k1; });
            __syncthreads();
            list_n = s_fill;
            listed = true;
        }
        __syncthreads();
        if (listed && in_digit <= (unsigned)kDirect && in_digit > 0u) {
            // few keys left: the wanted one has at most `rank` keys above it and more than `rank`
            // keys at or above it
            key_t* cand = reinterpret_cast<key_t*>(lds_hist);
            if (t == 0) {
                s_fill = 0u;
                s_answer = prefix;  // (a rank beyond the keys leaves the open bits zero, as the digits would)
            }
            __syncthreads();
            for (unsigned j = t; j < list_n; j += kFinishBlock) {
                const key_t k1 = s_list[j];
                if ((k1 & mask) == prefix) cand[atomicAdd(&s_fill, 1u)] = k1;
            }
            __syncthreads();
            const unsigned c = s_fill;  // == in_digit
            if ((unsigned)t < c) {
                const key_t me = cand[t];
                unsigned gt = 0, ge = 0;
                for (unsigned j = 0; j < c; ++j) {
                    const key_t x = cand[j];
                    gt += x > me ? 1u : 0u;
                    ge += x >= me ? 1u : 0u;
                }
                if ((unsigned long long)gt <= rank && rank < (unsigned long long)ge) s_answer = me;
            }
            __syncthreads();
            prefix = s_answer;
            lo = 0;
        }
    }
    if (t == 0) {
        T v = value_of(prefix, T());
        if (plus_one) v = (T)(v + 1);
        *thr_out = v;
    }
}

// ---- up to one block's worth of keys: ONE launch -------------------------------------------
// ThresholdTopK's default is 1000 strided samples (src/threshold.hxx:130,182-186), so this is what an
// ordinary writeRemote runs: the block gathers its keys straight into LDS and finishes there (digits
// from the first bit in which the keys differ, then direct ranking of the last few), instead of one
// launch that stores the keys and a second that reads them back.
template <typename T, int SMODE, bool HAS_ADD>
__global__ __launch_bounds__(kFinishBlock) void select_one_block_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                                        const int* __restrict__ idx, int m, int n,
                                                                        float stepsize, unsigned long long rank,
                                                                        int plus_one, T* __restrict__ thr_out,
                                                                        unsigned* __restrict__ zero_word) {
    using key_t = typename Elem<T>::key_t;
    constexpr int kKeyBits = Elem<T>::key_bits;
    constexpr key_t kAllBits = (key_t)(~(key_t)0) >> (8 * (int)sizeof(key_t) - kKeyBits);
    __shared__ __align__(8) unsigned lds_hist[kRadixBins];
    __shared__ key_t s_list[kFinishBlock];
    __shared__ key_t s_and, s_or, s_answer;
    __shared__ unsigned s_digit, s_fill;
    __shared__ unsigned long long s_above, s_sum[kFinishBlock / 64];
    const int t = threadIdx.x;
    const int lane = t & 63;
    if (t == 0) {
        s_and = kAllBits;
        s_or = (key_t)0;
    }
    if (zero_word && t == 0) *zero_word = 0u;
    __syncthreads();
    const bool have = t < m;
    key_t mine = 0;
    if (have) {
        long long p;
        bool ok = true;
        if (SMODE == 0) {
            p = t;
        } else if (SMODE == 1) {
            p = (long long)(int)__fmul_rn((float)t, stepsize);  // (int)(i * stepsize), product in fp32
            if (p > (long long)n - 1) p = (long long)n - 1;     // the reference would read out of bounds
            if (p < 0) p = 0;
        } else {
            p = idx[t];
            ok = p >= 0 && p < (long long)n;  // positions outside the vector count as magnitude 0
            if (!ok) p = 0;
        }
        T v = vec[p];
        if (HAS_ADD) v = (T)(v + add[p]);
        mine = ok ? key_of(v) : (key_t)0;
        s_list[t] = mine;
    }
    key_t all_and = have ? mine : kAllBits, all_or = have ? mine : (key_t)0;
    wave_and_or<key_t>(all_and, all_or);
    if (lane == 0) {
        atomicAnd(&s_and, all_and);
        atomicOr(&s_or, all_or);
    }
    __syncthreads();
    const key_t differ = s_and ^ s_or;
    int lo = differ ? 64 - __clzll((unsigned long long)differ) : 0;  // the bits below this one are still open
    const key_t open_bits = lo >= 8 * (int)sizeof(key_t) ? (key_t)~(key_t)0 : (key_t)(((key_t)1 << lo) - 1);
    key_t mask = kAllBits & ~open_bits;
    key_t prefix = s_and & mask;
    while (lo > 0) {
        const int bits = lo < kRadixBits ? lo : kRadixBits;
        const int shift = lo - bits;
        const unsigned digit_mask = (1u << bits) - 1u;
        for (int b = t; b < kRadixBins; b += kFinishBlock) lds_hist[b] = 0u;
        __syncthreads();
        if (have && (mine & mask) == prefix) atomicAdd(&lds_hist[(unsigned)(mine >> shift) & digit_mask], 1u);
        __syncthreads();
        unsigned digit;
        unsigned long long above;
        block_pick<kFinishBlock>(lds_hist, rank, s_sum, &s_digit, &s_above, digit, above);
        const unsigned in_digit = lds_hist[digit];
        prefix |= (key_t)digit << shift;
        mask |= (key_t)((1ull << bits) - 1ull) << shift;
        rank -= above;
        lo = shift;
        if (lo == 0) break;
        __syncthreads();
        if (in_digit <= (unsigned)kDirect && in_digit > 0u) {
            // few keys left: the wanted one has at most `rank` keys above it and more than `rank` at or above it
            key_t* cand = reinterpret_cast<key_t*>(lds_hist);
            if (t == 0) {
                s_fill = 0u;
                s_answer = prefix;
            }
            __syncthreads();
            if (have && (mine & mask) == prefix) cand[atomicAdd(&s_fill, 1u)] = mine;
            __syncthreads();
            const unsigned c = s_fill;  // == in_digit
            if ((unsigned)t < c) {
                const key_t me = cand[t];
                unsigned gt = 0, ge = 0;
                for (unsigned j = 0; j < c; ++j) {
                    const key_t x = cand[j];
                    gt += x > me ? 1u : 0u;
                    ge += x >= me ? 1u : 0u;
                }
                if ((unsigned long long)gt <= rank && rank < (unsigned long long)ge) s_answer = me;
            }
            __syncthreads();
            prefix = s_answer;
            lo = 0;
        }
    }
    if (t == 0) {
        T v = value_of(prefix, T());
        if (plus_one) v = (T)(v + 1);
        *thr_out = v;
    }
}

// ---- whole-vector selection with a sampled lower bound ---------------------------------
// Copies every key >= the key of *d_bound into `cand` (order irrelevant).  Each wavefront
// gathers its matches in an LDS segment and appends the segment with ONE global atomic when it
// fills up and at the end, so the counter sees a few thousand atomics per pass, not one per hit.
// *cand_count keeps counting past `cap`; the passes that follow see it and take the whole vector(s) instead.
// Cache policy of the one-pass candidate collection: both vectors bypass the caches.  Measured on 100 M
// fp32 elements, threshold alone / threshold + compress as two calls: both nontemporal 0.165 / 0.360 ms,
// the gradient only 0.168 / 0.373 ms, neither 0.178 / 0.403 ms.  16-byte loads in flight per lane:
// 2 / 4 / 8 give 0.196 / 0.168 / 0.171 ms for the threshold alone.
constexpr bool kCollectNontemporalVec = true;    // first vector (the residual, when there are two)
constexpr bool kCollectNontemporalAdd = true;   // second vector (the gradient)
constexpr int kCollectUnroll = 4;               // 16-byte loads in flight per lane
// every wavefront ends with one returning atomic on the one counter, and those queue up: measured on
// 100 M elements, 256 / 512 / 1024 / 2048 / 4096 blocks take 0.252 / 0.207 / 0.218 / 0.243 / 0.306 ms
constexpr int kCollectBlocks = 512;

template <typename T, bool HAS_ADD, int VEC>
__global__ __launch_bounds__(kBlock) void select_collect_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                                long long m, const T* __restrict__ d_bound,
                                                                typename Elem<T>::key_t* __restrict__ cand, unsigned cap,
                                                                unsigned* __restrict__ cand_count, int reverse,
                                                                unsigned* __restrict__ top_hist) {
    using key_t = typename Elem<T>::key_t;
    constexpr int kPerIter = 64 * VEC * kCollectUnroll;  // keys a wavefront looks at per iteration
    constexpr int kSegKeys = 2 * kPerIter;
    constexpr int shift0 = Elem<T>::key_bits - kRadixBits;
    __shared__ key_t seg[kBlock / 64][kSegKeys];
    __shared__ unsigned lds_hist[kRadixBins];  // top digits of the block's candidates
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) lds_hist[b] = 0u;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const key_t bound = key_of(*d_bound);
    key_t* my = seg[wave];
    unsigned held = 0;  // keys in this wavefront's segment (same value in every lane)

    auto flush = [&]() {
        if (held == 0) return;
        unsigned base = 0;
        if (lane == 0) base = atomicAdd(cand_count, held);
        base = __shfl(base, 0, 64);
        for (unsigned i = lane; i < held; i += 64)
            if (base + i < cap) cand[base + i] = my[i];
        held = 0;
    };
    // appends this lane's hits (bit q of `mask` = key kk[q] is a candidate): one prefix sum over
    // the lanes' hit counts places them; their order inside the segment does not matter
    auto append = [&](const key_t* kk, unsigned mask, int nkeys) {
        const unsigned cnt = __popc(mask);
        unsigned incl = cnt;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const unsigned up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        unsigned at = held + incl - cnt;
        for (int q = 0; q < nkeys; ++q)
            if ((mask >> q) & 1u) {
                my[at++] = kk[q];
                atomicAdd(&lds_hist[(unsigned)(kk[q] >> shift0)], 1u);
            }
        held += __shfl(incl, 63, 64);
    };

    const long long nvec = m / VEC;
    const long long waves = (long long)gridDim.x * (kBlock / 64);
    const long long wave_id = (long long)blockIdx.x * (kBlock / 64) + wave;
    // a wavefront takes kCollectUnroll consecutive groups of 64 vectors per iteration; whole
    // wavefronts stay in the loop together (cross-lane operations)
    const long long ngroups = (nvec + 63) / 64;
    for (long long g0 = wave_id * kCollectUnroll; g0 < ngroups; g0 += waves * kCollectUnroll) {
        if (held + kPerIter > kSegKeys) flush();
        Pack<T, VEC> a[kCollectUnroll], b[kCollectUnroll];
        bool in[kCollectUnroll];
#pragma unroll
        for (int u = 0; u < kCollectUnroll; ++u) {
            // reversed passes start at the far end, where the previous pass over the vectors ended
            const long long g = reverse ? ngroups - 1 - (g0 + u) : g0 + u;
            const long long i = g * 64 + lane;
            in[u] = g >= 0 && i < nvec;
            if (in[u]) {
                typedef T vec_t __attribute__((ext_vector_type(VEC)));
                const vec_t va = kCollectNontemporalVec ? __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(vec) + i)
                                                        : reinterpret_cast<const vec_t*>(vec)[i];
#pragma unroll
                for (int c = 0; c < VEC; ++c) a[u].x[c] = va[c];
                if (HAS_ADD) {
                    const vec_t vb = kCollectNontemporalAdd
                                         ? __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(add) + i)
                                         : reinterpret_cast<const vec_t*>(add)[i];
#pragma unroll
                    for (int c = 0; c < VEC; ++c) b[u].x[c] = vb[c];
                }
            }
        }
        key_t kk[kCollectUnroll * VEC];
        unsigned mask = 0;
#pragma unroll
        for (int u = 0; u < kCollectUnroll; ++u) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                T v = (T)0;
                if (in[u]) v = HAS_ADD ? (T)(a[u].x[c] + b[u].x[c]) : a[u].x[c];
                const key_t k = key_of(v);
                kk[u * VEC + c] = k;
                mask |= ((in[u] && k >= bound) ? 1u : 0u) << (u * VEC + c);
            }
        }
        if (__any(mask != 0u)) append(kk, mask, kCollectUnroll * VEC);
    }
    if (blockIdx.x == 0 && wave == 0) {  // elements past the last full vector
        const long long i = nvec * VEC + lane;
        if (held + 64 > kSegKeys) flush();
        T v = (T)0;
        if (i < m) {
            v = vec[i];
            if (HAS_ADD) v = (T)(v + add[i]);
        }
        const key_t k = key_of(v);
        append(&k, (i < m && k >= bound) ? 1u : 0u, 1);
    }
    // what the block's wavefronts still hold leaves with ONE atomic on the counter (those atomics
    // return a value and queue up: one per wavefront cost the exact threshold 15 of its 198 us on
    // 100 M elements; more blocks than 512 gain nothing either way)
    __shared__ unsigned s_held[kBlock / 64], s_base;
    if (lane == 0) s_held[wave] = held;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned total = 0;
        for (int w = 0; w < kBlock / 64; ++w) total += s_held[w];
        s_base = total ? atomicAdd(cand_count, total) : 0u;
    }
    __syncthreads();
    unsigned base = s_base;
    for (int w = 0; w < wave; ++w) base += s_held[w];
    for (unsigned i = lane; i < held; i += 64)
        if (base + i < cap) cand[base + i] = my[i];
    // the candidates are the largest keys: they share a few top digits, so this is a few atomics per block
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) {
        const unsigned c = lds_hist[b];
        if (c) atomicAdd(&top_hist[b], c);
    }
}

template <typename T> __global__ void set_scalar_kernel(T* out, T v) { *out = v; }

template <typename T, int SMODE, bool HAS_ADD, int VEC>
void launch_hist(cx_handle h, const T* vec, const T* add, const int* idx, long long m, int n, float stepsize, int p,
                 unsigned long long rank0, typename Elem<T>::key_t* keys_out) {
    // Blocks: every block merges its histogram with atomics, few blocks leave memory idle.  Measured,
    // three passes + pick, 256-thread blocks with 2 / 4 / 8 / 16 16-byte loads per thread: 150 000 keys 17.0 /
    // 17.9 / 20.6 / 26.3 us, 2^20 keys 28.7 / 23.9 / 23.6 / 27.9 us, 2^22 keys 73.0 / 49.9 / 38.5 / 37.1 us: about
    // 128 blocks while 2048 to 65 536 keys per block allow it (again with four loads in flight, 2^20 keys, at
    // least 64 / 96 / 128 / 256 / 512 blocks: 23.6 / 22.5 / 21.5 / 23.1 / 28.9 us).
    const long long fine = 256ll * VEC * 2, coarse = (long long)kHistBlock * VEC * 16;
    const long long at_most = (m + fine - 1) / fine, at_least = (m + coarse - 1) / coarse;
    long long blocks = at_least > 128 ? at_least : 128;
    if (blocks > at_most) blocks = at_most;
    if (blocks < 1) blocks = 1;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL((select_hist_kernel<T, SMODE, HAS_ADD, VEC>), dim3((unsigned)blocks), dim3(kHistBlock), 0, h->stream,
                       vec, add, idx, m, n, stepsize, h->sel, p, rank0, keys_out);
}

template <typename T, bool HAS_ADD>
void dispatch_hist(cx_handle h, int smode, bool vec_ok, const T* vec, const T* add, const int* idx, long long m, int n,
                   float stepsize, int p, unsigned long long rank0, typename Elem<T>::key_t* keys_out = nullptr) {
    constexpr int kVec = 16 / (int)sizeof(T);
    if (smode == kSampleFull) {
        if (vec_ok) launch_hist<T, 0, HAS_ADD, kVec>(h, vec, add, idx, m, n, stepsize, p, rank0, nullptr);
        else launch_hist<T, 0, HAS_ADD, 1>(h, vec, add, idx, m, n, stepsize, p, rank0, nullptr);
    } else if (smode == kSampleStrided) {
        launch_hist<T, 1, HAS_ADD, 1>(h, vec, add, idx, m, n, stepsize, p, rank0, keys_out);
    } else {
        launch_hist<T, 2, HAS_ADD, 1>(h, vec, add, idx, m, n, stepsize, p, rank0, keys_out);
    }
}

}  // namespace

// End of a chained selection: the last pick, from the last pass's histogram.  Either a launch of the
// one-block kernel, or (defer_pick) left to the compress pass that follows, whose blocks make it themselves.
template <typename T> int launch_pending_pick(cx_handle h) {
    if (!h->pending_pick.active) return CX_OK;
    h->pending_pick.active = false;
    hipLaunchKernelGGL(select_final_kernel<T>, dim3(1), dim3(kBlock), 0, h->stream, h->sel, h->pending_pick.rank,
                       h->pending_pick.plus_one, static_cast<T*>(h->pending_pick.thr_out));
    CX_HIP(hipGetLastError());
    return CX_OK;
}
template int launch_pending_pick<float>(cx_handle);
template int launch_pending_pick<double>(cx_handle);
template int launch_pending_pick<int>(cx_handle);

template <typename T> int finish_chained(cx_handle h, unsigned long long rank, int plus_one, T* d_thr_out) {
    h->pending_pick.active = true;
    h->pending_pick.rank = rank;
    h->pending_pick.plus_one = plus_one;
    h->pending_pick.thr_out = d_thr_out;
    return h->defer_pick ? CX_OK : launch_pending_pick<T>(h);
}

// The key of descending rank `rank` among the m keys described by (vec, add_vec, d_idx, mode).
// key array of the two-launch select (2 MB), then its short list
int ensure_select_keys(cx_handle h) {
    const size_t want_bytes = (size_t)kSmallSelect * sizeof(unsigned long long);
    if (h->sel_keys_bytes < want_bytes) {
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->sel_keys) CX_HIP(hipFree(h->sel_keys));
        h->sel_keys = nullptr;
        h->sel_keys_bytes = 0;
        CX_HIP(hipMalloc(&h->sel_keys, want_bytes + (size_t)kShortGlobalKeys * sizeof(unsigned long long)));
        h->sel_keys_bytes = want_bytes;
    }
    return CX_OK;
}

// candidate buffer of the one-pass exact selections
int ensure_candidates(cx_handle h, size_t need) {
    if (need > h->cand_bytes) {
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->cand) CX_HIP(hipFree(h->cand));
        h->cand = nullptr;
        h->cand_bytes = 0;
        CX_HIP(hipMalloc(&h->cand, need + 256));
        h->cand_bytes = need;
    }
    return CX_OK;
}

// From how many elements on the whole-vector threshold takes one candidate pass instead of three
// histogram passes.  Measured on N(0,1) vectors, top 0.1 % / 1 %, candidate pass against three passes:
// 5 Mi elements 47.0 / 50.5 us against 37.7 / 39.3 us, 6 M 49.0 / 50.6 against 41.4 / 42.7, 8 Mi 50.0 / 51.3
// against 48.4 / 50.2, 12 M 56.6 / 58.1 against 58.9 / 61.6, 16 Mi 62.3 / 64.4 against 75.2 / 77.7, 32 Mi 77.3 /
// 78.9 against 129.6 / 130.4; followed by the compress in the same call: 8 Mi 74.0 / 77.4 against 72.3 / 73.0,
// 12 M 85.5 / 87.8 against 87.9 / 89.4.
constexpr int kCandidatePassMinN = 10 << 20;
// candidates kept for a vector of m elements: a sixteenth of it, at least 4 Mi
inline size_t candidate_capacity(long long m) {
    return (size_t)m / 16 > ((size_t)1 << 22) ? (size_t)m / 16 : ((size_t)1 << 22);
}

template <typename T>
int select_rank(cx_handle h, const T* vec, const T* add_vec, int n, const int* d_idx, int m, int sample_mode,
                float stepsize, unsigned long long rank, int plus_one, T* d_thr_out, unsigned* zero_word = nullptr) {
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    using key_t = typename Elem<T>::key_t;

    // short list of the two-launch select: see below
    int short_k = 0;
    const unsigned short_cap = (unsigned)kShortGlobalKeys;
    if (m <= kSmallSelect) {
        const int blocks = (m + kFirstBlock - 1) / kFirstBlock;
        const double share = (double)(rank + 1) / (double)blocks;
        short_k = (int)(share + 8.0 * std::sqrt(share) + 8.0);
        if (!h->select_short_list || m < 8192 || short_k > kFirstBlock / 8 ||
            (double)blocks * (short_k + 16.0) > (double)short_cap)
            short_k = 0;
    }
    // Two launches or chained passes?  Measured on N(0,1) keys, whole vector (+ second vector), threshold
    // alone, top 1 % / 3 % / 10 % / 30 %, two launches against chained passes: 40 000 keys 11.8 / 14.3 /
    // 14.2 / 14.9 us against 15.6 / 15.5 / 15.4 / 15.7 us, 61 706 keys 12.4 / 15.6 / 16.9 / 18.3 against
    // 15.9 / 15.8 / 15.6 / 15.8, 100 000 keys 13.6 / 18.1 / 22.2 / 24.0 against 16.0 / 16.3 / 16.1 / 16.4,
    // 150 000 keys 15.6 / 21.9 / 28.2 / 31.1 against 16.9 / 16.9 / 16.7 / 17.2, 200 000 keys 17.6 / 25.5 /
    // 34.7 / 38.6 against 17.3 / 17.4 / 17.5 / 18.0, 262 144 keys 20.0 / 49.5 / 40.9 / 38.8 against 18.3 /
    // 18.5 / 18.6 / 19.4: the one-block second launch grows with what the short list leaves it.  Sampled
    // keys (two dependent gathers per key and pass) and 8-byte keys (six passes) stay with the two launches.
    const bool two_launches = m <= kSmallSelect && (sample_mode != kSampleFull || kPasses > 3 || zero_word ||
                                                     m <= 40960 || (short_k > 0 && rank <= 1500ull));
    if (two_launches && m <= kFinishBlock) {
#define CX_ONE(SM, HA)                                                                                              \
    hipLaunchKernelGGL((select_one_block_kernel<T, SM, HA>), dim3(1), dim3(kFinishBlock), 0, h->stream, vec, add_vec, \
                       d_idx, m, n, stepsize, rank, plus_one, d_thr_out, zero_word)
#define CX_ONE_MODE(HA)                                      \
    do {                                                     \
        if (sample_mode == kSampleFull) CX_ONE(0, HA);       \
        else if (sample_mode == kSampleStrided) CX_ONE(1, HA); \
        else CX_ONE(2, HA);                                  \
    } while (0)
        if (add_vec) CX_ONE_MODE(true);
        else CX_ONE_MODE(false);
#undef CX_ONE_MODE
#undef CX_ONE
        CX_HIP(hipGetLastError());
        return CX_OK;
    }
    if (two_launches) {
        int rc_keys = ensure_select_keys(h);
        if (rc_keys != CX_OK) return rc_keys;
        key_t* keys = static_cast<key_t*>(h->sel_keys);
        key_t* short_keys = reinterpret_cast<key_t*>(static_cast<char*>(h->sel_keys) + h->sel_keys_bytes);
        const int blocks = (m + kFirstBlock - 1) / kFirstBlock;
        // short list: worth it when the wanted rank is near the top, so that a block's share of the
        // keys above it (plus 8 sigma) is a small part of the block, and the shares fit the list.
        // Measured, threshold alone, list on / off: 200 000 N(0,1) keys, top 1 % 17.9 / 27.6 us, 3 %
        // 25.4 / 34.3 us, 10 % 49.1 / 34.9 us; 61 706 such keys 12.4 / 14.7, 15.7 / 16.9, 19.3 / 16.9 us;
        // 61 706 keys in segments of very different scale (the list can never decide there) 18.1 / 13.5,
        // 19.4 / 14.4, 22.4 / 16.6 us.  Hence an eighth of the block at most (top 5 % or so).
#define CX_FIRST(SM, HA)                                                                                             \
    hipLaunchKernelGGL((select_first_kernel<T, SM, HA>), dim3(blocks), dim3(kFirstBlock), 0, h->stream, vec, add_vec, \
                       d_idx, m, n, stepsize, keys, h->sel, short_k, short_keys, short_cap)
#define CX_FIRST_MODE(HA)                                      \
    do {                                                       \
        if (sample_mode == kSampleFull) CX_FIRST(0, HA);       \
        else if (sample_mode == kSampleStrided) CX_FIRST(1, HA); \
        else CX_FIRST(2, HA);                                  \
    } while (0)
        if (add_vec) CX_FIRST_MODE(true);
        else CX_FIRST_MODE(false);
#undef CX_FIRST_MODE
#undef CX_FIRST
        hipLaunchKernelGGL(select_finish_kernel<T>, dim3(1), dim3(kFinishBlock), 0, h->stream, keys, m, h->sel, rank,
                           plus_one, d_thr_out, short_k > 0 ? 1 : 0, short_keys, short_cap, zero_word);
        CX_HIP(hipGetLastError());
        return CX_OK;
    }
    if (zero_word) return fail(CX_ERR_INTERNAL, "select: only the two-launch path clears a counter");

    const bool vec_ok =
        ((reinterpret_cast<uintptr_t>(vec) | reinterpret_cast<uintptr_t>(add_vec)) & 15u) == 0;  // null add is aligned
    // chained radix passes (no pick launch in between), then the last pick
    // A large sample (more keys than the two launches take) is gathered once: pass 0 leaves the keys in the
    // candidate buffer and the later passes read them from there, consecutive, instead of following the
    // positions again (10^6 positions in 10^8 elements: 37 us per gathering pass, random reads of two vectors).
    // Only where the buffer cx_reserve sizes for a vector of n elements holds them.
    key_t* cached = nullptr;
    if (sample_mode != kSampleFull && n >= (1 << 23) && (size_t)m <= candidate_capacity(n)) {
        int rc_cand = ensure_candidates(h, candidate_capacity(n) * sizeof(key_t));
        if (rc_cand != CX_OK) return rc_cand;
        cached = static_cast<key_t*>(h->cand);
    }
    for (int p = 0; p < kPasses; ++p) {
        if (cached && p > 0)
            dispatch_hist<T, false>(h, kSampleFull, true, reinterpret_cast<const T*>(cached), nullptr, nullptr, (long long)m,
                                    m, 1.0f, p, rank);
        else if (add_vec)
            dispatch_hist<T, true>(h, sample_mode, vec_ok, vec, add_vec, d_idx, (long long)m, n, stepsize, p, rank, cached);
        else
            dispatch_hist<T, false>(h, sample_mode, vec_ok, vec, add_vec, d_idx, (long long)m, n, stepsize, p, rank, cached);
    }
    return finish_chained<T>(h, rank, plus_one, d_thr_out);
}

// Whole-vector selection in ONE pass over the vector(s) when the wanted rank is near the top:
//   1. a strided sample gives a lower bound L that, with overwhelming probability, has at
//      least rank+1 keys at or above it, and not many more;
//   2. one pass copies the keys >= L into a candidate buffer and counts them;
//   3. chained radix passes whose blocks read that count: when rank < count <= capacity they run
//      over the candidates (the answer is the key of the same rank among them), otherwise (bound too
//      high, or ties flooded the buffer) over the whole vector(s).  Exact either way, and the host
//      never waits: the call is asynchronous like the others.
// Sets *done when the selection was launched; leaves it 0 when the path does not apply.
template <typename T>
int select_rank_bracketed(cx_handle h, const T* vec, const T* add_vec, int m, unsigned long long rank, int plus_one,
                          T* d_thr_out, int* done) {
    using key_t = typename Elem<T>::key_t;
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    *done = 0;
    // (sample size, measured on 100 M elements at 1 %: 2^14 / 2^15 / 2^16 / 2^17 samples give 0.153 / 0.155 /
    // 0.158 / 0.162 ms for this call and 0.306 / 0.301 / 0.297 / 0.297 ms for the single pass below, which uses
    // the same bound: a smaller sample is cheaper to select from and leaves more candidates)
    constexpr int kSample = 1 << 16;
    const double p = (double)(rank + 1) / (double)m;
    const double expect = p * kSample;
    const unsigned long long sample_rank = (unsigned long long)(expect + 8.0 * std::sqrt(expect) + 8.0);
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(vec) | reinterpret_cast<uintptr_t>(add_vec)) & 15u) == 0;
    if (m < kCandidatePassMinN || sample_rank >= (unsigned long long)kSample / 16 || !vec_ok) return CX_OK;

    const size_t cap = candidate_capacity(m);
    int rc_cand = ensure_candidates(h, cap * sizeof(key_t));
    if (rc_cand != CX_OK) return rc_cand;
    // 1. lower bound from the sample, left in the second half of the threshold slot; the kernel that
    //    writes it also clears the candidate counter
    T* d_bound = reinterpret_cast<T*>(static_cast<char*>(h->d_thr) + 64);
    unsigned* d_count = reinterpret_cast<unsigned*>(static_cast<char*>(h->d_thr) + 128);
    const float stepsize = (float)m / (float)kSample;
    int rc = select_rank<T>(h, vec, add_vec, m, nullptr, kSample, kSampleStrided, stepsize, sample_rank, 0, d_bound,
                            d_count);
    if (rc != CX_OK) return rc;
    // 2. candidates; the pass starts at the end of the vectors where the previous pass stopped
    const int reverse = h->stage_alternate ? (int)h->parity : 0;
    h->parity ^= 1u;  // the next full pass (the compress that follows) walks the other way
    constexpr int kVec = 16 / (int)sizeof(T);
    key_t* cand = static_cast<key_t*>(h->cand);
    if (add_vec)
        hipLaunchKernelGGL((select_collect_kernel<T, true, kVec>), dim3(kCollectBlocks), dim3(kBlock), 0, h->stream, vec, add_vec,
                           (long long)m, d_bound, cand, (unsigned)cap, d_count, reverse, h->sel->pass_hist[kPasses]);
    else
        hipLaunchKernelGGL((select_collect_kernel<T, false, kVec>), dim3(kCollectBlocks), dim3(kBlock), 0, h->stream, vec,
                           add_vec, (long long)m, d_bound, cand, (unsigned)cap, d_count, reverse,
                           h->sel->pass_hist[kPasses]);
    // 3. the passes, over whichever the count allows
    const long long per_block = (long long)kBlock * kVec * 8;
    long long blocks = ((long long)m + per_block - 1) / per_block;
    if (blocks > 2048) blocks = 2048;
    for (int q = 0; q < kPasses; ++q) {
        if (add_vec)
            hipLaunchKernelGGL((select_hist_either_kernel<T, true, kVec>), dim3((unsigned)blocks), dim3(kEitherBlock), 0, h->stream,
                               vec, add_vec, (long long)m, cand, (unsigned)cap, d_count, h->sel, q, rank);
        else
            hipLaunchKernelGGL((select_hist_either_kernel<T, false, kVec>), dim3((unsigned)blocks), dim3(kEitherBlock), 0, h->stream,
                               vec, add_vec, (long long)m, cand, (unsigned)cap, d_count, h->sel, q, rank);
    }
    *done = 1;
    return finish_chained<T>(h, rank, plus_one, d_thr_out);
}

template <typename T>
int launch_topk_threshold(cx_handle h, const T* vec, const T* add_vec, int n, const int* d_idx, int m, int sample_mode,
                          float stepsize, float topK, T* d_thr_out);

// Exact whole-vector top-k threshold and the fused compress in ONE pass over both vectors:
//   1. a strided sample gives a lower bound L of the threshold (as in select_rank_bracketed);
//   2. one streaming pass does update += data and moves every |update| > L out of the residual
//      into a list of candidate pairs, ascending (the fused compress with threshold L);
//   3. the threshold t >= L is the wanted order statistic among the candidates' magnitudes;
//   4. the candidates above t are copied to the message, the others go back into the residual.
// The list is unusable when it holds too few candidates (L too high: ties, a freak sample) or
// not all of them (more than its capacity; the excess never left the residual); the device
// notices, step 4 returns every listed candidate instead, and since `update` then holds the
// complete sum the answer comes from update alone: whole-vector selection on it and the
// update-only compress.  Same bits either way.  One host synchronisation, at the end.
template <typename T>
int launch_compress_topk(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                         float topK, T* d_thr_out, int* d_size_prefix) {
    if (!d_thr_out) d_thr_out = static_cast<T*>(h->d_thr);
    h->fused_topk_taken = 0;
    constexpr int kSample = 1 << 16;
    constexpr int PW = Elem<T>::pair_words;
    const int pos = n > 0 ? cx_topk_pos((size_t)n, topK) : 0;
    unsigned long long rank = pos > 0 ? (unsigned long long)pos : 0ull;
    if (n > 0 && rank > (unsigned long long)(n - 1)) rank = (unsigned long long)(n - 1);
    const double expect = n > 0 ? (double)(rank + 1) / (double)n * kSample : 0.0;
    const unsigned long long sample_rank = (unsigned long long)(expect + 8.0 * std::sqrt(expect) + 8.0);
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(update)) & 15u) == 0;
    const bool msg_ok = out_msg && (reinterpret_cast<uintptr_t>(out_msg) & 3u) == 0 && out_capacity >= 8;
    // From how many elements on?  Measured on N(0,1) vectors, top 0.1 % / 1 %, this single pass (which
    // ends with a wait) against the threshold followed by the compress (which never wait):
    // 8 Mi elements 73 / 81 us against 69 / 70 us, 12 M 81 / 87 against 81 / 84, 16 Mi 89 / 97 against
    // 94 / 96, 20 Mi 100 / 108 against 109 / 111, 25.6 M 107 / 114 against 121 / 123, 32 Mi 119 / 129 against
    // 142 / 146.  (Option fused_topk = 2 takes the single pass from 2^23 elements on.)
    constexpr int kSinglePassMinN = 20 << 20;
    const int single_pass_from = h->fused_topk >= 2 ? (1 << 23) : kSinglePassMinN;
    const bool single_pass = h->fused_topk && data && update && n >= single_pass_from && pos > 0 && vec_ok && msg_ok &&
                             sample_rank < (unsigned long long)kSample / 16;
    if (!single_pass) {
        h->defer_pick = data && update && n > 0;  // the compress pass makes a chained selection's last pick
        int rc = launch_topk_threshold<T>(h, update, data, n, nullptr, n, kSampleFull, 1.0f, topK, d_thr_out);
        h->defer_pick = false;
        if (rc == CX_OK) rc = launch_compact<T>(h, out_msg, out_capacity, data, update, n, nullptr, d_thr_out, d_size_prefix);
        const int rc_pick = launch_pending_pick<T>(h);  // only if the compress never got as far as its pass
        return rc != CX_OK ? rc : rc_pick;
    }

    const size_t cap = candidate_capacity(n);
    int rc = ensure_candidates(h, 8 + cap * PW * 4);
    if (rc != CX_OK) return rc;
    unsigned* cand_words = static_cast<unsigned*>(h->cand);
    T* d_bound = reinterpret_cast<T*>(static_cast<char*>(h->d_thr) + 64);
    unsigned* d_result = reinterpret_cast<unsigned*>(static_cast<char*>(h->d_thr) + 128);

    // 1. lower bound
    rc = select_rank<T>(h, update, data, n, nullptr, kSample, kSampleStrided, (float)n / (float)kSample, sample_rank,
                            0, d_bound);
    if (rc != CX_OK) return rc;
    // 2. accumulate + candidates
    rc = launch_candidates<T>(h, cand_words, (long long)cap, data, update, n, d_bound);
    if (rc != CX_OK) return rc;
    // 3. threshold among the candidates
    // (chained passes: the pick after each pass is redone by every block of the next kernel, the
    // last one by the filter, which also writes the threshold and clears the histograms; block shape:
    // see kPairsBlock).
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    for (int p = 0; p < kPasses; ++p)
        hipLaunchKernelGGL(select_hist_pairs_kernel<T>, dim3(kPairsBlocks), dim3(kPairsBlock), 0, h->stream, cand_words, (unsigned)cap,
                           h->sel, p, rank);
    CX_HIP(hipGetLastError());
    // 4. message + residual
    rc = launch_filter<T>(h, cand_words, (unsigned)cap, rank, d_thr_out, update, n, static_cast<unsigned*>(out_msg),
                          (out_capacity - 8) / (4 * PW), d_size_prefix, d_result,
                          (unsigned long long)((double)sample_rank / (double)kSample * (double)n));
    if (rc != CX_OK) return rc;
    // (letting the last kernel store the result words in pinned host memory itself, without this copy, was
    // measured: 1 us or less on a call of 105 us)
    CX_HIP(hipMemcpyAsync(h->h_pinned + 12, d_result, 2 * sizeof(unsigned), hipMemcpyDeviceToHost, h->stream));
    CX_HIP(hipStreamSynchronize(h->stream));
    h->fused_topk_taken = 1;
    if (h->h_pinned[12] == 0) return CX_OK;

    // change of plan: `update` holds the complete sum, the message has not been touched
    h->fused_topk_taken = 2;
    rc = select_rank<T>(h, update, nullptr, n, nullptr, n, kSampleFull, 1.0f, rank, 0, d_thr_out);
    if (rc != CX_OK) return rc;
    return launch_compact<T>(h, out_msg, out_capacity, nullptr, update, n, nullptr, d_thr_out, d_size_prefix);
}

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
    if (sample_mode == kSampleFull && h->select_bracket) {
        int done = 0;
        int rc = select_rank_bracketed<T>(h, vec, add_vec, m, rank, plus_one, d_thr_out, &done);
        if (rc != CX_OK || done) return rc;
    }
    return select_rank<T>(h, vec, add_vec, n, d_idx, m, sample_mode, stepsize, rank, plus_one, d_thr_out);
}

template <typename T> int reserve_select(cx_handle h, int n) {
    int rc = ensure_select_keys(h);
    if (rc != CX_OK) return rc;
    // shorter vectors never take the one-pass selections (cx_ip_compress_topk's single pass can be asked for from
    // 2^23 elements on: option fused_topk = 2)
    if (n < kCandidatePassMinN && n < (1 << 23)) return CX_OK;
    const size_t cap = candidate_capacity(n);
    const size_t as_keys = cap * sizeof(typename Elem<T>::key_t), as_pairs = 8 + cap * Elem<T>::pair_words * 4;
    return ensure_candidates(h, as_keys > as_pairs ? as_keys : as_pairs);
}
template int reserve_select<float>(cx_handle, int);
template int reserve_select<double>(cx_handle, int);
template int reserve_select<int>(cx_handle, int);
template int launch_topk_threshold<float>(cx_handle, const float*, const float*, int, const int*, int, int, float, float, float*);
template int launch_topk_threshold<double>(cx_handle, const double*, const double*, int, const int*, int, int, float, float, double*);
template int launch_topk_threshold<int>(cx_handle, const int*, const int*, int, const int*, int, int, float, float, int*);
template int launch_compress_topk<float>(cx_handle, void*, long long, const float*, float*, int, float, float*, int*);
template int launch_compress_topk<double>(cx_handle, void*, long long, const double*, double*, int, float, double*, int*);
template int launch_compress_topk<int>(cx_handle, void*, long long, const int*, int*, int, float, int*, int*);

}  // namespace cx
