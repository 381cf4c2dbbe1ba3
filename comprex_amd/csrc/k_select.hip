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

#include <cmath>

namespace cx {

namespace {

constexpr int kBlock = 256;
constexpr int kSmallSelect = 1 << 18;  // sample sets up to this size take the two-launch path

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
            bool ok = true;
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
            T v = vec[p];
            if (HAS_ADD) v = (T)(v + add[p]);
            const key_t k = ok ? key_of(v) : (key_t)0;
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

// ---- small sample sets: two launches ---------------------------------------------------
// First launch: one thread per sample gathers its key, stores it to `keys` and counts the
// top digit (LDS histogram merged into the global one).  Second launch, one block: picks the
// top digit, then finishes the remaining digits over the stored keys with LDS histograms only.
constexpr int kFinishBlock = 1024;

template <typename T, int SMODE, bool HAS_ADD>
__global__ __launch_bounds__(kBlock) void select_first_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                              const int* __restrict__ idx, int m, int n, float stepsize,
                                                              typename Elem<T>::key_t* __restrict__ keys,
                                                              SelectState* __restrict__ st, int shift, int bits) {
    using key_t = typename Elem<T>::key_t;
    __shared__ unsigned lds_hist[kRadixBins];
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) lds_hist[b] = 0u;
    __syncthreads();
    const unsigned digit_mask = (1u << bits) - 1u;
    const int stride = gridDim.x * kBlock;
    for (int i = blockIdx.x * kBlock + threadIdx.x; i < m; i += stride) {
        long long p;
        bool ok = true;
        if (SMODE == 0) {
            p = i;
        } else if (SMODE == 1) {
            p = (long long)(int)__fmul_rn((float)i, stepsize);  // (int)(i * stepsize), product in fp32
            if (p > (long long)n - 1) p = (long long)n - 1;     // the reference would read out of bounds
            if (p < 0) p = 0;
        } else {
            p = idx[i];
            ok = p >= 0 && p < (long long)n;  // positions outside the vector count as magnitude 0
            if (!ok) p = 0;
        }
        T v = vec[p];
        if (HAS_ADD) v = (T)(v + add[p]);
        const key_t k = ok ? key_of(v) : (key_t)0;
        keys[i] = k;
        atomicAdd(&lds_hist[(unsigned)(k >> shift) & digit_mask], 1u);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < kRadixBins; b += kBlock) {
        const unsigned c = lds_hist[b];
        if (c) atomicAdd(&st->hist[b], c);
    }
}

// Block-wide: digit holding descending rank `rank` in hist[0..kRadixBins), and how many keys
// lie above that digit.  All threads get the result.
__device__ __forceinline__ void block_pick(const unsigned* hist, unsigned long long rank, unsigned long long* s_sum,
                                           unsigned* s_digit, unsigned long long* s_above, unsigned& digit,
                                           unsigned long long& above) {
    constexpr int kPer = kRadixBins / kFinishBlock;  // 2 bins per thread
    const int t = threadIdx.x;
    const int hi = kRadixBins - 1 - t * kPer;
    unsigned cnt[kPer];
    unsigned long long local = 0;
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        cnt[q] = hist[hi - q];
        local += cnt[q];
    }
    // inclusive scan over threads, top digits first
    unsigned long long incl = local;
    const int lane = t & 63, wave = t >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned long long up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) s_sum[wave] = incl;
    if (t == 0) {
        *s_digit = 0u;
        *s_above = 0ull;
    }
    __syncthreads();
    unsigned long long before = incl - local;
    for (int w = 0; w < wave; ++w) before += s_sum[w];
    if (rank >= before && rank < before + local) {
        unsigned long long acc = before;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            if (rank < acc + cnt[q]) {
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

template <typename T>
__global__ __launch_bounds__(kFinishBlock) void select_finish_kernel(const typename Elem<T>::key_t* __restrict__ keys,
                                                                     int m, SelectState* __restrict__ st,
                                                                     unsigned long long rank, int plus_one,
                                                                     T* __restrict__ thr_out) {
    using key_t = typename Elem<T>::key_t;
    constexpr int kKeyBits = Elem<T>::key_bits;
    constexpr int kPasses = (kKeyBits + kRadixBits - 1) / kRadixBits;
    __shared__ unsigned lds_hist[kRadixBins];
    __shared__ unsigned long long s_sum[kFinishBlock / 64];
    __shared__ unsigned s_digit;
    __shared__ unsigned long long s_above;
    const int t = threadIdx.x;

    // top digit: counted by the first launch into the global histogram
    for (int b = t; b < kRadixBins; b += kFinishBlock) {
        lds_hist[b] = st->hist[b];
        st->hist[b] = 0u;  // leave it clean for the next run
    }
    __syncthreads();
    key_t prefix = 0, mask = 0;
    for (int p = 0; p < kPasses; ++p) {
        int shift = kKeyBits - kRadixBits * (p + 1);
        int bits = kRadixBits;
        if (shift < 0) {
            bits += shift;
            shift = 0;
        }
        if (p > 0) {
            for (int b = t; b < kRadixBins; b += kFinishBlock) lds_hist[b] = 0u;
            __syncthreads();
            const unsigned digit_mask = (1u << bits) - 1u;
            constexpr int KV = 16 / (int)sizeof(key_t);  // keys per 16-byte load
            const int nvec = m / KV;
            const Pack<key_t, KV>* kv = reinterpret_cast<const Pack<key_t, KV>*>(keys);
            for (int v0 = 0; v0 < nvec; v0 += kFinishBlock * 4) {
                Pack<key_t, KV> kk[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int v = v0 + q * kFinishBlock + t;
                    if (v < nvec) kk[q] = kv[v];
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (v0 + q * kFinishBlock + t < nvec) {
#pragma unroll
                        for (int c = 0; c < KV; ++c)
                            if ((kk[q].x[c] & mask) == prefix)
                                atomicAdd(&lds_hist[(unsigned)(kk[q].x[c] >> shift) & digit_mask], 1u);
                    }
                }
            }
            for (int i = nvec * KV + t; i < m; i += kFinishBlock) {
                const key_t k1 = keys[i];
                if ((k1 & mask) == prefix) atomicAdd(&lds_hist[(unsigned)(k1 >> shift) & digit_mask], 1u);
            }
            __syncthreads();
        }
        unsigned digit;
        unsigned long long above;
        block_pick(lds_hist, rank, s_sum, &s_digit, &s_above, digit, above);
        prefix |= (key_t)digit << shift;
        mask |= (key_t)((1ull << bits) - 1ull) << shift;
        rank -= above;
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
// *cand_count keeps counting past `cap`; the host falls back when it overflows.
constexpr int kCollectUnroll = 4;  // 16-byte loads in flight per lane

template <typename T, bool HAS_ADD, int VEC>
__global__ __launch_bounds__(kBlock) void select_collect_kernel(const T* __restrict__ vec, const T* __restrict__ add,
                                                                long long m, const T* __restrict__ d_bound,
                                                                typename Elem<T>::key_t* __restrict__ cand, unsigned cap,
                                                                unsigned* __restrict__ cand_count, int reverse) {
    using key_t = typename Elem<T>::key_t;
    constexpr int kPerIter = 64 * VEC * kCollectUnroll;  // keys a wavefront looks at per iteration
    constexpr int kSegKeys = 2 * kPerIter;
    __shared__ key_t seg[kBlock / 64][kSegKeys];
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
            if ((mask >> q) & 1u) my[at++] = kk[q];
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
                a[u] = reinterpret_cast<const Pack<T, VEC>*>(vec)[i];
                if (HAS_ADD) b[u] = reinterpret_cast<const Pack<T, VEC>*>(add)[i];
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
    flush();
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

// The key of descending rank `rank` among the m keys described by (vec, add_vec, d_idx, mode).
template <typename T>
int select_rank(cx_handle h, const T* vec, const T* add_vec, int n, const int* d_idx, int m, int sample_mode,
                float stepsize, unsigned long long rank, int plus_one, T* d_thr_out) {
    constexpr int kKeyBits = Elem<T>::key_bits;
    constexpr int kPasses = (kKeyBits + kRadixBits - 1) / kRadixBits;
    using key_t = typename Elem<T>::key_t;

    if (m <= kSmallSelect) {
        if ((size_t)m * sizeof(key_t) > h->sel_keys_bytes) {
            CX_HIP(hipStreamSynchronize(h->stream));
            if (h->sel_keys) CX_HIP(hipFree(h->sel_keys));
            h->sel_keys = nullptr;
            h->sel_keys_bytes = 0;
            size_t bytes = (size_t)kSmallSelect * sizeof(unsigned long long);
            CX_HIP(hipMalloc(&h->sel_keys, bytes));
            h->sel_keys_bytes = bytes;
        }
        key_t* keys = static_cast<key_t*>(h->sel_keys);
        const int shift0 = kKeyBits - kRadixBits;
        int blocks = (m + kBlock - 1) / kBlock;
        if (blocks > 2048) blocks = 2048;
#define CX_FIRST(SM, HA)                                                                                          \
    hipLaunchKernelGGL((select_first_kernel<T, SM, HA>), dim3(blocks), dim3(kBlock), 0, h->stream, vec, add_vec, d_idx, \
                       m, n, stepsize, keys, h->sel, shift0, kRadixBits)
        if (add_vec) {
            if (sample_mode == kSampleFull) CX_FIRST(0, true);
            else if (sample_mode == kSampleStrided) CX_FIRST(1, true);
            else CX_FIRST(2, true);
        } else {
            if (sample_mode == kSampleFull) CX_FIRST(0, false);
            else if (sample_mode == kSampleStrided) CX_FIRST(1, false);
            else CX_FIRST(2, false);
        }
#undef CX_FIRST
        hipLaunchKernelGGL(select_finish_kernel<T>, dim3(1), dim3(kFinishBlock), 0, h->stream, keys, m, h->sel, rank,
                           plus_one, d_thr_out);
        CX_HIP(hipGetLastError());
        return CX_OK;
    }

    const bool vec_ok =
        ((reinterpret_cast<uintptr_t>(vec) | reinterpret_cast<uintptr_t>(add_vec)) & 15u) == 0;  // null add is aligned
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

// Whole-vector selection in ONE pass over the vector(s) when the wanted rank is near the top:
//   1. a strided sample gives a lower bound L that, with overwhelming probability, has at
//      least rank+1 keys at or above it, and not many more;
//   2. one pass copies the keys >= L into a candidate buffer;
//   3. the host reads the candidate count (the only synchronisation); when rank < count <= capacity
//      the answer is the key of the same rank among the candidates, found on that small set.
// Otherwise *done stays 0 and the caller runs the full three-pass selection.  Exact either way.
template <typename T>
int select_rank_bracketed(cx_handle h, const T* vec, const T* add_vec, int m, unsigned long long rank, int plus_one,
                          T* d_thr_out, int* done) {
    using key_t = typename Elem<T>::key_t;
    *done = 0;
    constexpr int kSample = 1 << 16;
    const double p = (double)(rank + 1) / (double)m;
    const double expect = p * kSample;
    const unsigned long long sample_rank = (unsigned long long)(expect + 8.0 * std::sqrt(expect) + 8.0);
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(vec) | reinterpret_cast<uintptr_t>(add_vec)) & 15u) == 0;
    if (m < (1 << 23) || sample_rank >= (unsigned long long)kSample / 16 || !vec_ok) return CX_OK;

    const size_t cap = (size_t)m / 16 > ((size_t)1 << 22) ? (size_t)m / 16 : ((size_t)1 << 22);
    if (cap * sizeof(key_t) > h->cand_bytes) {
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->cand) CX_HIP(hipFree(h->cand));
        h->cand = nullptr;
        h->cand_bytes = 0;
        CX_HIP(hipMalloc(&h->cand, cap * sizeof(key_t) + 256));
        h->cand_bytes = cap * sizeof(key_t);
    }
    // 1. lower bound from the sample, left in the second half of the threshold slot
    T* d_bound = reinterpret_cast<T*>(static_cast<char*>(h->d_thr) + 64);
    unsigned* d_count = reinterpret_cast<unsigned*>(static_cast<char*>(h->d_thr) + 128);
    const float stepsize = (float)m / (float)kSample;
    int rc = select_rank<T>(h, vec, add_vec, m, nullptr, kSample, kSampleStrided, stepsize, sample_rank, 0, d_bound);
    if (rc != CX_OK) return rc;
    // 2. candidates; the pass starts at the end of the vectors where the previous pass stopped
    const int reverse = h->stage_alternate ? (int)h->parity : 0;
    h->parity ^= 1u;  // the next full pass (the compress that follows) walks the other way
    CX_HIP(hipMemsetAsync(d_count, 0, sizeof(unsigned), h->stream));
    constexpr int kVec = 16 / (int)sizeof(T);
    key_t* cand = static_cast<key_t*>(h->cand);
    if (add_vec)
        hipLaunchKernelGGL((select_collect_kernel<T, true, kVec>), dim3(2048), dim3(kBlock), 0, h->stream, vec, add_vec,
                           (long long)m, d_bound, cand, (unsigned)cap, d_count, reverse);
    else
        hipLaunchKernelGGL((select_collect_kernel<T, false, kVec>), dim3(2048), dim3(kBlock), 0, h->stream, vec,
                           add_vec, (long long)m, d_bound, cand, (unsigned)cap, d_count, reverse);
    CX_HIP(hipGetLastError());
    // 3. how many?
    CX_HIP(hipMemcpyAsync(h->h_pinned + 12, d_count, sizeof(unsigned), hipMemcpyDeviceToHost, h->stream));
    CX_HIP(hipStreamSynchronize(h->stream));
    const unsigned long long count = (unsigned)h->h_pinned[12];
    if (count <= rank || count > cap) return CX_OK;  // bound too high (or ties flooded the buffer): full selection
    // magnitudes' bit patterns order like the magnitudes: the candidates are a vector of |x|
    rc = select_rank<T>(h, reinterpret_cast<const T*>(cand), nullptr, (int)count, nullptr, (int)count, kSampleFull,
                        1.0f, rank, plus_one, d_thr_out);
    if (rc == CX_OK) *done = 1;
    return rc;
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

template int launch_topk_threshold<float>(cx_handle, const float*, const float*, int, const int*, int, int, float, float, float*);
template int launch_topk_threshold<double>(cx_handle, const double*, const double*, int, const int*, int, int, float, float, double*);
template int launch_topk_threshold<int>(cx_handle, const int*, const int*, int, const int*, int, int, float, float, int*);

}  // namespace cx
