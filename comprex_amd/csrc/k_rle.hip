// Run-length codec on the GPU: CompressorRLE<T> (reference src/compressor.hxx:158-532).
//
// Message, as the reference's decoder reads it (:415-447):
//   int32 n | int32 c | c values of T | int32 runs | int32 signum | runs x int32 run lengths
// Runs alternate "sent" / "not sent" and start with a "sent" run when signum == 1; an element
// is sent when |x| >= threshold (:214,234,273,312; note >=).  The reference's encoder stores a
// sent element at its VECTOR position inside the value area (:238,277,316) while it advances
// the output by one value per sent element, so it only produces a well-formed message when
// every element is sent; the values are stored densely here, which is what its decoder expects.
//
// Compress: the IndexPairs path does the heavy pass (accumulate, select, ordered compaction,
// residual zeroing) into scratch with the strict comparison against the threshold's predecessor
// (|x| >= t  <=>  |x| > pred(t)); the ascending (index, value) pairs then become values + runs:
// a pair starts a "sent" run when its index does not continue the previous pair's, the gap
// before it is the "not sent" run in front of it.
// Decompress / add: exclusive prefix sums over the run lengths give every run's position and
// value offset; one thread per value finds its run by binary search.
#include "cx_common.hpp"

namespace cx {

namespace {

constexpr int kBlock = 256;
constexpr int kConvBlocks = 1024;  // blocks that share the pairs of a message
constexpr int kScanItems = 8;      // runs per thread in the prefix-sum kernels

template <typename T> __device__ __forceinline__ void store_words(unsigned* dst, T v);
template <> __device__ __forceinline__ void store_words<float>(unsigned* dst, float v) { dst[0] = __float_as_uint(v); }
template <> __device__ __forceinline__ void store_words<int>(unsigned* dst, int v) { dst[0] = (unsigned)v; }
template <> __device__ __forceinline__ void store_words<double>(unsigned* dst, double v) {
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    dst[0] = (unsigned)b;
    dst[1] = (unsigned)(b >> 32);
}
template <typename T> __device__ __forceinline__ T load_words(const unsigned* w);
template <> __device__ __forceinline__ float load_words<float>(const unsigned* w) { return __uint_as_float(w[0]); }
template <> __device__ __forceinline__ int load_words<int>(const unsigned* w) { return (int)w[0]; }
template <> __device__ __forceinline__ double load_words<double>(const unsigned* w) {
    return __longlong_as_double((long long)(((unsigned long long)w[1] << 32) | w[0]));
}

// Largest value u with: |x| > u  <=>  |x| >= t, for every x that is not NaN.
__device__ __forceinline__ float strict_equivalent(float t) {
    if (t != t) return t;        // NaN: nothing is sent either way
    if (!(t > 0.0f)) return -1.0f;  // |x| >= t holds for every number
    return __uint_as_float(__float_as_uint(t) - 1u);  // previous float (0 below the smallest denormal; FLT_MAX below inf)
}
__device__ __forceinline__ double strict_equivalent(double t) {
    if (t != t) return t;
    if (!(t > 0.0)) return -1.0;
    return __longlong_as_double(__double_as_longlong(t) - 1ll);
}
__device__ __forceinline__ int strict_equivalent(int t) { return t > 0 ? t - 1 : -1; }

template <typename T> __global__ void rle_threshold_kernel(const T* d_thr, T thr_val, T* out) {
    *out = strict_equivalent(d_thr ? *d_thr : thr_val);
}

// inclusive prefix sum over the block's threads; *total = the block's sum
__device__ __forceinline__ unsigned block_inclusive_scan(unsigned v, unsigned* s_wave, unsigned* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    __syncthreads();  // s_wave may still be read from the previous call
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    unsigned before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) {
        if (w < wave) before += s_wave[w];
        all += s_wave[w];
    }
    *total = all;
    return incl + before;
}

// a block's share [lo, hi) of k pairs
__device__ __forceinline__ void share_of(unsigned k, unsigned& lo, unsigned& hi) {
    const unsigned share = (k + kConvBlocks - 1) / kConvBlocks;
    lo = blockIdx.x * share < k ? blockIdx.x * share : k;
    hi = lo + share < k ? lo + share : k;
}

// pair j starts a "sent" run
template <int PW> __device__ __forceinline__ bool run_starts_at(const unsigned* pairs, unsigned j) {
    return j == 0u || pairs[(size_t)PW * j] != pairs[(size_t)PW * (j - 1)] + 1u;
}

// pass 1 over the pairs: "sent" runs that start in every block's share
template <typename T>
__global__ __launch_bounds__(kBlock) void rle_count_kernel(const unsigned* __restrict__ ip_words,
                                                           unsigned* __restrict__ block_counts) {
    constexpr int PW = Elem<T>::pair_words;
    __shared__ unsigned s_cnt;
    if (threadIdx.x == 0) s_cnt = 0u;
    __syncthreads();
    const unsigned k = ip_words[1];
    unsigned lo, hi;
    share_of(k, lo, hi);
    unsigned mine = 0;
    for (unsigned j = lo + threadIdx.x; j < hi; j += kBlock) mine += run_starts_at<PW>(ip_words + 2, j) ? 1u : 0u;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off, 64);
    if ((threadIdx.x & 63) == 0) atomicAdd(&s_cnt, mine);  // LDS
    __syncthreads();
    if (threadIdx.x == 0) block_counts[blockIdx.x] = s_cnt;
}

// Stores one int32 of the message if it fits; a message that does not fit is reported and then
// replaced by an empty one (rle_overflow_kernel).
__device__ __forceinline__ void put_word(unsigned* msg_words, long long word, long long cap_words, unsigned v,
                                         bool& overflow) {
    if (word < cap_words) msg_words[word] = v;
    else overflow = true;
}

// pass 2 (ENDS == false): values, the start index of every "sent" run (parked in the run's
// length slot) and the "not sent" run in front of it; pass 3 (ENDS == true): every "sent" run's
// length from its last pair, then header fields, the trailing "not sent" run and the byte count.
template <typename T, bool ENDS>
__global__ __launch_bounds__(kBlock) void rle_write_kernel(const unsigned* __restrict__ ip_words,
                                                           const unsigned* __restrict__ block_counts, int n,
                                                           unsigned* __restrict__ msg_words, long long cap_words,
                                                           int* __restrict__ size_prefix, int* __restrict__ result,
                                                           DeviceStatus* status) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int VW = (int)sizeof(T) / 4;  // words per value
    __shared__ unsigned s_wave[kBlock / 64];
    __shared__ unsigned s_before;
    const unsigned* pairs = ip_words + 2;
    const unsigned k = ip_words[1];
    const int tid = threadIdx.x;
    bool overflow = false;

    if (k == 0u) {  // nothing sent: one "not sent" run over the vector
        if (ENDS && blockIdx.x == 0 && tid == 0) {
            const unsigned runs = n > 0 ? 1u : 0u;
            put_word(msg_words, 0, cap_words, (unsigned)n, overflow);
            put_word(msg_words, 1, cap_words, 0u, overflow);
            put_word(msg_words, 2, cap_words, runs, overflow);
            put_word(msg_words, 3, cap_words, 0u, overflow);
            if (runs) put_word(msg_words, 4, cap_words, (unsigned)n, overflow);
            const int bytes = 16 + 4 * (int)runs;
            if (size_prefix) *size_prefix = bytes;
            result[0] = bytes;
            if (overflow) atomicOr(&status->detail, 1);
        }
        return;
    }

    // runs that start before this block's share
    if (tid == 0) s_before = 0u;
    __syncthreads();
    unsigned before = 0;
    for (unsigned b = tid; b < blockIdx.x; b += kBlock) before += block_counts[b];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off, 64);
    if ((tid & 63) == 0 && before) atomicAdd(&s_before, before);  // LDS
    __syncthreads();
    unsigned runs_before = s_before;

    const unsigned lead = pairs[0] > 0u ? 1u : 0u;                  // the message starts with a "not sent" run
    const long long trailer = 2 + (long long)k * VW + 2;            // word index of the first run length
    unsigned lo, hi;
    share_of(k, lo, hi);
    for (unsigned j0 = lo; j0 < hi; j0 += kBlock) {  // uniform trip count per block
        const unsigned j = j0 + tid;
        const bool in = j < hi;
        const bool starts = in && run_starts_at<PW>(pairs, j);
        unsigned chunk_total;
        const unsigned incl = block_inclusive_scan(starts ? 1u : 0u, s_wave, &chunk_total);
        if (in) {
            const unsigned y = runs_before + incl - 1u;  // the "sent" run pair j belongs to
            const unsigned idx = pairs[(size_t)PW * j];
            if (!ENDS) {
                unsigned v[VW];
                store_words<T>(v, load_words<T>(pairs + (size_t)PW * j + 1));
#pragma unroll
                for (int w = 0; w < VW; ++w) put_word(msg_words, 2 + (long long)j * VW + w, cap_words, v[w], overflow);
                if (starts) {
                    put_word(msg_words, trailer + lead + 2ll * y, cap_words, idx, overflow);  // parked: start index
                    if (j > 0u)
                        put_word(msg_words, trailer + lead + 2ll * y - 1, cap_words,
                                 idx - pairs[(size_t)PW * (j - 1)] - 1u, overflow);
                    else if (lead)
                        put_word(msg_words, trailer, cap_words, idx, overflow);
                }
            } else {
                const bool ends = j + 1u == k || pairs[(size_t)PW * (j + 1)] != idx + 1u;
                if (ends) {
                    const long long slot = trailer + lead + 2ll * y;
                    if (slot < cap_words) msg_words[slot] = idx + 1u - msg_words[slot];
                    else overflow = true;
                }
                if (j + 1u == k) {  // the last pair closes the message
                    const unsigned sent_runs = y + 1u;
                    const unsigned tail = idx + 1u < (unsigned)n ? 1u : 0u;
                    const unsigned runs = lead + 2u * sent_runs - 1u + tail;
                    if (tail) put_word(msg_words, trailer + runs - 1, cap_words, (unsigned)n - idx - 1u, overflow);
                    put_word(msg_words, 0, cap_words, (unsigned)n, overflow);
                    put_word(msg_words, 1, cap_words, k, overflow);
                    put_word(msg_words, trailer - 2, cap_words, runs, overflow);
                    put_word(msg_words, trailer - 1, cap_words, lead ? 0u : 1u, overflow);
                    const int bytes = (int)(4 * (trailer + runs));
                    if (size_prefix) *size_prefix = bytes;
                    result[0] = bytes;
                }
            }
        }
        runs_before += chunk_total;
    }
    if (overflow) atomicOr(&status->detail, 1);
}

// A message that did not fit (result[0] = its true size > capacity): nothing of it may be taken
// for a message, and nothing may be lost.  The pairs the first pass took out of `update` go back
// (it cleared them, so storing restores the sums), and the buffer gets the empty message (one
// "not sent" run over the vector) when it has room for that, whose size is then what is reported.
template <typename T>
__global__ __launch_bounds__(kBlock) void rle_overflow_kernel(const unsigned* __restrict__ ip_words, T* __restrict__ update,
                                                              int n, unsigned* __restrict__ msg_words, long long capacity,
                                                              int* __restrict__ size_prefix, int* __restrict__ result) {
    constexpr int PW = Elem<T>::pair_words;
    if ((long long)result[0] <= capacity) return;
    const unsigned k = ip_words[1];
    if (update) {
        for (unsigned j = blockIdx.x * kBlock + threadIdx.x; j < k; j += gridDim.x * kBlock) {
            const unsigned* w = ip_words + 2 + (size_t)PW * j;
            if (w[0] < (unsigned)n) store_words<T>(reinterpret_cast<unsigned*>(update + w[0]), load_words<T>(w + 1));
        }
    }
    __threadfence();
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) {
        int bytes = 0;
        if (capacity >= 20) {
            msg_words[0] = (unsigned)n;
            msg_words[1] = 0u;
            msg_words[2] = n > 0 ? 1u : 0u;
            msg_words[3] = 0u;
            msg_words[4] = (unsigned)n;
            bytes = n > 0 ? 20 : 16;
        }
        if (size_prefix) *size_prefix = bytes;
        // result[0] is read by the other blocks of this kernel: it keeps the true size (the host
        // compares it with the capacity and reports CX_ERR_CAPACITY)
    }
}

// ---- decode: prefix sums over the run lengths ---------------------------------------------
// run r is a "sent" run when its parity matches signum
__device__ __forceinline__ bool run_is_sent(unsigned r, int signum) { return ((r & 1u) == 0u) == (signum != 0); }

__global__ __launch_bounds__(kBlock) void rle_scan_sums_kernel(const int* __restrict__ lens, int runs, int signum,
                                                               unsigned* __restrict__ sums) {
    __shared__ unsigned s_len, s_sent;
    if (threadIdx.x == 0) s_len = s_sent = 0u;
    __syncthreads();
    unsigned len = 0, sent = 0;
    const long long base = (long long)blockIdx.x * kBlock * kScanItems;
    for (int q = 0; q < kScanItems; ++q) {
        const long long r = base + (long long)q * kBlock + threadIdx.x;
        if (r < runs) {
            const unsigned l = (unsigned)lens[r];
            len += l;
            if (run_is_sent((unsigned)r, signum)) sent += l;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        len += __shfl_xor(len, off, 64);
        sent += __shfl_xor(sent, off, 64);
    }
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&s_len, len);  // LDS
        atomicAdd(&s_sent, sent);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        sums[2 * blockIdx.x] = s_len;
        sums[2 * blockIdx.x + 1] = s_sent;
    }
}

// exclusive prefix sums of the per-block sums, in place; one block
__global__ __launch_bounds__(kBlock) void rle_scan_top_kernel(unsigned* __restrict__ sums, int nblocks) {
    __shared__ unsigned s_wave[kBlock / 64];
    unsigned carry_len = 0, carry_sent = 0;
    for (int b0 = 0; b0 < nblocks; b0 += kBlock) {
        const int b = b0 + threadIdx.x;
        const unsigned len = b < nblocks ? sums[2 * b] : 0u;
        const unsigned sent = b < nblocks ? sums[2 * b + 1] : 0u;
        unsigned tot_len, tot_sent;
        const unsigned incl_len = block_inclusive_scan(len, s_wave, &tot_len);
        const unsigned incl_sent = block_inclusive_scan(sent, s_wave, &tot_sent);
        if (b < nblocks) {
            sums[2 * b] = carry_len + incl_len - len;
            sums[2 * b + 1] = carry_sent + incl_sent - sent;
        }
        carry_len += tot_len;
        carry_sent += tot_sent;
    }
}

// pos[r] = elements before run r, voff[r] = sent values before run r
__global__ __launch_bounds__(kBlock) void rle_scan_apply_kernel(const int* __restrict__ lens, int runs, int signum,
                                                                const unsigned* __restrict__ sums,
                                                                unsigned* __restrict__ pos, unsigned* __restrict__ voff) {
    __shared__ unsigned s_wave[kBlock / 64];
    unsigned carry_len = sums[2 * blockIdx.x], carry_sent = sums[2 * blockIdx.x + 1];
    const long long base = (long long)blockIdx.x * kBlock * kScanItems;
    for (int q = 0; q < kScanItems; ++q) {
        const long long r = base + (long long)q * kBlock + threadIdx.x;
        const unsigned len = r < runs ? (unsigned)lens[r] : 0u;
        const unsigned sent = (r < runs && run_is_sent((unsigned)r, signum)) ? len : 0u;
        unsigned tot_len, tot_sent;
        const unsigned incl_len = block_inclusive_scan(len, s_wave, &tot_len);
        const unsigned incl_sent = block_inclusive_scan(sent, s_wave, &tot_sent);
        if (r < runs) {
            pos[r] = carry_len + incl_len - len;
            voff[r] = carry_sent + incl_sent - sent;
        }
        carry_len += tot_len;
        carry_sent += tot_sent;
    }
}

// one thread per sent value: its run by binary search over the "sent" runs' value offsets
template <typename T, bool ADD>
__global__ __launch_bounds__(kBlock) void rle_scatter_kernel(T* __restrict__ out, int n, const unsigned* __restrict__ values,
                                                             int c, int runs, int signum,
                                                             const unsigned* __restrict__ pos,
                                                             const unsigned* __restrict__ voff, DeviceStatus* status) {
    constexpr int VW = (int)sizeof(T) / 4;
    const unsigned first = signum ? 0u : 1u;  // first "sent" run
    if ((unsigned)runs <= first) return;
    const unsigned sent_runs = ((unsigned)runs - first + 1u) / 2u;
    const long long stride = (long long)gridDim.x * kBlock;
    bool bad = false;
    for (long long j = (long long)blockIdx.x * kBlock + threadIdx.x; j < c; j += stride) {
        unsigned lo = 0, hi = sent_runs - 1u;  // largest y with voff[first + 2y] <= j
        while (lo < hi) {
            const unsigned mid = (lo + hi + 1u) >> 1;
            if (voff[first + 2u * mid] <= (unsigned)j) lo = mid;
            else hi = mid - 1u;
        }
        const unsigned r = first + 2u * lo;
        const unsigned long long at = (unsigned long long)pos[r] + ((unsigned)j - voff[r]);
        if (at >= (unsigned long long)n) {  // a message whose runs do not add up
            bad = true;
            continue;
        }
        const T v = load_words<T>(values + (size_t)j * VW);
        out[at] = ADD ? (T)(out[at] + v) : v;
    }
    if (bad) atomicCAS(&status->code, 0, (int)CX_ERR_INDEX);
}

int ensure_bytes(cx_handle h, void** p, size_t* have, size_t need) {
    if (need <= *have) return CX_OK;
    CX_HIP(hipStreamSynchronize(h->stream));
    if (*p) CX_HIP(hipFree(*p));
    *p = nullptr;
    *have = 0;
    CX_HIP(hipMalloc(p, need + 256));
    *have = need;
    return CX_OK;
}

}  // namespace

template <typename T>
int launch_rle_compress(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                        const T* thr_host, const T* d_thr, int* d_size_prefix, int* d_result) {
    constexpr int kPairBytes = 4 * Elem<T>::pair_words;
    if (!out_msg || n < 0) return fail(CX_ERR_INVALID, "compress: null message buffer or negative size");
    if ((reinterpret_cast<uintptr_t>(out_msg) & 3u) != 0)
        return fail(CX_ERR_INVALID, "compress: message buffer must be 4-byte aligned");
    if (!data && !update && n > 0) return fail(CX_ERR_INVALID, "Compression needs a valid input vector!");
    // the pairs of every element that could be sent
    const size_t ip_bytes = 8 + (size_t)n * kPairBytes;
    int rc = ensure_bytes(h, &h->rle_pairs, &h->rle_pairs_bytes, ip_bytes);
    if (rc != CX_OK) return rc;
    rc = ensure_bytes(h, reinterpret_cast<void**>(&h->rle_scan), &h->rle_scan_bytes, (size_t)kConvBlocks * sizeof(unsigned));
    if (rc != CX_OK) return rc;
    T* d_strict = reinterpret_cast<T*>(static_cast<char*>(h->d_thr) + 192);
    hipLaunchKernelGGL(rle_threshold_kernel<T>, dim3(1), dim3(1), 0, h->stream, thr_host ? nullptr : (d_thr ? d_thr : static_cast<const T*>(h->d_thr)),
                       thr_host ? *thr_host : (T)0, d_strict);
    rc = launch_compact<T>(h, h->rle_pairs, (long long)ip_bytes, data, update, n, nullptr, d_strict, nullptr);
    if (rc != CX_OK) return rc;
    const unsigned* ip_words = static_cast<const unsigned*>(h->rle_pairs);
    unsigned* msg_words = static_cast<unsigned*>(out_msg);
    const long long cap_words = out_capacity / 4;
    hipLaunchKernelGGL(rle_count_kernel<T>, dim3(kConvBlocks), dim3(kBlock), 0, h->stream, ip_words, h->rle_scan);
    hipLaunchKernelGGL((rle_write_kernel<T, false>), dim3(kConvBlocks), dim3(kBlock), 0, h->stream, ip_words, h->rle_scan, n,
                       msg_words, cap_words, d_size_prefix, d_result, h->d_status);
    hipLaunchKernelGGL((rle_write_kernel<T, true>), dim3(kConvBlocks), dim3(kBlock), 0, h->stream, ip_words, h->rle_scan, n,
                       msg_words, cap_words, d_size_prefix, d_result, h->d_status);
    hipLaunchKernelGGL(rle_overflow_kernel<T>, dim3(kConvBlocks), dim3(kBlock), 0, h->stream, ip_words, update, n, msg_words,
                       out_capacity, d_size_prefix, d_result);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

// Reads the message's four header fields (two dependent host reads), then decodes.
template <typename T>
int launch_rle_decode(cx_handle h, T* out, int out_n, const void* msg, int add, int* n_out) {
    if (!out || !msg || out_n < 0) return fail(CX_ERR_INVALID, "decompress: bad arguments");
    const unsigned* words = static_cast<const unsigned*>(msg);
    constexpr int VW = (int)sizeof(T) / 4;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, words, 8, hipMemcpyDeviceToHost, h->stream));
    CX_HIP(hipStreamSynchronize(h->stream));
    const int n = h->h_pinned[8], c = h->h_pinned[9];
    if (n_out) *n_out = n;
    if (n > out_n) return fail(CX_ERR_MSG_TOO_LARGE, "Decompression vector size is bigger than output buffer!");
    if (n < 0 || c < 0 || c > n) return fail(CX_ERR_INVALID, "run-length message: bad header (n %d, values %d)", n, c);
    const unsigned* trailer = words + 2 + (size_t)c * VW;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, trailer, 8, hipMemcpyDeviceToHost, h->stream));
    CX_HIP(hipStreamSynchronize(h->stream));
    const int runs = h->h_pinned[8], signum = h->h_pinned[9];
    if (runs < 0 || runs > n + 1) return fail(CX_ERR_INVALID, "run-length message: bad run count %d", runs);
    if (!add) {  // every position of the vector is either a sent value or a zero
        int rc = launch_zero<T>(h, out, n);
        if (rc != CX_OK) return rc;
    }
    if (c == 0 || runs == 0) return CX_OK;
    const int nblocks = (runs + kBlock * kScanItems - 1) / (kBlock * kScanItems);
    const size_t need = ((size_t)2 * nblocks + (size_t)2 * runs) * sizeof(unsigned);
    int rc = ensure_bytes(h, reinterpret_cast<void**>(&h->rle_scan), &h->rle_scan_bytes, need);
    if (rc != CX_OK) return rc;
    unsigned* sums = h->rle_scan;
    unsigned* pos = sums + (size_t)2 * nblocks;
    unsigned* voff = pos + runs;
    const int* lens = reinterpret_cast<const int*>(trailer + 2);
    hipLaunchKernelGGL(rle_scan_sums_kernel, dim3(nblocks), dim3(kBlock), 0, h->stream, lens, runs, signum, sums);
    hipLaunchKernelGGL(rle_scan_top_kernel, dim3(1), dim3(kBlock), 0, h->stream, sums, nblocks);
    hipLaunchKernelGGL(rle_scan_apply_kernel, dim3(nblocks), dim3(kBlock), 0, h->stream, lens, runs, signum, sums, pos, voff);
    int grid = (c + kBlock - 1) / kBlock;
    if (grid > 4096) grid = 4096;
    if (add)
        hipLaunchKernelGGL((rle_scatter_kernel<T, true>), dim3(grid), dim3(kBlock), 0, h->stream, out, n, words + 2, c, runs,
                           signum, pos, voff, h->d_status);
    else
        hipLaunchKernelGGL((rle_scatter_kernel<T, false>), dim3(grid), dim3(kBlock), 0, h->stream, out, n, words + 2, c, runs,
                           signum, pos, voff, h->d_status);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T> int reserve_rle(cx_handle h, int n) {
    int rc = ensure_bytes(h, &h->rle_pairs, &h->rle_pairs_bytes, 8 + (size_t)n * 4 * Elem<T>::pair_words);
    if (rc != CX_OK) return rc;
    rc = ensure_bytes(h, reinterpret_cast<void**>(&h->rle_scan), &h->rle_scan_bytes, (size_t)kConvBlocks * sizeof(unsigned));
    if (rc != CX_OK) return rc;
    return reserve_compact<T>(h, n);  // the pairs are made by the compaction
}
template int reserve_rle<float>(cx_handle, int);
template int reserve_rle<double>(cx_handle, int);
template int reserve_rle<int>(cx_handle, int);

#define CX_INSTANTIATE_RLE(T)                                                                                   \
    template int launch_rle_compress<T>(cx_handle, void*, long long, const T*, T*, int, const T*, const T*, int*, int*); \
    template int launch_rle_decode<T>(cx_handle, T*, int, const void*, int, int*);
CX_INSTANTIATE_RLE(float)
CX_INSTANTIATE_RLE(double)
CX_INSTANTIATE_RLE(int)
#undef CX_INSTANTIATE_RLE

}  // namespace cx
