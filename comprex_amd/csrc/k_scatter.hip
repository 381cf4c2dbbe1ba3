// Receive side of the IndexPairs codec and the residual's streaming maintenance.
//
//   decompress  CompressorIndexPairs<T>::decompression_strategy (reference src/compressor.hxx:613-638)
//   add         CompressorIndexPairs<T>::add_strategy            (:640-658)
//   reduce      the chief's rank-ordered loop of Comprex_AllToOneAllreduce::apply (src/allreduce.tpp:183-189)
//   zero / add_vec / threshold_apply
//               ComprEx<T>::resetRests, addRests (src/comprEx.tpp:121-126,159-169),
//               ThresholdFunction<T>::apply / apply_split (src/threshold.hxx:19-50)
//
// A message's header (n, k) is read on the device, so no host round trip is needed to
// size the work.  Indices inside one message are non-decreasing (the compressor emits
// them strictly ascending); a run of equal indices is applied by the thread that owns
// the run's first pair, in message order, so the result equals the sequential loop's
// without atomics.  Summing several messages in a fixed order is done one message after
// the other (stream order) or, in the tiled variant, rank by rank inside an LDS tile.
#include "cx_common.hpp"

namespace cx {

namespace {

constexpr int kBlock = 256;

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T x[V]; };

__device__ __forceinline__ float mag(float v) { return fabsf(v); }
__device__ __forceinline__ double mag(double v) { return fabs(v); }
__device__ __forceinline__ int mag(int v) { return v < 0 ? -v : v; }

template <typename T> __device__ __forceinline__ T load_value(const unsigned* w);
template <> __device__ __forceinline__ float load_value<float>(const unsigned* w) { return __uint_as_float(w[0]); }
template <> __device__ __forceinline__ int load_value<int>(const unsigned* w) { return (int)w[0]; }
template <> __device__ __forceinline__ double load_value<double>(const unsigned* w) {
    return __longlong_as_double((long long)(((unsigned long long)w[1] << 32) | w[0]));
}

__device__ __forceinline__ void atomic_accumulate(float* p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_accumulate(double* p, double v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_accumulate(int* p, int v) { atomicAdd(p, v); }

// OP 0: out[idx] = val (last pair of a run wins)   OP 1: out[idx] += val in order   OP 2: atomic +=
template <typename T, int OP>
__global__ __launch_bounds__(kBlock) void scatter_kernel(T* __restrict__ out, int out_n,
                                                         const unsigned* __restrict__ msg, DeviceStatus* status) {
    constexpr int PW = Elem<T>::pair_words;
    const int n_msg = (int)msg[0];
    const long long k = (long long)(int)msg[1];
    if (n_msg > out_n) {
        if (blockIdx.x == 0 && threadIdx.x == 0) atomicCAS(&status->code, 0, (int)CX_ERR_MSG_TOO_LARGE);
        return;
    }
    const unsigned* pairs = msg + 2;
    const long long stride = (long long)gridDim.x * kBlock;
    bool bad = false;
    for (long long j = (long long)blockIdx.x * kBlock + threadIdx.x; j < k; j += stride) {
        const unsigned* p = pairs + PW * j;
        const int idx = (int)p[0];
        if ((unsigned)idx >= (unsigned)out_n) {
            bad = true;
            continue;
        }
        if (OP == 2) {
            atomic_accumulate(out + idx, load_value<T>(p + 1));
        } else if (OP == 1) {
            if (j > 0 && (int)p[-PW] == idx) continue;  // not the head of its run
            T acc = out[idx];
            long long q = j;
            do {
                acc = (T)(acc + load_value<T>(pairs + PW * q + 1));
                ++q;
            } while (q < k && (int)pairs[PW * q] == idx);
            out[idx] = acc;
        } else {
            if (j + 1 < k && (int)p[PW] == idx) continue;  // a later pair overwrites this one
            out[idx] = load_value<T>(p + 1);
        }
    }
    if (bad) atomicCAS(&status->code, 0, (int)CX_ERR_INDEX);
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void zero_kernel(T* __restrict__ v, long long n) {
    const long long stride = (long long)gridDim.x * kBlock;
    const long long nvec = n / VEC;
    Pack<T, VEC> z;
#pragma unroll
    for (int c = 0; c < VEC; ++c) z.x[c] = (T)0;
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += stride)
        reinterpret_cast<Pack<T, VEC>*>(v)[i] = z;
    for (long long i = nvec * VEC + (long long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) v[i] = (T)0;
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void add_vec_kernel(T* __restrict__ data, const T* __restrict__ rests,
                                                         long long n) {
    const long long stride = (long long)gridDim.x * kBlock;
    const long long nvec = n / VEC;
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += stride) {
        Pack<T, VEC> a = reinterpret_cast<Pack<T, VEC>*>(data)[i];
        const Pack<T, VEC> b = reinterpret_cast<const Pack<T, VEC>*>(rests)[i];
#pragma unroll
        for (int c = 0; c < VEC; ++c) a.x[c] = (T)(a.x[c] + b.x[c]);
        reinterpret_cast<Pack<T, VEC>*>(data)[i] = a;
    }
    for (long long i = nvec * VEC + (long long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        data[i] = (T)(data[i] + rests[i]);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void threshold_apply_kernel(T* __restrict__ high, T* __restrict__ low,
                                                                 const T* __restrict__ in, long long n,
                                                                 const T* __restrict__ thr_ptr, T thr_val) {
    const T thr = thr_ptr ? *thr_ptr : thr_val;
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const T v = in[i];
        const bool keep = mag(v) >= thr;  // '>=' here, '>' in the compressor
        high[i] = keep ? v : (T)0;
        if (low) low[i] = keep ? (T)0 : v;
    }
}

inline unsigned grid_for(long long work_items, long long per_thread) {
    long long blocks = (work_items + kBlock * per_thread - 1) / (kBlock * per_thread);
    if (blocks < 1) blocks = 1;
    if (blocks > 4096) blocks = 4096;
    return (unsigned)blocks;
}

}  // namespace

template <typename T> int launch_zero(cx_handle h, T* v, int n) {
    if (n < 0 || (!v && n > 0)) return fail(CX_ERR_INVALID, "zero: bad arguments");
    if (n == 0) return CX_OK;
    constexpr int kVec = 16 / (int)sizeof(T);
    if ((reinterpret_cast<uintptr_t>(v) & 15u) == 0)
        hipLaunchKernelGGL((zero_kernel<T, kVec>), dim3(grid_for(n, 4 * kVec)), dim3(kBlock), 0, h->stream, v,
                           (long long)n);
    else
        hipLaunchKernelGGL((zero_kernel<T, 1>), dim3(grid_for(n, 4)), dim3(kBlock), 0, h->stream, v, (long long)n);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T> int launch_add_vec(cx_handle h, T* data, const T* rests, int n) {
    if (n < 0 || ((!data || !rests) && n > 0)) return fail(CX_ERR_INVALID, "add_vec: bad arguments");
    if (n == 0) return CX_OK;
    constexpr int kVec = 16 / (int)sizeof(T);
    if (((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(rests)) & 15u) == 0)
        hipLaunchKernelGGL((add_vec_kernel<T, kVec>), dim3(grid_for(n, 4 * kVec)), dim3(kBlock), 0, h->stream, data,
                           rests, (long long)n);
    else
        hipLaunchKernelGGL((add_vec_kernel<T, 1>), dim3(grid_for(n, 4)), dim3(kBlock), 0, h->stream, data, rests,
                           (long long)n);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T>
int launch_threshold_apply(cx_handle h, T* high, T* low, const T* in, int n, const T* thr_host, const T* d_thr) {
    if (n < 0 || ((!high || !in) && n > 0)) return fail(CX_ERR_INVALID, "threshold_apply: bad arguments");
    if (n == 0) return CX_OK;
    const T thr_val = thr_host ? *thr_host : (T)0;
    const T* thr_ptr = thr_host ? nullptr : (d_thr ? d_thr : static_cast<const T*>(h->d_thr));
    hipLaunchKernelGGL(threshold_apply_kernel<T>, dim3(grid_for(n, 4)), dim3(kBlock), 0, h->stream, high, low, in,
                       (long long)n, thr_ptr, thr_val);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T> int launch_add(cx_handle h, T* out, int out_n, const void* msg, int atomic) {
    if (!out || !msg || out_n < 0) return fail(CX_ERR_INVALID, "add: bad arguments");
    const unsigned* words = static_cast<const unsigned*>(msg);
    const unsigned grid = grid_for(out_n, 1);  // k <= n <= out_n for any message that passes the size check
    if (atomic)
        hipLaunchKernelGGL((scatter_kernel<T, 2>), dim3(grid), dim3(kBlock), 0, h->stream, out, out_n, words,
                           h->d_status);
    else
        hipLaunchKernelGGL((scatter_kernel<T, 1>), dim3(grid), dim3(kBlock), 0, h->stream, out, out_n, words,
                           h->d_status);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T> int launch_decompress(cx_handle h, T* out, int out_n, const void* msg) {
    if (!out || !msg || out_n < 0) return fail(CX_ERR_INVALID, "decompress: bad arguments");
    int rc = launch_zero<T>(h, out, out_n);  // the whole output, also when the size check fails afterwards
    if (rc != CX_OK) return rc;
    hipLaunchKernelGGL((scatter_kernel<T, 0>), dim3(grid_for(out_n, 1)), dim3(kBlock), 0, h->stream, out, out_n,
                       static_cast<const unsigned*>(msg), h->d_status);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T>
int launch_reduce(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int accumulate, int mode) {
    if (!out || out_n < 0 || n_msgs < 0 || (n_msgs > 0 && !msgs)) return fail(CX_ERR_INVALID, "reduce: bad arguments");
    if (!accumulate) {
        int rc = launch_zero<T>(h, out, out_n);
        if (rc != CX_OK) return rc;
    }
    for (int r = 0; r < n_msgs; ++r) {
        int rc = launch_add<T>(h, out, out_n, msgs[r], mode == 1);
        if (rc != CX_OK) return rc;
    }
    return CX_OK;
}

#define CX_INSTANTIATE(T)                                                                         \
    template int launch_zero<T>(cx_handle, T*, int);                                              \
    template int launch_add_vec<T>(cx_handle, T*, const T*, int);                                 \
    template int launch_threshold_apply<T>(cx_handle, T*, T*, const T*, int, const T*, const T*); \
    template int launch_add<T>(cx_handle, T*, int, const void*, int);                             \
    template int launch_decompress<T>(cx_handle, T*, int, const void*);                           \
    template int launch_reduce<T>(cx_handle, T*, int, const void* const*, int, int, int);
CX_INSTANTIATE(float)
CX_INSTANTIATE(double)
CX_INSTANTIATE(int)

}  // namespace cx
