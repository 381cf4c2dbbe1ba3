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

// ---- tiled, rank-ordered reduce ------------------------------------------------------------
// out (+)= sum of up to kMaxMsgs index-sorted messages, applied in the order given, with the
// dense vector written exactly once:
//   bounds_kernel  one pass over every message's indices: for every dense tile t, the first
//                  pair of each message whose index is >= t * kReduceTile (plus an end marker);
//   tiled_kernel   one block per dense tile: the tile starts as zeros (or the old contents),
//                  lives in LDS, receives message 0's pairs, then message 1's, ... (a barrier
//                  between messages keeps the order of additions; pairs of one message never
//                  collide), and is streamed out.
// Traffic: 4 B per dense element written (+4 read when accumulating) + 8 B per pair, against
// one read-modify-write of a scattered 4-byte element per pair for the per-message scatter.
#ifndef CX_REDUCE_TILE_BYTES
#define CX_REDUCE_TILE_BYTES 16384
#endif
template <typename T> struct ReduceTile { static constexpr int value = CX_REDUCE_TILE_BYTES / (int)sizeof(T); };
constexpr int kMaxMsgs = 16;

struct MsgList {
    const unsigned* msg[kMaxMsgs];
};

// bounds[t * kMaxMsgs + r] = first pair of message r whose index is >= t * (tile elements), for
// t in [0, ntiles]; blockIdx.y selects the message.
template <typename T>
__global__ __launch_bounds__(kBlock) void bounds_kernel(MsgList list, int out_n, unsigned ntiles,
                                                        unsigned* __restrict__ bounds, DeviceStatus* status) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int kReduceTile = ReduceTile<T>::value;
    const int r = blockIdx.y;
    const unsigned* msg = list.msg[r];
    const int n_msg = (int)msg[0];
    long long k = (long long)(int)msg[1];
    if (n_msg > out_n || k < 0) k = 0;  // reported by the tile kernel; no pair of it is applied
    const unsigned* pairs = msg + 2;
    const long long stride = (long long)gridDim.x * kBlock;
    bool bad = false;
    // pair j opens every tile in (tile(j-1), tile(j)]; "pair" k closes the remaining ones
    for (long long j = (long long)blockIdx.x * kBlock + threadIdx.x; j <= k; j += stride) {
        long long t_prev = -1, t_here = ntiles;  // j == 0 opens from tile 0; j == k closes up to ntiles
        if (j > 0) {
            const int ip = (int)pairs[PW * (j - 1)];
            if ((unsigned)ip >= (unsigned)out_n) bad = true;
            t_prev = (unsigned)ip >= (unsigned)out_n ? (long long)ntiles - 1 : ip / kReduceTile;
        }
        if (j < k) {
            const int ih = (int)pairs[PW * j];
            if ((unsigned)ih >= (unsigned)out_n) bad = true;
            t_here = (unsigned)ih >= (unsigned)out_n ? (long long)ntiles - 1 : ih / kReduceTile;
            if (j > 0 && t_here < t_prev) {  // not sorted: cannot be tiled
                bad = true;
                t_here = t_prev;
            }
        }
        for (long long t = t_prev + 1; t <= t_here; ++t) bounds[(size_t)t * kMaxMsgs + r] = (unsigned)j;
    }
    if (bad) atomicCAS(&status->code, 0, (int)CX_ERR_INDEX);
}

// OP 0: out = scatter of the (single) message, last pair of a run of equal indices wins;
// OP 1: out (+)= messages in order.  RMAX: how many messages the launch may carry (register budget).
template <typename T, int OP, bool ACCUM, int RMAX>
__global__ __launch_bounds__(kBlock) void tiled_kernel(T* __restrict__ out, int out_n, MsgList list, int n_msgs,
                                                       unsigned ntiles, const unsigned* __restrict__ bounds,
                                                       DeviceStatus* status) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int kReduceTile = ReduceTile<T>::value;
    __shared__ T tile[kReduceTile];
    const int tid = threadIdx.x, lane = tid & 63;
    const unsigned t = blockIdx.x;
    const long long base = (long long)t * kReduceTile;
    const int valid = (int)((long long)out_n - base < kReduceTile ? (long long)out_n - base : kReduceTile);

    // this tile's slice of every message (the same for all threads: scalar loads), clamped to the
    // message because the bounds of a message that is not index-sorted are meaningless
    const unsigned* bt = bounds + (size_t)t * kMaxMsgs;
    long long lo[RMAX], hi[RMAX];
    bool too_large = false;
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        lo[r] = hi[r] = 0;
        if (r < n_msgs) {
            const unsigned* msg = list.msg[r];
            const long long k = (long long)(int)msg[1];
            lo[r] = bt[r];
            hi[r] = bt[kMaxMsgs + r];
            if (hi[r] > k) hi[r] = k;
            if (lo[r] > hi[r]) lo[r] = hi[r];
            too_large |= (int)msg[0] > out_n;
        }
    }
    if (too_large) {
        if (t == 0 && tid == 0) atomicCAS(&status->code, 0, (int)CX_ERR_MSG_TOO_LARGE);
        if (ACCUM) return;  // add: nothing is touched
        n_msgs = 0;         // decompress: the output is zeroed all the same
    }

    // every message's pairs for this tile are fetched before any is applied: one pair per thread
    // and message (the common case); longer slices are finished from memory below.  p_edge holds
    // what the neighbouring wavefront would have supplied: the previous pair's index for lane 0,
    // the next pair's for lane 63.
    unsigned p_idx[RMAX], p_edge[RMAX];
    T p_val[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        p_idx[r] = p_edge[r] = 0xffffffffu;
        p_val[r] = (T)0;
        if (r < n_msgs) {
            const long long j = lo[r] + tid;
            if (j < hi[r]) {
                const unsigned* p = list.msg[r] + 2 + PW * j;
                p_idx[r] = p[0];
                p_val[r] = load_value<T>(p + 1);
                if (lane == 0 && j > lo[r]) p_edge[r] = p[-PW];
                if (lane == 63 && j + 1 < hi[r]) p_edge[r] = p[PW];
            }
        }
    }

    const bool vec_ok = (reinterpret_cast<uintptr_t>(out) & 15u) == 0 && valid == kReduceTile;
    if (ACCUM) {
        if (vec_ok) {
            for (int i = tid * VEC; i < kReduceTile; i += kBlock * VEC)
                *reinterpret_cast<Pack<T, VEC>*>(&tile[i]) = *reinterpret_cast<const Pack<T, VEC>*>(out + base + i);
        } else {
            for (int i = tid; i < valid; i += kBlock) tile[i] = out[base + i];
        }
    } else {
        for (int i = tid; i < kReduceTile; i += kBlock) tile[i] = (T)0;
    }
    __syncthreads();

#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        if (r < n_msgs) {
            const unsigned* pairs = list.msg[r] + 2;
            // neighbours inside the wavefront hold the adjacent pairs of the same message
            unsigned prev = __shfl_up(p_idx[r], 1, 64), next = __shfl_down(p_idx[r], 1, 64);
            if (lane == 0) prev = p_edge[r];
            if (lane == 63) next = p_edge[r];
            for (long long j = lo[r] + tid; j < hi[r]; j += kBlock) {
                unsigned idx;
                T val;
                if (j == lo[r] + tid) {
                    idx = p_idx[r];
                    val = p_val[r];
                    if (j == lo[r]) prev = 0xffffffffu;
                    if (j + 1 >= hi[r]) next = 0xffffffffu;
                } else {  // slices longer than the block: straight from memory
                    const unsigned* p = pairs + PW * j;
                    idx = p[0];
                    val = load_value<T>(p + 1);
                    prev = p[-PW];
                    next = j + 1 < hi[r] ? p[PW] : 0xffffffffu;
                }
                const unsigned local = (unsigned)((long long)(int)idx - base);
                if (local >= (unsigned)valid) continue;  // index outside the vector: reported by bounds_kernel
                if (OP == 0) {
                    if (next == idx) continue;  // a later pair overwrites this one
                    tile[local] = val;
                } else {
                    if (prev == idx) continue;  // not the head of its run
                    T acc = (T)(tile[local] + val);
                    if (next == idx) {  // a run of equal indices: add the rest in message order
                        long long q = j + 1;
                        do {
                            acc = (T)(acc + load_value<T>(pairs + PW * q + 1));
                            ++q;
                        } while (q < hi[r] && pairs[PW * q] == idx);
                    }
                    tile[local] = acc;
                }
            }
            __syncthreads();  // the next message's additions come after this one's
        }
    }

    if (vec_ok) {
        for (int i = tid * VEC; i < kReduceTile; i += kBlock * VEC)
            *reinterpret_cast<Pack<T, VEC>*>(out + base + i) = *reinterpret_cast<const Pack<T, VEC>*>(&tile[i]);
    } else {
        for (int i = tid; i < valid; i += kBlock) out[base + i] = tile[i];
    }
}

template <typename T>
int launch_tiled(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int op, int accumulate) {
    if (out_n == 0) return CX_OK;
    constexpr int kReduceTile = ReduceTile<T>::value;
    const unsigned ntiles = (unsigned)(((long long)out_n + kReduceTile - 1) / kReduceTile);
    const size_t need = (size_t)kMaxMsgs * (ntiles + 1);
    if (need > h->reduce_bounds_cap) {
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->reduce_bounds) CX_HIP(hipFree(h->reduce_bounds));
        h->reduce_bounds = nullptr;
        h->reduce_bounds_cap = 0;
        CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->reduce_bounds), need * sizeof(unsigned)));
        h->reduce_bounds_cap = need;
    }
    for (int first = 0; first < n_msgs || first == 0; first += kMaxMsgs) {
        MsgList list;
        const int cnt = n_msgs - first < kMaxMsgs ? n_msgs - first : kMaxMsgs;
        for (int r = 0; r < kMaxMsgs; ++r) list.msg[r] = r < cnt ? static_cast<const unsigned*>(msgs[first + r]) : nullptr;
        if (cnt > 0) {
            unsigned grid = (unsigned)(((long long)out_n / 64 + kBlock - 1) / kBlock);  // k <= n: ~1 thread per 64 elements
            if (grid < 1) grid = 1;
            if (grid > 1024) grid = 1024;
            hipLaunchKernelGGL(bounds_kernel<T>, dim3(grid, cnt), dim3(kBlock), 0, h->stream, list, out_n, ntiles,
                               h->reduce_bounds, h->d_status);
        }
        const bool acc = accumulate || first > 0;
#define CX_TILED(OP, ACC, RMAX)                                                                                     \
    hipLaunchKernelGGL((tiled_kernel<T, OP, ACC, RMAX>), dim3(ntiles), dim3(kBlock), 0, h->stream, out, out_n, list, \
                       cnt, ntiles, h->reduce_bounds, h->d_status)
        if (op == 0) CX_TILED(0, false, 1);
        else if (cnt <= 8) { if (acc) CX_TILED(1, true, 8); else CX_TILED(1, false, 8); }
        else { if (acc) CX_TILED(1, true, kMaxMsgs); else CX_TILED(1, false, kMaxMsgs); }
#undef CX_TILED
        if (n_msgs == 0) break;
    }
    CX_HIP(hipGetLastError());
    return CX_OK;
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
    if (h->reduce_variant == 0) return launch_tiled<T>(h, out, out_n, &msg, 1, 0, 0);
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
    if (mode == 0 && h->reduce_variant == 0) return launch_tiled<T>(h, out, out_n, msgs, n_msgs, 1, accumulate);
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
