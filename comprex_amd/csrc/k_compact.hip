// Fused error-feedback accumulate + magnitude select + ordered compaction + residual zeroing.
//
// Replaces the sequential loop of CompressorIndexPairs<T>::compression_strategy
// (reference src/compressor.hxx:556-611).  One pass over the vector:
//
//   - each 256-thread block takes one tile of 256*VEC*ITEMS consecutive elements with
//     16-byte vector loads, lane-contiguous so a wavefront reads 1 KiB per instruction;
//   - s = update + data (one IEEE add, as the reference's `update[i] += data[i]`),
//     survivors are |s| > threshold (strict; NaN never survives);
//   - the rank of a survivor inside the tile comes from wavefront ballots + popcounts,
//     tile totals are chained across tiles with a decoupled look-back over 64-bit
//     descriptors {count, launch epoch, state}, so pairs land in ascending index order
//     exactly as the sequential loop writes them;
//   - the residual is written back once with survivors replaced by +0.
//
// HBM traffic per element (fp32): 4 B data + 4 B residual in, 4 B residual out, plus 8 B
// per survivor.  No scratch traffic beyond one 8-byte descriptor per tile.
//
// Every wait on another tile is bounded: a wave that exhausts its spin budget records
// CX_ERR_INTERNAL in the status word and carries on with a zero prefix, so the grid
// always drains.
#include "cx_common.hpp"

namespace cx {

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;
constexpr unsigned kSpinLimit = 1u << 22;

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T x[V]; };

__device__ __forceinline__ float mag(float v) { return fabsf(v); }
__device__ __forceinline__ double mag(double v) { return fabs(v); }
__device__ __forceinline__ int mag(int v) { return v < 0 ? -v : v; }

__device__ __forceinline__ unsigned word_of(float v) { return __float_as_uint(v); }
__device__ __forceinline__ unsigned word_of(int v) { return (unsigned)v; }

// descriptor: [63:32] value | [31:2] epoch | [1:0] state (1 = tile count, 2 = inclusive prefix)
__device__ __forceinline__ unsigned long long make_desc(unsigned value, unsigned epoch, unsigned state) {
    return ((unsigned long long)value << 32) | ((unsigned long long)(epoch << 2) | state);
}

__device__ __forceinline__ unsigned wave_sum(unsigned v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Exclusive prefix of tile `tile`: sum of the counts of tiles [0, tile).  Run by one
// full wavefront; every lane returns the same value.
__device__ unsigned look_back(const unsigned long long* desc, unsigned tile, unsigned epoch, int lane,
                              DeviceStatus* status) {
    unsigned running = 0;
    int top = (int)tile - 1;  // nearest predecessor still to be accounted for
    while (top >= 0) {
        const int idx = top - lane;  // lane 0 looks at the nearest predecessor
        unsigned long long d = 0;
        unsigned spins = 0;
        bool ready;
        for (;;) {
            ready = true;
            if (idx >= 0) {
                d = __hip_atomic_load(desc + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const unsigned lo = (unsigned)d;
                ready = ((lo >> 2) == epoch) && ((lo & 3u) != 0u);
            }
            if (__all(ready)) break;
            if (++spins > kSpinLimit ||
                ((spins & 1023u) == 0 &&
                 __hip_atomic_load(&status->code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == CX_ERR_INTERNAL)) {
                if (lane == 0) atomicCAS(&status->code, 0, (int)CX_ERR_INTERNAL);
                return running;  // bounded wait expired: give up, the host reports the error
            }
            __builtin_amdgcn_s_sleep(1);
        }
        const unsigned state = (idx >= 0) ? ((unsigned)d & 3u) : 2u;  // before tile 0: prefix 0
        const unsigned value = (idx >= 0) ? (unsigned)(d >> 32) : 0u;
        const unsigned long long has_prefix = __ballot(state == 2u);
        if (has_prefix != 0ull) {
            const int first = __ffsll((long long)has_prefix) - 1;  // nearest tile with a full prefix
            running += wave_sum(lane <= first ? value : 0u);
            return running;
        }
        running += wave_sum(value);
        top -= 64;
    }
    return running;
}

// MODE 0: update += data, select on update, zero selected   (compress_add_update)
// MODE 1: select on update, zero selected                    (compress_update)
// MODE 2: select on data, nothing written back               (compress)
template <typename T, int MODE, int VEC, int ITEMS>
__global__ __launch_bounds__(kBlock) void compact_kernel(
    const T* __restrict__ data, T* __restrict__ update, int n, const T* __restrict__ thr_ptr, T thr_val,
    unsigned* __restrict__ msg_words, long long cap_pairs, int pairs_aligned8, int* __restrict__ size_prefix,
    unsigned long long* __restrict__ tile_desc, unsigned* __restrict__ tile_counter, unsigned counter_base,
    unsigned epoch, unsigned ntiles, int static_tile_ids, DeviceStatus* __restrict__ status) {
    constexpr int kTile = kBlock * VEC * ITEMS;
    constexpr int kPairWords = Elem<T>::pair_words;

    __shared__ unsigned s_tile;
    __shared__ unsigned s_prefix;
    __shared__ unsigned s_wsum[ITEMS][kWaves];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    unsigned tile;
    if (static_tile_ids) {
        tile = blockIdx.x;
    } else {
        if (tid == 0) s_tile = atomicAdd(tile_counter, 1u) - counter_base;
        __syncthreads();
        tile = s_tile;
    }
    if (tile >= ntiles) return;  // cannot happen with a consistent counter; keeps indices in range

    const T thr = thr_ptr ? *thr_ptr : thr_val;
    const long long base = (long long)tile * kTile;
    const bool full = base + kTile <= (long long)n;

    T s[ITEMS][VEC];
    unsigned sel[ITEMS];  // bit c set = element c of load j survives

#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const long long e0 = base + (long long)j * (kBlock * VEC) + (long long)tid * VEC;
        Pack<T, VEC> u, d;
        unsigned valid = 0;
        if (full) {
            if (MODE != 2) u = *reinterpret_cast<const Pack<T, VEC>*>(update + e0);
            if (MODE != 1) d = *reinterpret_cast<const Pack<T, VEC>*>(data + e0);
            valid = (1u << VEC) - 1u;
        } else {
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                const bool in = e0 + c < (long long)n;
                u.x[c] = (MODE != 2 && in) ? update[e0 + c] : (T)0;
                d.x[c] = (MODE != 1 && in) ? data[e0 + c] : (T)0;
                valid |= (in ? 1u : 0u) << c;
            }
        }
        unsigned m = 0;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            T v;
            if (MODE == 0) v = (T)(u.x[c] + d.x[c]);
            else if (MODE == 1) v = u.x[c];
            else v = d.x[c];
            s[j][c] = v;
            m |= ((mag(v) > thr) ? 1u : 0u) << c;
        }
        m &= valid;
        sel[j] = m;
        if (MODE != 2) {
            Pack<T, VEC> w;
#pragma unroll
            for (int c = 0; c < VEC; ++c) w.x[c] = ((m >> c) & 1u) ? (T)0 : s[j][c];
            if (full) {
                if (MODE == 0 || m != 0u) *reinterpret_cast<Pack<T, VEC>*>(update + e0) = w;
            } else {
#pragma unroll
                for (int c = 0; c < VEC; ++c)
                    if (((valid >> c) & 1u) && (MODE == 0 || ((m >> c) & 1u))) update[e0 + c] = w.x[c];
            }
        }
    }

    // ranks inside each (load j, wavefront): lane-major, then element c
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    unsigned rank[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        unsigned before = 0, total = 0;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const unsigned long long b = __ballot((sel[j] >> c) & 1u);
            before += __popcll(b & below);
            total += __popcll(b);
        }
        rank[j] = before;
        if (lane == 0) s_wsum[j][wave] = total;
    }
    __syncthreads();

    // offsets of this wavefront's groups inside the tile, order (j, wave)
    unsigned tile_total = 0;
    unsigned off[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            if (w == wave) off[j] = tile_total;
            tile_total += s_wsum[j][w];
        }
    }

    if (wave == 0) {
        unsigned prefix = 0;
        if (tile == 0) {
            if (lane == 0)
                __hip_atomic_store(tile_desc, make_desc(tile_total, epoch, 2u), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        } else {
            if (lane == 0)
                __hip_atomic_store(tile_desc + tile, make_desc(tile_total, epoch, 1u), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            prefix = look_back(tile_desc, tile, epoch, lane, status);
            if (lane == 0)
                __hip_atomic_store(tile_desc + tile, make_desc(prefix + tile_total, epoch, 2u), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane == 0) s_prefix = prefix;
    }
    __syncthreads();
    const unsigned prefix = s_prefix;

    unsigned* const pairs = msg_words + 2;
    bool overflow = false;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        unsigned m = sel[j];
        if (m == 0u) continue;
        long long pos = (long long)prefix + off[j] + rank[j];
        const long long e0 = base + (long long)j * (kBlock * VEC) + (long long)tid * VEC;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            if ((m >> c) & 1u) {
                if (pos < cap_pairs) {
                    const unsigned index = (unsigned)(e0 + c);
                    if constexpr (kPairWords == 2) {
                        if (pairs_aligned8) {
                            reinterpret_cast<uint2*>(pairs)[pos] = make_uint2(index, word_of(s[j][c]));
                        } else {
                            pairs[2 * pos] = index;
                            pairs[2 * pos + 1] = word_of(s[j][c]);
                        }
                    } else {
                        const unsigned long long bits = (unsigned long long)__double_as_longlong((double)s[j][c]);
                        pairs[3 * pos] = index;
                        pairs[3 * pos + 1] = (unsigned)bits;
                        pairs[3 * pos + 2] = (unsigned)(bits >> 32);
                    }
                } else {
                    overflow = true;
                }
                ++pos;
            }
        }
    }
    if (overflow) atomicCAS(&status->code, 0, (int)CX_ERR_CAPACITY);

    if (tile == ntiles - 1 && tid == 0) {
        const unsigned k = prefix + tile_total;
        msg_words[0] = (unsigned)n;
        msg_words[1] = k;
        if (size_prefix) *size_prefix = (int)(8u + k * (unsigned)(4 * kPairWords));
    }
}

template <typename T, int MODE, int VEC, int ITEMS>
void launch_variant(cx_handle h, const T* data, T* update, int n, const T* thr_ptr, T thr_val, unsigned* msg_words,
                    long long cap_pairs, int aligned8, int* size_prefix, unsigned ntiles) {
    hipLaunchKernelGGL((compact_kernel<T, MODE, VEC, ITEMS>), dim3(ntiles), dim3(kBlock), 0, h->stream, data, update, n,
                       thr_ptr, thr_val, msg_words, cap_pairs, aligned8, size_prefix, h->tile_desc, h->tile_counter,
                       h->counter_base, h->epoch, ntiles, h->compact_tile_ids, h->d_status);
}

template <typename T, int VEC, int ITEMS>
void launch_mode(cx_handle h, int mode, const T* data, T* update, int n, const T* thr_ptr, T thr_val,
                 unsigned* msg_words, long long cap_pairs, int aligned8, int* size_prefix, unsigned ntiles) {
    if (mode == 0)
        launch_variant<T, 0, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                                          size_prefix, ntiles);
    else if (mode == 1)
        launch_variant<T, 1, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                                          size_prefix, ntiles);
    else
        launch_variant<T, 2, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                                          size_prefix, ntiles);
}

__global__ void empty_message_kernel(unsigned* msg_words, int n, int* size_prefix) {
    msg_words[0] = (unsigned)n;
    msg_words[1] = 0u;
    if (size_prefix) *size_prefix = 8;
}

int ensure_descriptors(cx_handle h, size_t ntiles) {
    if (ntiles <= h->tile_desc_cap) return CX_OK;
    size_t cap = h->tile_desc_cap ? h->tile_desc_cap : 4096;
    while (cap < ntiles) cap *= 2;
    // the old array may still be read by a kernel in flight on the stream
    CX_HIP(hipStreamSynchronize(h->stream));
    if (h->tile_desc) CX_HIP(hipFree(h->tile_desc));
    h->tile_desc = nullptr;
    h->tile_desc_cap = 0;
    CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->tile_desc), cap * sizeof(unsigned long long)));
    CX_HIP(hipMemsetAsync(h->tile_desc, 0, cap * sizeof(unsigned long long), h->stream));
    h->tile_desc_cap = cap;
    return CX_OK;
}

}  // namespace

template <typename T>
int launch_compact(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                   const T* thr_host, const T* d_thr, int* d_size_prefix) {
    constexpr int kPairBytes = 4 * Elem<T>::pair_words;
    if (!out_msg || n < 0) return fail(CX_ERR_INVALID, "compress: null message buffer or negative size");
    if ((reinterpret_cast<uintptr_t>(out_msg) & 3u) != 0)
        return fail(CX_ERR_INVALID, "compress: message buffer must be 4-byte aligned");
    if (out_capacity < 8) return fail(CX_ERR_CAPACITY, "compress: message buffer smaller than its 8-byte header");
    unsigned* msg_words = static_cast<unsigned*>(out_msg);
    if (!data && !update) {
        // the reference falls through all three branches and emits an empty message
        hipLaunchKernelGGL(empty_message_kernel, dim3(1), dim3(1), 0, h->stream, msg_words, n, d_size_prefix);
        CX_HIP(hipGetLastError());
        return CX_OK;
    }
    const int mode = (data && update) ? 0 : (update ? 1 : 2);
    const long long cap_pairs = (out_capacity - 8) / kPairBytes;
    const int aligned8 = ((reinterpret_cast<uintptr_t>(out_msg) & 7u) == 0) ? 1 : 0;
    const T thr_val = thr_host ? *thr_host : (T)0;
    const T* thr_ptr = thr_host ? nullptr : (d_thr ? d_thr : static_cast<const T*>(h->d_thr));

    constexpr int kVec = 16 / (int)sizeof(T);
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(update)) & 15u) == 0;
    const int items = vec_ok ? h->compact_items : 16;
    const int vec = vec_ok ? kVec : 1;
    const long long tile = (long long)kBlock * vec * items;
    const long long nt = n == 0 ? 1 : ((long long)n + tile - 1) / tile;
    const unsigned ntiles = (unsigned)nt;

    int rc = ensure_descriptors(h, ntiles);
    if (rc != CX_OK) return rc;
    h->epoch = (h->epoch + 1u) & 0x3fffffffu;
    if (h->epoch == 0u) {  // 30-bit launch counter wrapped: forget every old descriptor
        CX_HIP(hipMemsetAsync(h->tile_desc, 0, h->tile_desc_cap * sizeof(unsigned long long), h->stream));
        h->epoch = 1u;
    }

    if (!vec_ok) {
        launch_mode<T, 1, 16>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                              d_size_prefix, ntiles);
    } else if (items == 4) {
        launch_mode<T, kVec, 4>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                                d_size_prefix, ntiles);
    } else if (items == 8) {
        launch_mode<T, kVec, 8>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                                d_size_prefix, ntiles);
    } else if (items == 2) {
        launch_mode<T, kVec, 2>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, aligned8,
                                d_size_prefix, ntiles);
    } else {
        return fail(CX_ERR_INVALID, "compress: unsupported compact_items %d", items);
    }
    CX_HIP(hipGetLastError());
    if (!h->compact_tile_ids) h->counter_base += ntiles;
    return CX_OK;
}

template int launch_compact<float>(cx_handle, void*, long long, const float*, float*, int, const float*, const float*, int*);
template int launch_compact<double>(cx_handle, void*, long long, const double*, double*, int, const double*, const double*, int*);
template int launch_compact<int>(cx_handle, void*, long long, const int*, int*, int, const int*, const int*, int*);

}  // namespace cx
