// Fused error-feedback accumulate + magnitude select + ordered compaction + residual zeroing.
//
// Replaces the sequential loop of CompressorIndexPairs<T>::compression_strategy
// (reference src/compressor.hxx:556-611).  Two launches on one stream (three for dense flushes), none of which
// ever waits on another workgroup (no spin loops, no global atomics on the data path):
//
//  1. stage_kernel   the HBM-bound pass.  Each wavefront owns one tile of 64*VEC*ITEMS
//                    consecutive elements, read with 16-byte lane-contiguous loads.
//                    s = update + data (one IEEE add, as the reference's
//                    `update[i] += data[i]`), survivors are |s| > threshold (strict, NaN
//                    never survives).  Ranks inside the tile come from wavefront ballots
//                    and popcounts, in ascending index order.  Survivors go to the tile's
//                    private slot of a staging buffer (capacity: 1/8 of the tile), the
//                    tile's count to counts[tile], and the residual is written back once
//                    with survivors replaced by +0.  A tile with more survivors than its
//                    slot holds does nothing but record its count with the "deferred" bit.
//  2. gather_kernel  each 256-thread block owns 64 tiles: it adds up the per-block survivor sums
//                    the streaming pass left for the tiles before them, scans the 64 counts,
//                    copies the staged slots to their final position in the message with
//                    lane-contiguous stores (all its wavefronts together) and processes the few
//                    deferred tiles it owns straight into their final position, which is known
//                    by now; the last block writes the header.
//  3. redo_kernel    launched only when the threshold is known to select (nearly) everything
//                    (flushRests passes 0): then every tile is deferred, pass 1 was a pure count
//                    pass, and this kernel does the write pass on the whole GPU.
//
// HBM traffic per element at low density (fp32): 4 B data + 4 B residual in, 4 B residual
// out, plus per survivor 8 B staged + 8 B re-read + 8 B final.
#include "cx_common.hpp"
#include "cx_select_dev.hpp"

#include <mutex>

namespace cx {

namespace {

// threads of a streaming block, one tile per wavefront.  Measured on 100 M fp32 elements at 1 %, whole
// step: 128 / 256 / 512 threads 0.210 / 0.208 / 0.209 ms back to back and 0.223 / 0.222 / 0.221 ms after
// the gradient was rewritten, i.e. alike within the spread between two runs (0.001 ms).
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / 64;
constexpr unsigned kDeferred = 0x80000000u;
// threads of a gather block and pairs a lane moves per round.  Measured, whole step on 100 M fp32
// elements at 1 % / threshold + compress on 61 706 elements at 10 % (one gather block moves all 6 170
// pairs there): 256 threads x 4 pairs 0.208 ms / 40.5 us, 256 x 8 0.209 / 40.2, 512 x 4 0.208 / 38.7,
// 512 x 8 0.212 / 37.9, 128 x 4 0.208 / 50 (measured with deferred tiles in the short vector).
constexpr int kGatherBlock = 512;
constexpr int kGatherUnroll = 4;
constexpr int kGatherTiles = 64;                // tiles a gather block owns: one lane per tile in its scan
static_assert(kGatherTiles % (kWavesPerBlock * 8) == 0, "a gather block's streaming blocks fill whole 16-byte loads of 16-bit sums");
static_assert(kWavesPerBlock * 64 * 4 * 16 <= 65535, "a streaming block's survivors fit 16 bits (largest tile: 64 lanes x 16 loads x 4 elements)");

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T x[V]; };

// Cache policy of the streaming pass.  The gradient is read once per step and the residual
// is rewritten once per step, so both bypass the caches (nontemporal).  The residual's READS
// stay cacheable over the last stage_cached_tail_mb (192) MB of the walk only: that tail is what the
// 256 MB memory-side cache still holds when the next launch walks the tiles in the opposite
// direction (stage_alternate) and starts there; earlier reads would be pushed out before anybody
// could use them, and by allocating they push out other lines first.  Measured on 100 M fp32
// elements (step, everything cacheable -> 192 MB tail): consecutive steps 0.214 -> 0.206 ms; after
// another kernel read 1 GiB 0.218 -> 0.214 ms, rewrote 1 GiB 0.265 -> 0.248 ms, rewrote the
// gradient itself 0.250 -> 0.221 ms.  (No cacheable reads at all: 0.221 / 0.223 / 0.232 / 0.224 ms.)
// (the same step with cacheable gradient loads: 0.208 -> 0.226 ms, after the gradient was rewritten
// 0.222 -> 0.267 ms; with cacheable residual stores: 0.229 and 0.253 ms)
constexpr bool kNontemporalData = true;         // gradient loads
constexpr bool kNontemporalUpdateStore = true;  // residual stores

template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack(const T* p, bool nt) {
    typedef T vec_t __attribute__((ext_vector_type(V)));
    Pack<T, V> r;
    if (nt) {
        vec_t v = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(p));
#pragma unroll
        for (int c = 0; c < V; ++c) r.x[c] = v[c];
    } else {
        r = *reinterpret_cast<const Pack<T, V>*>(p);
    }
    return r;
}
template <typename T, int V>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, V>& w, bool nt) {
    typedef T vec_t __attribute__((ext_vector_type(V)));
    if (nt) {
        vec_t v;
#pragma unroll
        for (int c = 0; c < V; ++c) v[c] = w.x[c];
        __builtin_nontemporal_store(v, reinterpret_cast<vec_t*>(p));
    } else {
        *reinterpret_cast<Pack<T, V>*>(p) = w;
    }
}

__device__ __forceinline__ float mag(float v) { return fabsf(v); }
__device__ __forceinline__ double mag(double v) { return fabs(v); }
__device__ __forceinline__ int mag(int v) { return v < 0 ? -v : v; }

__device__ __forceinline__ void put_pair(unsigned* w, unsigned index, float v) {
    w[0] = index;
    w[1] = __float_as_uint(v);
}
__device__ __forceinline__ void put_pair(unsigned* w, unsigned index, int v) {
    w[0] = index;
    w[1] = (unsigned)v;
}
__device__ __forceinline__ void put_pair(unsigned* w, unsigned index, double v) {
    const unsigned long long bits = (unsigned long long)__double_as_longlong(v);
    w[0] = index;
    w[1] = (unsigned)bits;
    w[2] = (unsigned)(bits >> 32);
}

template <typename T> __device__ __forceinline__ T pair_value(const unsigned* w);
template <> __device__ __forceinline__ float pair_value<float>(const unsigned* w) { return __uint_as_float(w[1]); }
template <> __device__ __forceinline__ int pair_value<int>(const unsigned* w) { return (int)w[1]; }
template <> __device__ __forceinline__ double pair_value<double>(const unsigned* w) {
    return __longlong_as_double((long long)((unsigned long long)w[1] | ((unsigned long long)w[2] << 32)));
}

// One wavefront, one tile.  MODE 0: update += data, select on update, zero selected
// (compress_add_update); MODE 1: select on update, zero selected (compress_update);
// MODE 2: select on data, nothing written back (compress); MODE 3: as MODE 0 for a list of
// CANDIDATES (fused exact top-k: the selected set is a superset of what is finally sent): a
// selected element that finds no room in the list is not an error, it keeps its value in update.
// DIRECT false: stage the pairs (or defer the tile); true: write them at `direct_pos`.
template <typename T, int MODE, int VEC, int ITEMS, bool DIRECT>
__device__ __forceinline__ unsigned process_tile(const T* __restrict__ data, T* __restrict__ update, long long n,
                                             T thr, unsigned tile, int lane, unsigned* __restrict__ staging,
                                             unsigned* __restrict__ counts,
                                             unsigned* __restrict__ redo_flag, unsigned epoch,
                                             unsigned* __restrict__ out_pairs, long long direct_pos,
                                             long long cap_pairs, DeviceStatus* status, bool nt_update = false,
                                             unsigned slot_pairs = 0u) {
    constexpr int kTile = 64 * VEC * ITEMS;
    constexpr int PW = Elem<T>::pair_words;
    const long long base = (long long)tile * kTile;
    const bool full = base + kTile <= n;
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

    T s[ITEMS][VEC];
    unsigned sel[ITEMS], rank[ITEMS];
    unsigned total = 0;
    unsigned valid_mask[ITEMS];

    // every load of the tile is issued before the first value is used: the cross-lane steps below
    // would otherwise fence each pair of loads off from the next
    Pack<T, VEC> uu[ITEMS], dd[ITEMS];
    if (full) {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const long long e0 = base + (long long)j * (64 * VEC) + (long long)lane * VEC;
            if (MODE != 2) uu[j] = load_pack<T, VEC>(update + e0, nt_update);
            if (MODE != 1) dd[j] = load_pack<T, VEC>(data + e0, kNontemporalData);
            valid_mask[j] = (1u << VEC) - 1u;
        }
    } else {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const long long e0 = base + (long long)j * (64 * VEC) + (long long)lane * VEC;
            unsigned valid = 0;
#pragma unroll
            for (int c = 0; c < VEC; ++c) {
                const bool in = e0 + c < n;
                uu[j].x[c] = (MODE != 2 && in) ? update[e0 + c] : (T)0;
                dd[j].x[c] = (MODE != 1 && in) ? data[e0 + c] : (T)0;
                valid |= (in ? 1u : 0u) << c;
            }
            valid_mask[j] = valid;
        }
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const Pack<T, VEC>& u = uu[j];
        const Pack<T, VEC>& d = dd[j];
        const unsigned valid = valid_mask[j];
        unsigned m = 0;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            T v;
            if (MODE == 0 || MODE == 3) v = (T)(u.x[c] + d.x[c]);
            else if (MODE == 1) v = u.x[c];
            else v = d.x[c];
            s[j][c] = v;
            m |= ((mag(v) > thr) ? 1u : 0u) << c;
        }
        m &= valid;
        sel[j] = m;
        unsigned before = total;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            const unsigned long long b = __ballot((m >> c) & 1u);
            before += __popcll(b & below);
            total += __popcll(b);
        }
        rank[j] = before;  // survivors of this tile that precede this lane's first element of load j
    }

    unsigned* dst;
    long long dst_limit;  // pairs that may be written through dst
    if (DIRECT) {
        dst = out_pairs + direct_pos * PW;
        dst_limit = cap_pairs - direct_pos;
    } else {
        if (total > slot_pairs) {
            if (lane == 0) {
                counts[tile] = total | kDeferred;
                *redo_flag = epoch;
            }
            return total;  // no side effects: the redo pass starts from untouched inputs
        }
        if (lane == 0) counts[tile] = total;
        dst = staging + (long long)tile * (long long)(slot_pairs * (unsigned)PW);
        dst_limit = slot_pairs;
    }

    bool overflow = false;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const long long e0 = base + (long long)j * (64 * VEC) + (long long)lane * VEC;
        const unsigned m = sel[j];
        long long pos = rank[j];
        Pack<T, VEC> w;
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            bool keep = (m >> c) & 1u;
            if (keep) {
                if (pos < dst_limit) {
                    put_pair(dst + pos * PW, (unsigned)(e0 + c), s[j][c]);
                } else {
                    keep = false;  // no room in the message: stays in the residual (the header counts what was written)
                    if (MODE != 3) overflow = true;
                }
                ++pos;
            }
            w.x[c] = keep ? (T)0 : s[j][c];
        }
        if (MODE != 2) {
            if (full) {
                if (MODE == 0 || MODE == 3 || m != 0u) store_pack<T, VEC>(update + e0, w, kNontemporalUpdateStore);
            } else {
#pragma unroll
                for (int c = 0; c < VEC; ++c)
                    if (((valid_mask[j] >> c) & 1u) && (MODE == 0 || MODE == 3 || ((m >> c) & 1u)))
                        update[e0 + c] = w.x[c];
            }
        }
    }
    if (DIRECT && overflow) atomicOr(&status->detail, 1);
    return total;
}

template <typename T, int MODE, int VEC, int ITEMS>
__device__ __forceinline__ void stage_block(const T* __restrict__ data, T* __restrict__ update, long long n, const T thr,
                                            unsigned* __restrict__ staging, unsigned* __restrict__ counts,
                                            unsigned* __restrict__ block_sums, unsigned* __restrict__ redo_flag,
                                            unsigned epoch, unsigned ntiles, int reverse, unsigned cached_from,
                                            unsigned slot_pairs, unsigned& s_sum, unsigned& s_done) {
    // reversed launches walk the blocks from the end: they start on what the previous pass left cached
    const unsigned block = reverse ? gridDim.x - 1u - blockIdx.x : blockIdx.x;
    const unsigned tile = block * kWavesPerBlock + (threadIdx.x >> 6);
    if (tile >= ntiles) return;
    // Only the last part of the walk can still be in the memory-side cache when the next launch
    // starts there: that part of the residual is read cacheably, everything before it bypasses the
    // caches like the gradient (a read that allocates pushes out lines that then have to be written
    // back, which costs most when the cache is full of another kernel's dirty lines).
    const unsigned walk_rank = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const bool nt_update = __builtin_amdgcn_readfirstlane((int)(walk_rank < cached_from)) != 0;
    const unsigned total = process_tile<T, MODE, VEC, ITEMS, false>(data, update, n, thr, tile, threadIdx.x & 63,
                                                                    staging, counts, redo_flag, epoch, nullptr, 0, 0,
                                                                    nullptr, nt_update, slot_pairs);
    if ((threadIdx.x & 63) == 0) {
        const unsigned tiles_here = ntiles - block * kWavesPerBlock < (unsigned)kWavesPerBlock
                                        ? ntiles - block * kWavesPerBlock
                                        : (unsigned)kWavesPerBlock;
        atomicAdd(&s_sum, total);  // LDS
        __threadfence_block();
        // 16 bits per sum (a block has at most a few thousand elements): every gather block reads
        // all the sums before its own, and halving them shortens that read
        if (atomicAdd(&s_done, 1u) == tiles_here - 1u)
            reinterpret_cast<unsigned short*>(block_sums)[block] = (unsigned short)atomicAdd(&s_sum, 0u);
    }
}

template <typename T, int MODE, int VEC, int ITEMS>
__global__ __launch_bounds__(kBlock) void stage_kernel(const T* __restrict__ data, T* __restrict__ update, long long n,
                                                       const T* __restrict__ thr_ptr, T thr_val,
                                                       unsigned* __restrict__ staging, unsigned* __restrict__ counts,
                                                       unsigned* __restrict__ block_sums,
                                                       unsigned* __restrict__ redo_flag, unsigned epoch,
                                                       unsigned ntiles, int reverse, unsigned cached_from,
                                                       unsigned slot_pairs) {
    // survivors of this block's tiles, summed in LDS; the wavefront that finishes last stores
    // the sum, which spares the gather kernel a scan over every tile count
    __shared__ unsigned s_sum, s_done;
    if (threadIdx.x == 0) {
        s_sum = 0u;
        s_done = 0u;
    }
    __syncthreads();
    const T thr = thr_ptr ? *thr_ptr : thr_val;
    stage_block<T, MODE, VEC, ITEMS>(data, update, n, thr, staging, counts, block_sums, redo_flag, epoch, ntiles, reverse,
                                     cached_from, slot_pairs, s_sum, s_done);
}

// The same pass behind a chained radix selection (k_select.hip) whose last pick has not been made: every
// block makes it for itself from the last pass's complete histogram, as the blocks of a chained pass do,
// so the one-block kernel that would only pick and store the threshold is not launched.  Block 0 stores
// the threshold for the kernels that follow (gather_kernel reads it, and clears the histograms).
template <typename T, int MODE, int VEC, int ITEMS>
__global__ __launch_bounds__(kBlock) void stage_pick_kernel(const T* __restrict__ data, T* __restrict__ update, long long n,
                                                            const SelectState* __restrict__ sel, unsigned long long rank0,
                                                            int plus_one, T* __restrict__ thr_out,
                                                            unsigned* __restrict__ staging, unsigned* __restrict__ counts,
                                                            unsigned* __restrict__ block_sums,
                                                            unsigned* __restrict__ redo_flag, unsigned epoch,
                                                            unsigned ntiles, int reverse, unsigned cached_from,
                                                            unsigned slot_pairs) {
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    using key_t = typename Elem<T>::key_t;
    __shared__ unsigned s_sum, s_done;
    __shared__ unsigned s_digit;
    __shared__ unsigned long long s_above, s_part[kBlock / 64];
    if (threadIdx.x == 0) {
        s_sum = 0u;
        s_done = 0u;
    }
    const PickState picked = state_entering_pass<T, kBlock>(sel, kPasses, rank0, s_part, &s_digit, &s_above);
    T thr = value_of((key_t)picked.prefix, T());
    if (plus_one) thr = (T)(thr + 1);
    if (blockIdx.x == 0 && threadIdx.x == 0) *thr_out = thr;
    stage_block<T, MODE, VEC, ITEMS>(data, update, n, thr, staging, counts, block_sums, redo_flag, epoch, ntiles, reverse,
                                     cached_from, slot_pairs, s_sum, s_done);
}

template <typename T, int MODE, int VEC, int ITEMS>
__global__ __launch_bounds__(kBlock) void redo_kernel(const T* __restrict__ data, T* __restrict__ update, long long n,
                                                      const T* __restrict__ thr_ptr, T thr_val,
                                                      const unsigned* __restrict__ counts,
                                                      const unsigned* __restrict__ offsets,
                                                      const unsigned* __restrict__ redo_flag, unsigned epoch,
                                                      unsigned ntiles, unsigned* __restrict__ out_pairs,
                                                      long long cap_pairs, DeviceStatus* status) {
    if (*redo_flag != epoch) return;  // nothing was deferred in this launch
    const T thr = thr_ptr ? *thr_ptr : thr_val;
    const unsigned nwaves = gridDim.x * kWavesPerBlock;
    for (unsigned tile = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); tile < ntiles; tile += nwaves) {
        if (!(counts[tile] & kDeferred)) continue;
        process_tile<T, MODE, VEC, ITEMS, true>(data, update, n, thr, tile, threadIdx.x & 63, nullptr, nullptr, nullptr,
                                                epoch, out_pairs, (long long)offsets[tile], cap_pairs, status);
    }
}

// Final offsets of the tiles and copy of the staged slots to their final place.  A block owns
// kGatherTiles (64) consecutive tiles: it adds up the per-block sums the streaming pass left for the
// tiles before its own (16-byte loads), every wavefront scans the 64 counts (one lane per tile),
// and all wavefronts together move the block's pairs with lane-contiguous stores, so that the
// whole GPU takes part in what is a latency-bound copy.  Deferred tiles are either processed
// here, shared out among the block's wavefronts (inline_redo), or left to redo_kernel, which then
// needs offsets[].  The block that owns the last tile writes the message header.
template <typename T, int MODE, int VEC, int ITEMS>
__global__ __launch_bounds__(kGatherBlock) void gather_kernel(
    const T* __restrict__ data, T* __restrict__ update, long long n, const T* __restrict__ thr_ptr, T thr_val,
    const unsigned* __restrict__ counts, const unsigned* __restrict__ block_sums, unsigned* __restrict__ offsets,
    const unsigned* __restrict__ staging, unsigned ntiles, unsigned* __restrict__ msg_words, long long cap_pairs,
    int* __restrict__ size_prefix, int inline_redo, DeviceStatus* status, unsigned slot_pairs,
    unsigned* __restrict__ zero_words, unsigned zero_count) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int kWaves = kGatherBlock / 64;
    // pairs a lane moves per round: searches and loads of one round are independent
    constexpr int kCopyUnroll = kGatherUnroll;
    __shared__ unsigned s_before[kWaves];
    __shared__ unsigned s_off[65];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // words a kernel before this one has finished with (a selection's histograms), cleared for their next
    // use by one block more than the tiles need
    if (zero_words && blockIdx.x * kGatherTiles >= ntiles) {
        for (unsigned b = tid; b < zero_count; b += kGatherBlock) zero_words[b] = 0u;
        return;
    }

    // Order of the loads: the tiles' counts first, then (their scan known) the staged pairs of the first
    // round, and only then the sums of the streaming blocks before this block's tiles, which give the
    // pairs' destination: the long read of the sums runs while the staged pairs are on their way,
    // instead of in front of everything (a memory round trip or two less on a kernel that is all latency).
    // every wavefront scans the same 64 counts
    const unsigned first = blockIdx.x * kGatherTiles;
    const unsigned tile = first + lane;  // tiles past the end count as empty
    const unsigned raw = tile < ntiles ? counts[tile] : 0u;
    const unsigned cnt = raw & ~kDeferred;
    unsigned incl = cnt;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    const unsigned block_pairs = __shfl(incl, 63, 64);
    if (wave == 0) {
        s_off[lane] = incl - cnt;
        if (lane == 63) s_off[64] = block_pairs;
    }
    const unsigned long long deferred = __ballot((raw & kDeferred) != 0u);
    __syncthreads();

    // one round of the copy: where a pair of this block comes from (its tile's slot) and its words
    unsigned src_idx[kCopyUnroll];
    bool live[kCopyUnroll];
    unsigned v[kCopyUnroll][PW];
    auto load_round = [&](unsigned p0) {
#pragma unroll
        for (int q = 0; q < kCopyUnroll; ++q) {
            const unsigned p = p0 + q * kGatherBlock + tid;
            live[q] = p < block_pairs;
            // owner: last tile of this block whose exclusive offset is <= p.  Six fixed steps
            // without branches, so that the searches of one round overlap their LDS reads.
            int lo = 0;
#pragma unroll
            for (int step = 32; step > 0; step >>= 1)
                lo += (s_off[lo + step > 63 ? 63 : lo + step] <= p && lo + step <= 63) ? step : 0;
            if ((deferred >> lo) & 1ull) live[q] = false;  // not staged
            src_idx[q] = (first + lo) * slot_pairs + (p - s_off[lo]);
        }
#pragma unroll
        for (int q = 0; q < kCopyUnroll; ++q)
            if (live[q]) {
#pragma unroll
                for (int w = 0; w < PW; ++w) v[q][w] = staging[(long long)src_idx[q] * PW + w];
            }
    };
    load_round(0u);

    unsigned before = 0;
    {
        // stage blocks before this block's first tile: kGatherTiles / kWavesPerBlock per gather block
        // (eight 16-bit sums per 16-byte load)
        const uint4* b4 = reinterpret_cast<const uint4*>(block_sums);
        const unsigned nvec = blockIdx.x * (kGatherTiles / kWavesPerBlock / 8);
#pragma unroll 8
        for (unsigned i = tid; i < nvec; i += kGatherBlock) {
            const uint4 c = b4[i];
            before += (c.x & 0xffffu) + (c.x >> 16) + (c.y & 0xffffu) + (c.y >> 16) + (c.z & 0xffffu) + (c.z >> 16) +
                      (c.w & 0xffffu) + (c.w >> 16);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off, 64);
    if (lane == 0) s_before[wave] = before;
    __syncthreads();
    unsigned block_base = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) block_base += s_before[w];
    const unsigned tile_off = block_base + (incl - cnt);
    if (wave == 0) {
        if (!inline_redo && tile < ntiles) offsets[tile] = tile_off;
        if (tile == ntiles - 1) {
            unsigned k = tile_off + cnt;
            // never announce more pairs than the buffer holds (candidate lists keep the full count:
            // their reader checks it against the capacity)
            if (MODE != 3 && (long long)k > cap_pairs) k = (unsigned)cap_pairs;
            msg_words[0] = (unsigned)n;
            msg_words[1] = k;
            if (size_prefix) *size_prefix = (int)(8u + k * (unsigned)(4 * PW));
        }
    }

    unsigned* const pairs = msg_words + 2;
    bool overflow = false;
    for (unsigned p0 = 0; p0 < block_pairs; p0 += kGatherBlock * kCopyUnroll) {
        if (p0 > 0u) load_round(p0);
#pragma unroll
        for (int q = 0; q < kCopyUnroll; ++q)
            if (live[q]) {
                const long long dst_pos = (long long)block_base + p0 + q * kGatherBlock + tid;
                if (dst_pos < cap_pairs) {
#pragma unroll
                    for (int w = 0; w < PW; ++w) pairs[dst_pos * PW + w] = v[q][w];
                } else {
                    // no room in the message (or candidate list): the value goes back into the residual
                    if (MODE != 2) update[v[q][0]] = pair_value<T>(v[q]);
                    if (MODE != 3) overflow = true;
                }
            }
    }
    if (overflow) atomicOr(&status->detail, 1);

    if (inline_redo && deferred != 0ull) {
        const T thr = thr_ptr ? *thr_ptr : thr_val;
        unsigned long long todo = deferred;
        int turn = 0;
        while (todo) {
            const int l = __ffsll((long long)todo) - 1;
            todo &= todo - 1;
            const unsigned pos = __shfl(tile_off, l, 64);
            if ((turn++ % kWaves) == wave)  // the block's wavefronts take the deferred tiles in turn
                process_tile<T, MODE, VEC, ITEMS, true>(data, update, n, thr, first + l, lane, nullptr, nullptr,
                                                        nullptr, 0u, pairs, (long long)pos, cap_pairs, status);
        }
    }
}

__global__ void empty_message_kernel(unsigned* msg_words, int n, int* size_prefix) {
    msg_words[0] = (unsigned)n;
    msg_words[1] = 0u;
    if (size_prefix) *size_prefix = 8;
}

// The compaction's scratch arrays: per-tile staging slots, counts, final offsets, per-block sums.
struct Scratch {
    unsigned* staging;
    unsigned* counts;
    unsigned* offsets;
    unsigned* block_sums;
};

// ---- scratch of the allocation-free entry point (cx_ip_compress_noalloc) -------------------
// One array per GPU, part of the code object, alive until the process ends.  Sized for vectors of
// up to kNoAllocMaxN elements of any supported type and tile shape: staging needs at most 3/8 of a
// 32-bit word per element (8-byte elements: 64 slots of 3 words per 512 elements), the smallest
// tile has 256 elements.  Every launch writes what it later reads (counts, sums, slots), so stale
// contents of an earlier call are harmless; two calls that overlap in time on one GPU would race.
constexpr long long kNoAllocMaxN = 1ll << 24;
constexpr size_t kStaticStagingWords = (size_t)kNoAllocMaxN * 3 / 8 + 1024;
// vectors up to this length get staging slots that hold a whole tile (32 to 48 MB of staging at most)
constexpr long long kWholeSlotMaxN = 1ll << 22;
constexpr size_t kStaticTiles = (size_t)kNoAllocMaxN / 256 + 64;
constexpr size_t kStaticSumsWords = kStaticTiles / 4 + 64;
constexpr size_t kStaticWords = kStaticStagingWords + 2 * kStaticTiles + kStaticSumsWords;
static __device__ __align__(256) unsigned scratch[kStaticWords];

int ensure_scratch(cx_handle h, size_t ntiles, size_t staging_words) {
    if (ntiles > h->tiles_cap) {
        size_t cap = h->tiles_cap ? h->tiles_cap : 4096;
        while (cap < ntiles) cap *= 2;
        CX_HIP(hipStreamSynchronize(h->stream));  // the old arrays may still be in use
        if (h->tile_counts) CX_HIP(hipFree(h->tile_counts));
        if (h->tile_offsets) CX_HIP(hipFree(h->tile_offsets));
        h->tile_counts = h->tile_offsets = nullptr;
        h->tiles_cap = 0;
        CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->tile_counts), cap * sizeof(unsigned)));
        CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->tile_offsets), cap * sizeof(unsigned)));
        if (h->block_sums) CX_HIP(hipFree(h->block_sums));
        h->block_sums = nullptr;
        CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->block_sums), (cap / kWavesPerBlock + 4) * sizeof(unsigned)));
        h->tiles_cap = cap;
    }
    if (staging_words > h->staging_cap) {
        size_t cap = staging_words + staging_words / 8;
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->staging) CX_HIP(hipFree(h->staging));
        h->staging = nullptr;
        h->staging_cap = 0;
        CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->staging), cap * sizeof(unsigned)));
        h->staging_cap = cap;
    }
    return CX_OK;
}

// Largest scratch any tile shape needs for n elements of T: the smallest tile (2 vectors per lane)
// has the most tiles; the slots hold an eighth of the elements whatever the shape.
template <typename T> void scratch_need(long long n, size_t* ntiles, size_t* staging_words) {
    constexpr int kVec = 16 / (int)sizeof(T);
    constexpr int PW = Elem<T>::pair_words;
    constexpr long long kSmallestTile = 64ll * kVec * 2, kLargestTile = 64ll * kVec * 8;
    *ntiles = (size_t)((n + kSmallestTile - 1) / kSmallestTile);
    const size_t slot = n <= kWholeSlotMaxN ? (size_t)kLargestTile : (size_t)(kLargestTile / 8);  // as launch_all chooses
    *staging_words = (size_t)((n + kLargestTile - 1) / kLargestTile) * slot * PW;
}

template <typename T, int MODE, int VEC, int ITEMS>
int launch_all(cx_handle h, const T* data, T* update, int n, const T* thr_ptr, T thr_val, unsigned* msg_words,
               long long cap_pairs, int* size_prefix, DeviceStatus* status, bool no_alloc) {
    constexpr int kTile = 64 * VEC * ITEMS;
    constexpr int PW = Elem<T>::pair_words;
    const unsigned ntiles = (unsigned)(((long long)n + kTile - 1) / kTile);
    // a threshold known to select (nearly) everything, as flushRests passes, defers every tile:
    // the second pass then gets the whole GPU instead of the gather kernel's few blocks
    const int dense_hint = (thr_ptr == nullptr && !(thr_val > (T)0)) ? 1 : 0;
    // Pairs a tile's staging slot holds.  An eighth of the tile keeps the staging area small on long
    // vectors (a tile with more survivors is deferred and processed again in the gather kernel, one
    // wavefront per tile).  Short vectors get whole-tile slots: nothing is ever deferred there, and
    // their gather kernel has too few blocks to hide such repeats (61 706 elements at 10 %: 3 to 5
    // deferred tiles made the gather kernel 11 us long instead of 5).
    const bool whole_slots = !no_alloc && MODE != 3 && !dense_hint && (long long)n <= kWholeSlotMaxN;
    const unsigned slot_pairs = whole_slots ? (unsigned)kTile : (unsigned)kTile / 8u;
    Scratch sc;
    if (no_alloc) {
        // the per-GPU static array, cut into the four arrays; never grows
        unsigned* base = h->static_scratch;
        if (!base) return fail(CX_ERR_INTERNAL, "compress: the static scratch array was not located on this device");
        if ((size_t)ntiles * slot_pairs * PW > kStaticStagingWords || (size_t)ntiles > kStaticTiles ||
            (size_t)(ntiles + kWavesPerBlock - 1) / kWavesPerBlock > kStaticSumsWords)
            return fail(CX_ERR_INVALID, "compress: %d elements exceed the static scratch array", n);
        sc.staging = base;
        sc.counts = base + kStaticStagingWords;
        sc.offsets = sc.counts + kStaticTiles;
        sc.block_sums = sc.offsets + kStaticTiles;
    } else {
        int rc = ensure_scratch(h, ntiles, (size_t)ntiles * slot_pairs * PW);
        if (rc != CX_OK) return rc;
        sc.staging = h->staging;
        sc.counts = h->tile_counts;
        sc.offsets = h->tile_offsets;
        sc.block_sums = h->block_sums;
    }
    h->epoch += 1u;
    if (h->epoch == 0u) h->epoch = 1u;  // 0 is what a fresh flag holds
    unsigned* redo_flag = h->redo_flag;
    const int reverse = h->stage_alternate ? (int)h->parity : 0;  // start where the previous full pass ended
    h->parity ^= 1u;

    const unsigned stage_blocks = (ntiles + kWavesPerBlock - 1) / kWavesPerBlock;
    // tiles at the end of the walk whose residual reads may stay in the caches
    const unsigned long long tail_tiles =
        h->stage_cached_tail_mb < 0 ? (unsigned long long)ntiles
                                    : ((unsigned long long)h->stage_cached_tail_mb << 20) / ((unsigned long long)kTile * sizeof(T));
    const unsigned cached_from = tail_tiles >= ntiles ? 0u : ntiles - (unsigned)tail_tiles;
    hipEvent_t* ev = nullptr;
    if (h->profile && h->profile_events && h->profile_count < cx_handle_s::kProfileRing &&
        (h->profile_tick++ % (unsigned)h->profile) == 0u) {  // every profile-th launch
        ev = h->profile_events + 2 * h->profile_count;
        h->profile_count += 1;
        CX_HIP(hipEventRecord(ev[0], h->stream));
    }
    unsigned* zero_words = nullptr;
    unsigned zero_count = 0u;
    bool picked_here = false;
    if constexpr (MODE == 0) {
        if (h->pending_pick.active) {
            // the selection before this call left its last pick to this pass (see stage_pick_kernel)
            constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
            h->pending_pick.active = false;
            picked_here = true;
            zero_words = &h->sel->pass_hist[0][0];
            zero_count = (unsigned)((kPasses + 1) * kRadixBins);
            hipLaunchKernelGGL((stage_pick_kernel<T, MODE, VEC, ITEMS>), dim3(stage_blocks), dim3(kBlock), 0, h->stream, data,
                               update, (long long)n, h->sel, h->pending_pick.rank, h->pending_pick.plus_one,
                               static_cast<T*>(h->pending_pick.thr_out), sc.staging, sc.counts, sc.block_sums, redo_flag,
                               h->epoch, ntiles, reverse, cached_from, slot_pairs);
        }
    }
    if (!picked_here)
        hipLaunchKernelGGL((stage_kernel<T, MODE, VEC, ITEMS>), dim3(stage_blocks), dim3(kBlock), 0, h->stream, data, update,
                           (long long)n, thr_ptr, thr_val, sc.staging, sc.counts, sc.block_sums, redo_flag, h->epoch, ntiles,
                           reverse, cached_from, slot_pairs);
    if (ev) CX_HIP(hipEventRecord(ev[1], h->stream));
    const unsigned gather_blocks = (ntiles + kGatherTiles - 1) / kGatherTiles;
    hipLaunchKernelGGL((gather_kernel<T, MODE, VEC, ITEMS>), dim3(gather_blocks + (zero_words ? 1u : 0u)),
                       dim3(kGatherBlock), 0, h->stream, data,
                       update, (long long)n, thr_ptr, thr_val, sc.counts, sc.block_sums,
                       sc.offsets, sc.staging, ntiles, msg_words, cap_pairs, size_prefix, dense_hint ? 0 : 1,
                       status, slot_pairs, zero_words, zero_count);
    if (dense_hint) {
        const unsigned redo_blocks = stage_blocks < 2048u ? stage_blocks : 2048u;
        hipLaunchKernelGGL((redo_kernel<T, MODE, VEC, ITEMS>), dim3(redo_blocks), dim3(kBlock), 0, h->stream, data,
                           update, (long long)n, thr_ptr, thr_val, sc.counts, sc.offsets, redo_flag, h->epoch,
                           ntiles, msg_words + 2, cap_pairs, status);
    }
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T, int VEC, int ITEMS>
int launch_mode(cx_handle h, int mode, const T* data, T* update, int n, const T* thr_ptr, T thr_val,
                unsigned* msg_words, long long cap_pairs, int* size_prefix, bool no_alloc = false) {
    DeviceStatus* st = h->d_status;
    if (mode == 0) return launch_all<T, 0, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, size_prefix, st, no_alloc);
    if (mode == 1) return launch_all<T, 1, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, size_prefix, st, no_alloc);
    if (mode == 2) return launch_all<T, 2, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, size_prefix, st, no_alloc);
    return launch_all<T, 3, VEC, ITEMS>(h, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, size_prefix, st, no_alloc);
}

}  // namespace

// Address of this device's copy of the static scratch array.  The array's name is only a
// host-side stand-in for the symbol; the address a kernel can use comes from the runtime, per
// device, with that device current.
int locate_static_scratch(unsigned** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static unsigned* per_device[kMaxDevices];  // each GPU holds its own copy at its own address
    *out = nullptr;
    int device = 0;
    CX_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(CX_ERR_INVALID, "device ordinal %d not supported", device);
    std::lock_guard<std::mutex> guard(lock);
    if (!per_device[device]) {
        void* p = nullptr;
        CX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(CX_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
        per_device[device] = static_cast<unsigned*>(p);
    }
    *out = per_device[device];
    return CX_OK;
}

long long noalloc_max_elements() { return kNoAllocMaxN; }

template <typename T>
int launch_compact(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                   const T* thr_host, const T* d_thr, int* d_size_prefix, bool no_alloc) {
    constexpr int kPairBytes = 4 * Elem<T>::pair_words;
    if (!out_msg || n < 0) return fail(CX_ERR_INVALID, "compress: null message buffer or negative size");
    if (no_alloc && (long long)n > kNoAllocMaxN)
        return fail(CX_ERR_INVALID, "cx_ip_compress_noalloc: %d elements exceed the limit of %lld", n, kNoAllocMaxN);
    if ((reinterpret_cast<uintptr_t>(out_msg) & 3u) != 0)
        return fail(CX_ERR_INVALID, "compress: message buffer must be 4-byte aligned");
    if (out_capacity < 8) return fail(CX_ERR_CAPACITY, "compress: message buffer smaller than its 8-byte header");
    unsigned* msg_words = static_cast<unsigned*>(out_msg);
    if ((!data && !update) || n == 0) {
        // no input vector: the reference falls through all three branches and emits an empty message
        hipLaunchKernelGGL(empty_message_kernel, dim3(1), dim3(1), 0, h->stream, msg_words, n, d_size_prefix);
        CX_HIP(hipGetLastError());
        return CX_OK;
    }
    const int mode = (data && update) ? 0 : (update ? 1 : 2);
    const long long cap_pairs = (out_capacity - 8) / kPairBytes;
    const T thr_val = thr_host ? *thr_host : (T)0;
    const T* thr_ptr = thr_host ? nullptr : (d_thr ? d_thr : static_cast<const T*>(h->d_thr));
    if (h->pending_pick.active && (mode != 0 || no_alloc || thr_ptr != h->pending_pick.thr_out)) {
        int rc = launch_pending_pick<T>(h);  // not a pass that can make the pick itself
        if (rc != CX_OK) return rc;
    }

    constexpr int kVec = 16 / (int)sizeof(T);
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(update)) & 15u) == 0;
    if (!vec_ok)  // sub-vectors at odd offsets: scalar loads, same tile order
        return launch_mode<T, 1, 16>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, d_size_prefix, no_alloc);
    // Tile shape (16-byte loads per lane).  Measured: 4 is the best on long vectors (the step on 100 M
    // elements: 0.219 / 0.208 / 0.213 ms with 2 / 4 / 8, on 64 Mi 150 / 144 us with 2 / 4); up to 8 Mi
    // elements 2 is as fast at 1 % density (40.3 / 40.8 us at 8 Mi) and faster where many survive, because
    // the gather kernel then has twice the blocks (61 706 elements at 10 %: 28.0 / 31.6 / 32.5 us).
    const int items = h->compact_items ? h->compact_items : (n <= (1 << 23) ? 2 : 4);
    switch (items) {
        case 2: return launch_mode<T, kVec, 2>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, d_size_prefix, no_alloc);
        case 4: return launch_mode<T, kVec, 4>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, d_size_prefix, no_alloc);
        case 8: return launch_mode<T, kVec, 8>(h, mode, data, update, n, thr_ptr, thr_val, msg_words, cap_pairs, d_size_prefix, no_alloc);
        default: return fail(CX_ERR_INVALID, "compress: unsupported compact_items %d", h->compact_items);
    }
}

// ---- fused exact top-k: candidate pass and final filter -------------------------------------
// Candidate pass: update += data; every element with |update| > *d_bound leaves the residual for
// the candidate list ((index, value) pairs, ascending, behind a message header in `cand_words`);
// what the list has no room for stays in the residual, the header counts it all the same.
template <typename T>
int launch_candidates(cx_handle h, unsigned* cand_words, long long cap_pairs, const T* data, T* update, int n,
                      const T* d_bound) {
    constexpr int kVec = 16 / (int)sizeof(T);
    switch (h->compact_items ? h->compact_items : 4) {  // (only long vectors come here)
        case 2: return launch_mode<T, kVec, 2>(h, 3, data, update, n, d_bound, (T)0, cand_words, cap_pairs, nullptr);
        case 4: return launch_mode<T, kVec, 4>(h, 3, data, update, n, d_bound, (T)0, cand_words, cap_pairs, nullptr);
        case 8: return launch_mode<T, kVec, 8>(h, 3, data, update, n, d_bound, (T)0, cand_words, cap_pairs, nullptr);
        default: return fail(CX_ERR_INVALID, "compress: unsupported compact_items %d", h->compact_items);
    }
}

namespace {

// Blocks of the two filter kernels: one per kFilterPerBlock candidates the caller expects, within these limits
// (measured as the whole single-pass call on 25.6 M elements at 0.1 %, about 54 000 candidates: 128 blocks
// 106.5 us, 2048 blocks 108.1 us; on 10^8 elements at 1 % no difference between 512, 1024 and 2048 per block).
constexpr int kFilterBlocks = 2048;
constexpr int kFilterMinBlocks = 128;
constexpr int kFilterPerBlock = 1024;
constexpr int kFilterBlock = 256;

// The candidate list is usable when it holds the wanted order statistic (more candidates than
// the rank) and nothing was dropped from it.
__device__ __forceinline__ bool candidates_usable(unsigned count, unsigned cap, unsigned long long rank) {
    return (unsigned long long)count > rank && count <= cap;
}

// Survivors (|value| > threshold) per block-sized share of the candidate list.  The threshold
// is the key the chained radix passes over the candidates end on: every block does the last
// pick itself from the last pass's histogram, block 0 stores the threshold for everyone after.
template <typename T>
__global__ __launch_bounds__(kFilterBlock) void filter_count_kernel(const unsigned* __restrict__ cand_words,
                                                                    unsigned cand_cap, unsigned long long rank,
                                                                    const SelectState* __restrict__ st,
                                                                    T* __restrict__ thr_out,
                                                                    unsigned* __restrict__ block_counts) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    using key_t = typename Elem<T>::key_t;
    __shared__ unsigned s_cnt, s_digit;
    __shared__ unsigned long long s_above, s_sum[kFilterBlock / 64];
    if (threadIdx.x == 0) s_cnt = 0u;
    const PickState done = state_entering_pass<T, kFilterBlock>(st, kPasses, rank, s_sum, &s_digit, &s_above);
    const T thr = value_of((key_t)done.prefix, T());
    if (blockIdx.x == 0 && threadIdx.x == 0) *thr_out = thr;
    const unsigned count = cand_words[1];
    unsigned mine = 0;
    if (candidates_usable(count, cand_cap, rank)) {
        const unsigned share = (count + gridDim.x - 1) / gridDim.x;
        const unsigned lo = blockIdx.x * share;
        const unsigned hi = lo + share < count ? lo + share : count;
        for (unsigned i = lo + threadIdx.x; i < hi; i += kFilterBlock)
            mine += mag(pair_value<T>(cand_words + 2 + (size_t)i * PW)) > thr ? 1u : 0u;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off, 64);
    if ((threadIdx.x & 63) == 0) atomicAdd(&s_cnt, mine);  // LDS
    __syncthreads();
    if (threadIdx.x == 0) block_counts[blockIdx.x] = s_cnt;
}

// Copies the survivors to the message in list order and gives the other candidates back to the
// residual (the candidate pass cleared them all); the last block writes the header.  When the
// list is not usable every listed candidate goes back and the message is not touched.
// result[0]: 0 = done, 1 = list not usable; result[1]: pairs in the message, or the candidate count.
template <typename T>
__global__ __launch_bounds__(kFilterBlock) void filter_write_kernel(
    const unsigned* __restrict__ cand_words, unsigned cand_cap, unsigned long long rank, const T* __restrict__ thr_ptr,
    const unsigned* __restrict__ block_counts, T* __restrict__ update, int n, unsigned* __restrict__ msg_words,
    long long cap_pairs, int* __restrict__ size_prefix, unsigned* __restrict__ result, DeviceStatus* status,
    SelectState* __restrict__ st) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int kWaves = kFilterBlock / 64;
    constexpr int kPasses = (Elem<T>::key_bits + kRadixBits - 1) / kRadixBits;
    __shared__ unsigned s_before;
    __shared__ unsigned s_wave[kWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (blockIdx.x == 0)  // the chained passes' histograms have been read by everyone who needs them
        for (int b = tid; b < kPasses * kRadixBins; b += kFilterBlock) (&st->pass_hist[0][0])[b] = 0u;
    const unsigned count = cand_words[1];
    if (!candidates_usable(count, cand_cap, rank)) {
        const unsigned listed = count < cand_cap ? count : cand_cap;
        for (unsigned i = blockIdx.x * kFilterBlock + tid; i < listed; i += gridDim.x * kFilterBlock) {
            const unsigned* w = cand_words + 2 + (size_t)i * PW;
            if (w[0] < (unsigned)n) update[w[0]] = pair_value<T>(w);
        }
        if (blockIdx.x == 0 && tid == 0) {
            result[0] = 1u;
            result[1] = count;
        }
        return;
    }
    if (tid == 0) s_before = 0u;
    __syncthreads();
    unsigned before = 0;
    for (unsigned b = tid; b < blockIdx.x; b += kFilterBlock) before += block_counts[b];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off, 64);
    if (lane == 0 && before) atomicAdd(&s_before, before);  // LDS
    __syncthreads();
    unsigned pos = s_before;  // survivors before the part of the share not yet walked

    const unsigned share = (count + gridDim.x - 1) / gridDim.x;
    const unsigned lo = blockIdx.x * share;
    const unsigned hi = lo + share < count ? lo + share : count;
    const T thr = *thr_ptr;
    const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    unsigned* const pairs = msg_words + 2;
    bool overflow = false;
    for (unsigned i0 = lo; i0 < hi; i0 += kFilterBlock) {  // uniform trip count per block
        const unsigned i = i0 + tid;
        unsigned w[PW];
        bool keep = false;
        if (i < hi) {
#pragma unroll
            for (int q = 0; q < PW; ++q) w[q] = cand_words[2 + (size_t)i * PW + q];
            keep = mag(pair_value<T>(w)) > thr;
            if (!keep && w[0] < (unsigned)n) update[w[0]] = pair_value<T>(w);  // stays behind
        }
        const unsigned long long votes = __ballot(keep);
        if (lane == 0) s_wave[wave] = (unsigned)__popcll(votes);
        __syncthreads();
        unsigned at = pos + (unsigned)__popcll(votes & below);
        unsigned all = 0;
#pragma unroll
        for (int q = 0; q < kWaves; ++q) {
            if (q < wave) at += s_wave[q];
            all += s_wave[q];
        }
        if (keep) {
            if ((long long)at < cap_pairs) {
#pragma unroll
                for (int q = 0; q < PW; ++q) pairs[(size_t)at * PW + q] = w[q];
            } else {
                if (w[0] < (unsigned)n) update[w[0]] = pair_value<T>(w);  // no room in the message: stays in the residual
                overflow = true;
            }
        }
        pos += all;
        __syncthreads();
    }
    if (overflow) atomicOr(&status->detail, 1);
    if (blockIdx.x == gridDim.x - 1 && tid == 0) {
        if ((long long)pos > cap_pairs) pos = (unsigned)cap_pairs;  // never announce more than was written
        msg_words[0] = (unsigned)n;
        msg_words[1] = pos;
        if (size_prefix) *size_prefix = (int)(8u + pos * (unsigned)(4 * PW));
        result[0] = 0u;
        result[1] = pos;
    }
}

}  // namespace

// Final steps of the fused exact top-k: the threshold (last pick of the chained passes over the
// candidates, left in *d_thr), then the candidates above it become the message, the
// others return to the residual; when the candidate list cannot hold the answer (result[0] = 1)
// all of them return and the residual holds the complete sum again.
template <typename T>
int launch_filter(cx_handle h, const unsigned* cand_words, unsigned cand_cap, unsigned long long rank, T* d_thr,
                  T* update, int n, unsigned* msg_words, long long cap_pairs, int* size_prefix, unsigned* d_result,
                  unsigned long long expected_candidates) {
    // per-share counts live behind the per-block sums of the streaming pass, which are consumed by now
    int rc = ensure_scratch(h, (size_t)kFilterBlocks * kWavesPerBlock, 0);
    if (rc != CX_OK) return rc;
    // every block redoes the last pick and sums the counts of the blocks before it: no more blocks than the
    // candidates the caller expects can keep busy (a longer list only makes the shares longer)
    unsigned long long want = (expected_candidates + kFilterPerBlock - 1) / kFilterPerBlock;
    if (want < (unsigned long long)kFilterMinBlocks) want = kFilterMinBlocks;
    if (want > (unsigned long long)kFilterBlocks) want = kFilterBlocks;
    const unsigned blocks = (unsigned)want;
    hipLaunchKernelGGL(filter_count_kernel<T>, dim3(blocks), dim3(kFilterBlock), 0, h->stream, cand_words,
                       cand_cap, rank, h->sel, d_thr, h->block_sums);
    hipLaunchKernelGGL(filter_write_kernel<T>, dim3(blocks), dim3(kFilterBlock), 0, h->stream, cand_words,
                       cand_cap, rank, d_thr, h->block_sums, update, n, msg_words, cap_pairs, size_prefix, d_result,
                       h->d_status, h->sel);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

#define CX_INSTANTIATE_FUSED(T)                                                                                      \
    template int launch_candidates<T>(cx_handle, unsigned*, long long, const T*, T*, int, const T*);                 \
    template int launch_filter<T>(cx_handle, const unsigned*, unsigned, unsigned long long, T*, T*, int,             \
                                  unsigned*, long long, int*, unsigned*, unsigned long long);
CX_INSTANTIATE_FUSED(float)
CX_INSTANTIATE_FUSED(double)
CX_INSTANTIATE_FUSED(int)
#undef CX_INSTANTIATE_FUSED

template <typename T> int reserve_compact(cx_handle h, int n) {
    size_t ntiles, words;
    scratch_need<T>(n, &ntiles, &words);
    if (ntiles < (size_t)kFilterBlocks * kWavesPerBlock) ntiles = (size_t)kFilterBlocks * kWavesPerBlock;  // launch_filter
    return ensure_scratch(h, ntiles, words);
}
template int reserve_compact<float>(cx_handle, int);
template int reserve_compact<double>(cx_handle, int);
template int reserve_compact<int>(cx_handle, int);
template int launch_compact<float>(cx_handle, void*, long long, const float*, float*, int, const float*, const float*, int*, bool);
template int launch_compact<double>(cx_handle, void*, long long, const double*, double*, int, const double*, const double*, int*, bool);
template int launch_compact<int>(cx_handle, void*, long long, const int*, int*, int, const int*, const int*, int*, bool);

}  // namespace cx
