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
                                                         const unsigned* __restrict__ msg, DeviceStatus* status,
                                                         const unsigned* __restrict__ skip_if = nullptr) {
    constexpr int PW = Elem<T>::pair_words;
    if (skip_if && *skip_if != 0u) return;  // the message is not index-sorted: the pair-after-pair kernel takes it
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
            if (j > 0 && (unsigned)p[-PW] > (unsigned)idx) bad = true;  // not index-sorted: equal indices may lie apart
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

struct MsgHeaders {
    static constexpr int kMax = 16;
    const unsigned* msg[kMax];
};

// The reference's loop for ANY message (src/compressor.hxx:613-658): pairs in the order they are
// stored, indices in any order, repeated anywhere.  One wavefront takes 64 pairs at a time; the
// chunks follow each other, and a chunk in which two pairs share an index is applied lane by lane.
// Slow (tens of ns per pair): the fallback for messages the sorted paths refuse.
template <typename T, int OP>
__global__ __launch_bounds__(64) void sequential_kernel(T* out, int out_n,
                                                       const unsigned* __restrict__ msg, DeviceStatus* status,
                                                       unsigned* run_if = nullptr) {
    constexpr int PW = Elem<T>::pair_words;
    if (run_if) {
        // launched behind the order check and the sorted-path kernel: runs only when the check found the
        // message unsorted (the sorted-path kernel then did nothing), and leaves the check's words clean
        const unsigned unsorted = run_if[0];
        __builtin_amdgcn_s_waitcnt(0);
        if (threadIdx.x == 0) {
            run_if[0] = 0u;
            run_if[1] = 0u;
        }
        if (unsorted == 0u) return;
    }
    const int n_msg = (int)msg[0];
    const long long k = (long long)(int)msg[1];
    if (n_msg > out_n) {
        if (threadIdx.x == 0) atomicCAS(&status->code, 0, (int)CX_ERR_MSG_TOO_LARGE);
        return;
    }
    const unsigned* pairs = msg + 2;
    const int lane = threadIdx.x;
    bool bad = false;
    for (long long j0 = 0; j0 < k; j0 += 64) {
        const long long j = j0 + lane;
        const bool live = j < k;
        const int idx = live ? (int)pairs[PW * j] : -1;
        const bool ok = live && (unsigned)idx < (unsigned)out_n;
        bad |= live && !ok;
        const T v = ok ? load_value<T>(pairs + PW * j + 1) : (T)0;
        bool shared = false;  // an earlier lane of this chunk has the same index
        for (int l = 0; l < 63; ++l) {
            const int other = __shfl(idx, l, 64);
            shared |= ok && l < lane && other == idx;
        }
        if (__ballot(shared) == 0ull) {
            if (ok) out[idx] = OP == 0 ? v : (T)(out[idx] + v);
        } else {
            for (int l = 0; l < 64; ++l) {
                if (l == lane && ok) out[idx] = OP == 0 ? v : (T)(out[idx] + v);
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                __builtin_amdgcn_s_waitcnt(0);  // the store has left before the next lane reads the element
            }
        }
        // the next chunk may touch the same elements: this one's stores come first
        __threadfence_block();
    }
    if (bad) atomicCAS(&status->code, 0, (int)CX_ERR_INDEX);
}

// *unsorted |= some message holds an index below its predecessor (or is made for a longer vector,
// which the caller's path then reports).  grid.y = message.  The fast paths need ascending indices;
// a caller that must take any order (the reference's loops do) asks first.  unsorted[1] += the
// messages' pair counts (what the dispatch between a pass over the whole vector and one scatter per
// message goes by).
__global__ __launch_bounds__(kBlock) void order_check_kernel(MsgHeaders list, unsigned* __restrict__ unsorted, int pair_words) {
    const unsigned* msg = list.msg[blockIdx.y];
    const long long k = (long long)(int)msg[1];
    if (blockIdx.x == 0 && threadIdx.x == 0 && k > 0) atomicAdd(unsorted + 1, (unsigned)k);
    const unsigned* pairs = msg + 2;
    const long long stride = (long long)gridDim.x * kBlock;
    bool bad = false;
    for (long long j = (long long)blockIdx.x * kBlock + threadIdx.x + 1; j < k; j += stride)
        bad |= pairs[(size_t)pair_words * j] < pairs[(size_t)pair_words * (j - 1)];
    if (__any(bad) && (threadIdx.x & 63) == 0) atomicOr(unsorted, 1u);
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
// (tiles of 8 / 32 / 48 KB in this design measured 140 / 95 / 99 us against 93 us on 64 Mi elements)
template <typename T> struct ReduceTile { static constexpr int value = 16384 / (int)sizeof(T); };
constexpr int kMaxMsgs = 16;

struct MsgList {
    const unsigned* msg[kMaxMsgs];
};

// bounds[t * kMaxMsgs + r] = first pair of message r whose index is >= t * (tile elements), for
// t in [0, ntiles]; blockIdx.y selects the message.
template <typename T>
__global__ __launch_bounds__(kBlock) void bounds_kernel(MsgList list, int out_n, unsigned ntiles,
                                                        unsigned* __restrict__ bounds, DeviceStatus* status,
                                                        const unsigned* __restrict__ skip_if) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int kReduceTile = ReduceTile<T>::value;
    if (skip_if && *skip_if != 0u) return;  // an order check in front found disorder: the pair-after-pair kernels take over
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
                                                       DeviceStatus* status, const unsigned* __restrict__ skip_if) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int VEC = 16 / (int)sizeof(T);
    constexpr int kReduceTile = ReduceTile<T>::value;
    __shared__ T tile[kReduceTile];
    if (skip_if && *skip_if != 0u) return;
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

// ---- merged, rank-ordered reduce: persistent blocks, no bounds pass ---------------------------
// out (+)= sum of up to kMergeMsgs index-sorted messages, applied in the order given, the dense
// vector written exactly once.  A block owns a CONTIGUOUS run of dense tiles; a message wavefront
// owns one or two of the messages.  At its start the wavefront finds (two memory round trips, all
// its searches side by side) where the block's index range begins and ends in its messages; from
// then on it walks them with a cursor: the slice streams through a ring of chunks in LDS, filled by asynchronous
// global-to-LDS loads a few chunks ahead of the cursor; each turn the wavefront looks at the 64
// pairs from the cursor on (lane 0 also at the pair before, for the order check), applies those
// below the tile's end to the LDS tile and moves the cursor.  So the only memory round trips a tile
// waits for were started several tiles earlier.
// Order of additions: the wavefronts apply messages 0 | 1 | ... | 7 (or 0,1 | 2,3 | 4,5 | 6,7) to a tile
// in consecutive steps, between barriers that wait for LDS only, never for the stores still in flight.
// Every pair of a message is looked at by exactly one block (the blocks' slices tile [0, k) by
// position), so a message that is not index-sorted, or holds an index outside the vector, is
// noticed: CX_ERR_INDEX, and no access leaves the tile.
constexpr int kMergeMsgs = 8;
// Adding into an existing vector: LOADER wavefronts bring a tile's old contents into its LDS buffer
// two steps before the first message wavefront gets there (asynchronous global-to-LDS loads in a
// queue of their own: a wavefront that also stores would wait for its stores with every load),
// which takes two more buffers.
constexpr int kPrefillAhead = 2;
// Shape of the pipeline for element type T, writing from zeros or adding into the vector.  All of
// a compute unit's 160 KB of LDS go to one block: tiles of 16 KB, one per pipeline stage, plus a
// ring of chunks per message.
//   4-byte elements from zeros: one message per message wavefront (8 stages), rings of 4 x 64 pairs:
//     9 x 16 KB + 8 x 2 KB = 160 KB.  Measured on 64 Mi elements, 8 messages of 1 %: 51 us, against
//     65 us with two messages per wavefront (4 stages; a wavefront's turn costs ~800 cycles whatever
//     it finds, and the two turns of a step were the block's critical path), 77 us with 8 stages of
//     8 KB tiles, 72 us with 8 KB tiles and two blocks per compute unit, 104 us with 4 KB tiles.
//   adding (4 more loader wavefronts, 2 more buffers) and 8-byte elements (12-byte pairs): two
//     messages per wavefront; rings of 4 x 128 pairs for 4-byte elements adding (144 KB) and for
//     8-byte elements from zeros (128 KB), 4 x 64 pairs for 8-byte elements adding (136 KB; with
//     8 KB tiles instead: 118 us against 97 us).  8-byte elements from zeros with one message per
//     wavefront need smaller tiles to fit (9 x 12 KB + 24 KB): 87 us against 68 us.
//   Writer wavefronts: 4 when writing from zeros (52 us against 59 us with 8, 69 us with 2: the
//     stores of more wavefronts queue up behind each other), 8 when adding (no difference there).
template <typename T, bool ACCUM> struct MergeCfg {
    static constexpr bool wide = !ACCUM && sizeof(T) == 4;  // one message per message wavefront
    static constexpr int msg_waves = wide ? 8 : 4;
    static constexpr int writer_waves = ACCUM ? 8 : 4;
    static constexpr int loader_waves = ACCUM ? 4 : 0;
    static constexpr int msgs_per_wave = kMergeMsgs / msg_waves;
    static constexpr int tile = 16384 / (int)sizeof(T);     // elements of a tile
    static constexpr int bufs = msg_waves + 1 + (ACCUM ? kPrefillAhead : 0);
    static constexpr int block = 64 * (msg_waves + writer_waves + loader_waves);
    static constexpr int chunk = (wide || (ACCUM && sizeof(T) == 8)) ? 64 : 128;  // pairs per chunk of a ring
    static constexpr int ring_chunks = 4;
    static constexpr int ring_pairs = chunk * ring_chunks;
};

struct MergeList {
    const unsigned* msg[kMergeMsgs];
};

// Barrier that orders LDS traffic only: a full __syncthreads(), or a fence on the LDS address space,
// also waits for every global store the wavefront has in flight and for its asynchronous
// global-to-LDS loads, which would put a memory round trip into every tile.  Every wavefront's own
// LDS reads and writes are complete when it arrives, so what it wrote is visible to the others
// behind the barrier; the memory clobber keeps the compiler from moving LDS accesses across.
// One dword per active lane from global memory straight into LDS, at byte offset `lds_base` of the
// block's LDS plus 4 * lane; nothing waits for it here.  The compiler is not told: it would make
// every later LDS access it cannot tell apart from the target wait for the load.  Whoever reads the
// target waits for it first (s_waitcnt vmcnt; loads retire in the order they were issued).  M0
// carries the LDS offset and is restored.
__device__ __forceinline__ void async_load_to_lds(const unsigned* src, unsigned lds_base) {
    unsigned keep;
    asm volatile(
        "s_mov_b32 %0, m0\n\t"
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %1, off\n\t"
        "s_mov_b32 m0, %0"
        : "=&s"(keep)
        : "v"(src), "s"(lds_base)
        : "memory");
}

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// NS (at most four) lower bounds at once, by one wavefront: for each search s the first position j
// in [0, k[s]) of its message with index(j) >= target[s] (unsigned compare), k[s] if there is none.
// While a bracket is wider than 256 pairs, the 16 lanes of quarter s probe 16 evenly spaced
// positions of it (one memory round trip for all searches, 16 cache lines per search); then every
// bracket is read whole by the wavefront (four coalesced loads per lane: 16 cache lines) and the
// pairs below the target are counted.  The first bracket is a guess (indices spread evenly over
// [0, n_hint)), checked by two extra probes in the same round: two round trips then.  No load sits
// in a branch (a load whose result is merged behind a branch is waited for at the branch, and the
// searches would take their round trips one after the other): lanes with nothing to ask read a
// pair of their own bracket, or `safe` when there is no message.  Positions fit 32 bits (k < 2^31).
// The result depends on the message and the target only, so two blocks that look for the same
// boundary agree, also on a message that is not sorted (where it is just some position in [0, k];
// the callers notice the disorder).
template <int PW, int NS>
__device__ __forceinline__ void wave_lower_bound(const unsigned* const (&pairs)[NS], const unsigned (&k)[NS],
                                                 const unsigned (&target)[NS], unsigned n_hint, int lane,
                                                 const unsigned* safe, unsigned (&found)[NS]) {
    static_assert(NS >= 1 && NS <= 4, "one quarter of the wavefront probes for each search");
    constexpr unsigned kCountSpan = 256u;
    const unsigned sub = (unsigned)lane & 15u;
    const int quarter = lane >> 4;
    unsigned lo[NS], hi[NS];
    bool guessed[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        lo[s] = 0u;
        hi[s] = k[s];
        guessed[s] = false;
        if (k[s] > 16384u && n_hint > 0u && target[s] <= n_hint) {
            const unsigned g = (unsigned)((unsigned long long)target[s] * k[s] / n_hint);  // <= k
            lo[s] = g > 2048u ? g - 2048u : 0u;
            hi[s] = k[s] - g > 2048u ? g + 2048u : k[s];
            guessed[s] = true;
        }
    }
    for (int round = 0; round < 64; ++round) {  // 16-fold narrowing: a handful of rounds; bounded all the same
        bool wide = false;
#pragma unroll
        for (int s = 0; s < NS; ++s) wide |= guessed[s] || hi[s] - lo[s] > kCountSpan;
        if (!__any(wide)) break;
        unsigned step[NS], val[NS], edge[NS];
        bool probing[NS], valid[NS], edge_lo[NS], edge_hi[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const unsigned span = hi[s] - lo[s];
            probing[s] = guessed[s] || span > kCountSpan;
            step[s] = (span + 15u) >> 4;
            const unsigned* const idle = k[s] > 0u ? pairs[s] + (size_t)(lo[s] < k[s] ? lo[s] : k[s] - 1u) * PW : safe;
            const unsigned pos = lo[s] + sub * step[s];  // < 2^32: span < 2^31
            valid[s] = probing[s] && quarter == s && pos < hi[s];
            val[s] = *(valid[s] ? pairs[s] + (size_t)pos * PW : idle);
            // the guess holds when the pair before the bracket is below the target (lane 0 of the
            // quarter looks) and the pair at its end is not (lane 1 looks)
            edge_lo[s] = guessed[s] && quarter == s && sub == 0u && lo[s] > 0u;
            edge_hi[s] = guessed[s] && quarter == s && sub == 1u && hi[s] < k[s];
            edge[s] = *(edge_lo[s] ? pairs[s] + (size_t)(lo[s] - 1u) * PW
                                   : edge_hi[s] ? pairs[s] + (size_t)hi[s] * PW : idle);
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const bool chk = edge_lo[s] ? edge[s] < target[s] : edge_hi[s] ? edge[s] >= target[s] : true;
            const unsigned good = (unsigned)(__ballot(chk) >> (16 * s)) & 0xffffu;
            const unsigned ge = (unsigned)(__ballot(!valid[s] || val[s] >= target[s]) >> (16 * s)) & 0xffffu;
            if (!probing[s]) continue;
            if (guessed[s]) {
                guessed[s] = false;
                if (good != 0xffffu) {  // wrong guess: search the whole message
                    lo[s] = 0u;
                    hi[s] = k[s];
                    continue;
                }
            }
            const unsigned f = ge ? (unsigned)__ffs((int)ge) - 1u : 16u;  // first probe at or above the target
            const unsigned base = lo[s];
            if (f < 16u) {
                const unsigned pf = base + f * step[s];
                if (pf < hi[s]) hi[s] = pf;
            }
            if (f > 0u) {
                const unsigned pl = base + (f - 1u) * step[s] + 1u;
                lo[s] = pl < hi[s] ? pl : hi[s];
            }
        }
    }
    // every bracket holds at most 256 pairs now: those below the target are counted
    unsigned cidx[NS][4];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const unsigned* const idle = k[s] > 0u ? pairs[s] + (size_t)(lo[s] < k[s] ? lo[s] : k[s] - 1u) * PW : safe;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned p = lo[s] + (unsigned)(lane + 64 * j);
            cidx[s][j] = *(p < hi[s] ? pairs[s] + (size_t)p * PW : idle);
        }
    }
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        unsigned cnt = 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned p = lo[s] + (unsigned)(lane + 64 * j);
            cnt += (unsigned)__popcll(__ballot(p < hi[s] && cidx[s][j] < target[s]));
        }
        found[s] = lo[s] + cnt;
    }
}

// A message wavefront's view of one message: a ring of chunks of kChunk pairs each in
// LDS, filled straight from global memory, chunk by chunk, a few chunks ahead of the cursor (under
// a saturated write stream a read takes several microseconds, far more than a tile's turn, and
// chunks lie at fixed positions, so they can be asked for long before the cursor gets there).  Each
// turn the wavefront looks at the 64 pairs from the cursor on, one per lane.
constexpr unsigned kNoPair = 0xffffffffu;  // stands for a pair behind the end of the slice

// The index of the lane below (lane 0: `first`), without a trip through LDS.
__device__ __forceinline__ unsigned lane_below(unsigned v, unsigned first) {
    return (unsigned)__builtin_amdgcn_update_dpp((int)first, (int)v, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
}

// OP 0: out = scatter of the (single) message, the last pair of a run of equal indices wins;
// OP 1: out (+)= messages in order (without ACCUM: added to zeros).
//
// A block is a pipeline over its tiles.  MESSAGE wavefront w (MergeCfg::msg_waves of them, one
// or two messages each) adds its pairs to tile s - w in step s, so the additions to one tile happen in message order,
// one wavefront per step, while the wavefronts all work at once, on different tiles.  They never
// store to global memory and never wait for it, except for a chunk that has been on its way for
// several tiles.  WRITER wavefronts stream out the tile the last message wavefront finished a step
// ago and, when nothing is accumulated, leave its LDS buffer zeroed; they never load, so the stores
// of many tiles are in flight per block.  When accumulating, LOADER wavefronts fill a buffer with the
// old contents of the tile that uses it next, kPrefillAhead steps before the first message wavefront
// gets there.  MergeCfg::bufs LDS tiles rotate; one barrier per step.
template <typename T, int OP, bool ACCUM>
__global__ __launch_bounds__((MergeCfg<T, ACCUM>::block)) void merge_kernel(T* __restrict__ out, int out_n, MergeList list,
                                                            int n_msgs, unsigned ntiles, unsigned tiles_per_block,
                                                            DeviceStatus* status) {
    constexpr int PW = Elem<T>::pair_words;
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef MergeCfg<T, ACCUM> Cfg;
    constexpr int kMergeWaves = Cfg::msg_waves, kWriterWaves = Cfg::writer_waves, kLoaderWaves = Cfg::loader_waves;
    constexpr int kMsgsPerWave = Cfg::msgs_per_wave;
    constexpr int kChunk = Cfg::chunk;
    constexpr int kTile = Cfg::tile;
    constexpr int kRingChunks = Cfg::ring_chunks;
    constexpr int kRingPairs = Cfg::ring_pairs;
    constexpr int kWriters = 64 * kWriterWaves;      // writer threads
    constexpr int kVecs = kTile / VEC / kWriters;                  // 16-byte vectors a writer thread moves per tile
    static_assert(kVecs * kWriters * VEC == kTile, "the writers cover a tile exactly");
    constexpr int kBufs = Cfg::bufs;
    __shared__ T tiles[kBufs][kTile];
    __shared__ unsigned stage[kMergeWaves][kMsgsPerWave][kRingPairs * PW];  // the rings of chunks, per message
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same for the whole wavefront: scalar branches
    const bool writer = wave >= kMergeWaves && wave < kMergeWaves + kWriterWaves;
    const bool loader = ACCUM && wave >= kMergeWaves + kWriterWaves;
    const unsigned t0 = blockIdx.x * tiles_per_block;
    if (t0 >= ntiles) return;
    const unsigned t1 = t0 + tiles_per_block < ntiles ? t0 + tiles_per_block : ntiles;
    const unsigned my_tiles = t1 - t0;
    const unsigned steps = my_tiles + (unsigned)kMergeWaves;  // the last tile leaves kMergeWaves steps after it entered

    if (!ACCUM && writer) {
        // every buffer starts as zeros (before anything that waits for memory: the headers are on their way)
        constexpr int kZeroVecs = kBufs * kTile / VEC;
        Pack<T, VEC> z;
#pragma unroll
        for (int c = 0; c < VEC; ++c) z.x[c] = (T)0;
        Pack<T, VEC>* const all = reinterpret_cast<Pack<T, VEC>*>(&tiles[0][0]);
#pragma unroll 4
        for (int i = tid - 64 * kMergeWaves; i < kZeroVecs; i += kWriters) all[i] = z;
    }
    // headers (the same for every thread): both words of all of them in one round trip
    // (plain loads from addresses that are the same in every lane; an absent message reads `out`)
    unsigned hdr_n[kMergeMsgs], hdr_k[kMergeMsgs];
#pragma unroll
    for (int r = 0; r < kMergeMsgs; ++r) {
        const unsigned* m = r < n_msgs ? list.msg[r] : reinterpret_cast<const unsigned*>(out);
        hdr_n[r] = m[0];
        hdr_k[r] = m[1];
    }
    bool too_large = false;
#pragma unroll
    for (int r = 0; r < kMergeMsgs; ++r) too_large |= r < n_msgs && (int)hdr_n[r] > out_n;
    if (too_large) {
        if (blockIdx.x == 0 && tid == 0) atomicCAS(&status->code, 0, (int)CX_ERR_MSG_TOO_LARGE);
        if (ACCUM) return;  // add: nothing is touched
        n_msgs = 0;         // decompress: the output is zeroed all the same
    }
    const bool aligned = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    auto tile_valid = [&](unsigned t) {  // elements of the vector inside tile t (0 behind the block's last)
        if (t >= t1) return 0;
        const long long left = (long long)out_n - (long long)t * kTile;
        return (int)(left < kTile ? left : kTile);
    };

    typedef __attribute__((address_space(3))) void* lds_ptr_t;
    if (loader) {
        // ---- loader wavefronts (accumulating only) ----
        constexpr int kTileDwords = kTile * (int)sizeof(T) / 4;
        constexpr int kLoadDiv = kLoaderWaves > 0 ? kLoaderWaves : 1;
        constexpr int kLoadsPerWave = kTileDwords / 64 / kLoadDiv;  // one dword per lane each
        static_assert(!ACCUM || kLoadsPerWave * 64 * kLoaderWaves == kTileDwords, "the loaders cover a tile exactly");
        const int lw = wave - (kMergeWaves + kWriterWaves);
        const unsigned* const safe = reinterpret_cast<const unsigned*>(out);  // out_n > 0: the first element exists
        auto prefill = [&](unsigned a) {  // tile a of this block: old contents into its buffer
            const unsigned t = t0 + a;
            const unsigned valid_dwords = (unsigned)tile_valid(t) * (unsigned)(sizeof(T) / 4);
            const unsigned* src = reinterpret_cast<const unsigned*>(out + (long long)t * kTile);
            const unsigned lds = (unsigned)(uintptr_t)(lds_ptr_t)&tiles[a % (unsigned)kBufs][0];
#pragma unroll
            for (int c = 0; c < kLoadsPerWave; ++c) {
                const unsigned j = (unsigned)((lw * kLoadsPerWave + c) * 64 + lane);
                // (what lies behind the vector's end is never written out; those lanes read the first element)
                async_load_to_lds(j < valid_dwords ? src + j : safe,
                                  (unsigned)__builtin_amdgcn_readfirstlane((int)(lds + (unsigned)((lw * kLoadsPerWave + c) * 256))));
            }
        };
        for (unsigned a = 0; a < (unsigned)kPrefillAhead && a < my_tiles; ++a) prefill(a);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
        for (unsigned s = 0; s < steps; ++s) {
            // the buffer of tile s + kPrefillAhead was drained a step ago; the tile the first message
            // wavefront takes next step (asked for a step ago) has landed when only this step's
            // loads are still in flight
            const unsigned a = s + (unsigned)kPrefillAhead;
            if (a < my_tiles) {
                prefill(a);
                __builtin_amdgcn_s_waitcnt(0x0f70 | ((kLoadsPerWave & 0xf)) | ((kLoadsPerWave >> 4) << 14));
            } else {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            lds_barrier();
        }
        return;
    }
    if (writer) {
        const int wt = tid - 64 * kMergeWaves;
        lds_barrier();
        for (unsigned s = 0; s < steps; ++s) {
            const bool draining = s >= (unsigned)kMergeWaves;
            const unsigned d = s - (unsigned)kMergeWaves;  // tile (of this block) that is streamed out
            T* dbuf = tiles[d % (unsigned)kBufs];
            const long long base = (long long)(t0 + d) * kTile;
            const int valid = draining ? tile_valid(t0 + d) : 0;
            const bool fast = draining && aligned && valid == kTile;
#pragma unroll
            for (int q = 0; q < kVecs; ++q) {
                const int e = (q * kWriters + wt) * VEC;
                if (fast) {
                    const Pack<T, VEC> v = *reinterpret_cast<const Pack<T, VEC>*>(&dbuf[e]);
                    vec_t vv;
#pragma unroll
                    for (int c = 0; c < VEC; ++c) vv[c] = v.x[c];
                    // (nontemporal: the vector is written once.  Plain stores: 78 against 52 us from zeros and 100 against
                    // 95 us adding, 8 messages into 64 Mi fp32 elements; what reads the vector next gains nothing)
                    __builtin_nontemporal_store(vv, reinterpret_cast<vec_t*>(out + base + e));
                } else if (draining) {
#pragma unroll
                    for (int c = 0; c < VEC; ++c)
                        if (e + c < valid) out[base + e + c] = dbuf[e + c];
                }
                if (draining && !ACCUM) {  // the buffer's next tile starts from zeros (the loaders fill it otherwise)
                    Pack<T, VEC> z;
#pragma unroll
                    for (int c = 0; c < VEC; ++c) z.x[c] = (T)0;
                    *reinterpret_cast<Pack<T, VEC>*>(&dbuf[e]) = z;
                }
            }
            lds_barrier();
        }
        return;
    }

    // ---- message wavefronts ----
    // this wavefront's messages and the slice of each that belongs to the block's tiles
    const unsigned* pairs[kMsgsPerWave];
    unsigned cur[kMsgsPerWave], end[kMsgsPerWave];
    bool bad = false;
    {
        static_assert(kMsgsPerWave == 1 || kMsgsPerWave == 2, "a wavefront's quarters search two boundaries of up to two messages");
        // search 2s: where the block's range starts in message s, search 2s + 1: where it ends
        const unsigned* sp[2 * kMsgsPerWave];
        unsigned sk[2 * kMsgsPerWave], st[2 * kMsgsPerWave], sf[2 * kMsgsPerWave];
#pragma unroll
        for (int s = 0; s < kMsgsPerWave; ++s) {
            const int r = wave * kMsgsPerWave + s;
            const unsigned* msg = nullptr;
            int k = 0;
#pragma unroll
            for (int q = 0; q < kMergeMsgs; ++q)  // (a chain of selects: no indexing of registers)
                if (q == r && q < n_msgs) {
                    msg = list.msg[q];
                    k = (int)hdr_k[q];
                }
            pairs[s] = msg ? msg + 2 : nullptr;
            sp[2 * s] = sp[2 * s + 1] = pairs[s];
            sk[2 * s] = sk[2 * s + 1] = k > 0 ? (unsigned)k : 0u;
            st[2 * s] = t0 * (unsigned)kTile;  // < 2^31 + tile: fits 32 bits
            st[2 * s + 1] = t1 * (unsigned)kTile;
        }
        wave_lower_bound<PW, 2 * kMsgsPerWave>(sp, sk, st, (unsigned)out_n, lane, reinterpret_cast<const unsigned*>(out + (size_t)t0 * kTile), sf);
#pragma unroll
        for (int s = 0; s < kMsgsPerWave; ++s) {
            // (wave-uniform values, kept in scalar registers)
            cur[s] = t0 == 0u ? 0u : (unsigned)__builtin_amdgcn_readfirstlane((int)sf[2 * s]);  // the first block starts at the first pair,
            end[s] = t1 == ntiles ? sk[2 * s] : (unsigned)__builtin_amdgcn_readfirstlane((int)sf[2 * s + 1]);  // the last ends behind the last
            if (end[s] < cur[s]) {  // not sorted
                bad = true;
                end[s] = cur[s];
            }
        }
    }

    // per message: the ring of chunks.  Chunk j holds the pairs at positions origin + j * kChunk ..;
    // chunks up to `issued` - 1 have been asked for (the cursor's chunk and the kRingChunks - 1 behind it).  Every chunk is asked for with the same number
    // of load instructions (lanes behind the slice's end read the message's header instead), so
    // "all but the last two chunks have landed" is a count of loads still in flight.
    typedef __attribute__((address_space(3))) void* lptr_t;
    constexpr int kChunkLoads = kChunk * PW / 64;  // one dword per lane each
    unsigned origin[kMsgsPerWave], issued[kMsgsPerWave], last_idx[kMsgsPerWave], ring_base[kMsgsPerWave];
    const unsigned* lane_src[kMsgsPerWave];  // this lane's word of the slice's first 64
    auto fetch_chunk = [&](int s, unsigned j) {
        // words of the chunk that exist (the slice ends at `end`)
        const unsigned long long first = (unsigned long long)j * (unsigned)kChunk;
        const unsigned long long total = (unsigned long long)(end[s] - origin[s]);
        const unsigned long long have = first < total ? total - first : 0ull;
        const unsigned words = have >= (unsigned long long)kChunk ? (unsigned)(kChunk * PW) : (unsigned)have * PW;
        const unsigned* src = lane_src[s] + (size_t)first * PW;
        const unsigned slot = ring_base[s] + (j % (unsigned)kRingChunks) * (unsigned)(kChunk * PW * 4);
#pragma unroll
        for (int c = 0; c < kChunkLoads; ++c)
            async_load_to_lds((unsigned)(c * 64 + lane) < words ? src + c * 64 : pairs[s] - 2,
                              (unsigned)__builtin_amdgcn_readfirstlane((int)(slot + (unsigned)(c * 256))));
    };
#pragma unroll
    for (int s = 0; s < kMsgsPerWave; ++s) {
        origin[s] = cur[s];
        issued[s] = 0u;
        last_idx[s] = kNoPair;
        lane_src[s] = pairs[s] + (size_t)origin[s] * PW + lane;
        ring_base[s] = (unsigned)(uintptr_t)(lptr_t)&stage[wave][s][0];
        if (wave * kMsgsPerWave + s < n_msgs) {
            for (unsigned j = 0; j < (unsigned)kRingChunks; ++j) fetch_chunk(s, j);
            issued[s] = (unsigned)kRingChunks;
        }
    }
    // the pair before the slice belongs to the block before: it must lie below this block's range
    // (asked for behind the chunks, so that one round trip serves both)
#pragma unroll
    for (int s = 0; s < kMsgsPerWave; ++s) {
        if (wave * kMsgsPerWave + s < n_msgs) {
            unsigned before = kNoPair;
            if (lane == 0 && cur[s] > 0u && cur[s] <= end[s]) before = pairs[s][(size_t)(cur[s] - 1u) * PW];
            before = (unsigned)__builtin_amdgcn_readfirstlane((int)before);
            if (before != kNoPair && before >= t0 * (unsigned)kTile) bad = true;
            last_idx[s] = before;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the first chunks have landed
    // the 64 pairs from the cursor on, as the ring holds them; read again whenever the cursor moves
    unsigned nidx[kMsgsPerWave];
    T nval[kMsgsPerWave];
    auto read_ring = [&](int s) {
        const unsigned* w = &stage[wave][s][((cur[s] - origin[s] + (unsigned)lane) % (unsigned)kRingPairs) * PW];
        nidx[s] = w[0];
        nval[s] = load_value<T>(w + 1);
    };
#pragma unroll
    for (int s = 0; s < kMsgsPerWave; ++s) read_ring(s);
    lds_barrier();  // the writers have prepared the buffers

    unsigned buf = 0u;  // LDS buffer of the tile this wavefront works on
    for (unsigned step = 0; step < steps; ++step) {
        const unsigned a = step - (unsigned)wave;  // tile (of this block) this wavefront works on in this step
        if (step >= (unsigned)wave && a < my_tiles) {
            const unsigned t = t0 + a;
            T* tile = tiles[buf];
            buf = buf + 1u == (unsigned)kBufs ? 0u : buf + 1u;
            const unsigned base = t * (unsigned)kTile;
            const unsigned valid = (unsigned)tile_valid(t);
            const unsigned tile_end = base + valid;
#pragma unroll
            for (int s = 0; s < kMsgsPerWave; ++s) {
                const int r = wave * kMsgsPerWave + s;
                if (r >= n_msgs) continue;
                const bool store_first = OP == 0;
                for (;;) {  // once, unless 64 or more pairs of the message fall into this tile
                    // the 64 pairs from the cursor on, one per lane (read from the ring when the cursor moved)
                    const unsigned left = end[s] - cur[s];  // pairs of the slice not yet used
                    const unsigned idx = (unsigned)lane < left ? nidx[s] : kNoPair;
                    const T val = nval[s];
                    // with ascending indices the pairs below the tile's end are the first `cnt` lanes
                    const unsigned long long below = __ballot(idx < tile_end);
                    const unsigned cnt = (unsigned)__popcll(below);
                    const bool mine = (unsigned)lane < cnt;
                    const unsigned prev = lane_below(idx, last_idx[s]);
                    if (mine && prev != kNoPair && idx < prev) bad = true;
                    const unsigned local = idx - base;
                    const bool hit = mine && local < valid;
                    if (mine && !hit) bad = true;
                    if (!__any(mine && lane > 0 && idx == prev)) {
                        if (hit) tile[local] = store_first ? val : (T)(tile[local] + val);
                    } else {
                        // equal indices inside one message: one pair at a time, in message order
                        for (unsigned i = 0; i < cnt; ++i) {
                            if ((unsigned)lane == i && hit) tile[local] = store_first ? val : (T)(tile[local] + val);
                            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        }
                    }
                    if (cnt == 0u) break;
                    last_idx[s] = (unsigned)__builtin_amdgcn_readlane((int)idx, (int)(cnt - 1u));
                    const unsigned was = (cur[s] - origin[s]) / (unsigned)kChunk;
                    cur[s] += cnt;
                    const unsigned now = (cur[s] - origin[s]) / (unsigned)kChunk;
                    if (now != was) {
                        // the cursor has left a chunk behind: its place in the ring goes to the chunk
                        // kRingChunks - 1 ahead; then everything but the kRingChunks - 2 chunks asked for
                        // last has landed, which covers the cursor's chunk and the next
                        fetch_chunk(s, issued[s]);
                        issued[s] += 1u;
                        constexpr int kInFlight = (kRingChunks - 2) * kChunkLoads;  // loads that may still be out
                        static_assert(kInFlight < 64, "the wait counter has six bits");
                        __builtin_amdgcn_s_waitcnt(/* vmcnt = kInFlight, the other counters free */
                                                   (kInFlight & 0xf) | ((kInFlight >> 4) << 14) | 0x0f70);
                        asm volatile("" ::: "memory");
                    }
                    read_ring(s);  // for the next turn; nothing waits for it here
                    if (cnt < 64u || cur[s] >= end[s]) break;
                }
            }
        }
        lds_barrier();  // the next wavefront takes the tile over; the drained buffer is clean
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no window may land in LDS after the block has gone
    // pairs left over in the slice lie beyond the block's tiles: out of range, or not sorted
#pragma unroll
    for (int s = 0; s < kMsgsPerWave; ++s)
        if (cur[s] < end[s]) bad = true;
    if (bad) atomicCAS(&status->code, 0, (int)CX_ERR_INDEX);
}

// An empty output vector: nothing to write, but a message made for a longer vector is still an
// error (the reference throws, src/compressor.hxx:620-624,645-647).
__global__ void header_check_kernel(MsgHeaders list, int n_msgs, DeviceStatus* status) {
    for (int r = threadIdx.x; r < n_msgs; r += blockDim.x)
        if ((int)list.msg[r][0] > 0) atomicCAS(&status->code, 0, (int)CX_ERR_MSG_TOO_LARGE);
}

int check_headers(cx_handle h, const void* const* msgs, int n_msgs) {
    for (int first = 0; first < n_msgs; first += MsgHeaders::kMax) {
        MsgHeaders list;
        const int cnt = n_msgs - first < MsgHeaders::kMax ? n_msgs - first : MsgHeaders::kMax;
        for (int r = 0; r < MsgHeaders::kMax; ++r)
            list.msg[r] = r < cnt ? static_cast<const unsigned*>(msgs[first + r]) : nullptr;
        hipLaunchKernelGGL(header_check_kernel, dim3(1), dim3(64), 0, h->stream, list, cnt, h->d_status);
    }
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T>
int launch_tiled(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int op, int accumulate,
                 const unsigned* skip_if = nullptr);

template <typename T>
int launch_merged(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int op, int accumulate) {
    if (out_n == 0) return check_headers(h, msgs, n_msgs);
    // persistent blocks: a few per compute unit, each with a contiguous run of tiles
    unsigned want_blocks = (unsigned)(h->cu_count > 0 ? h->cu_count : 256) * (unsigned)h->reduce_blocks_per_cu;
    if (want_blocks < 1u) want_blocks = 1u;
    for (int first = 0; first < n_msgs || first == 0; first += kMergeMsgs) {
        MergeList list;
        const int cnt = n_msgs - first < kMergeMsgs ? n_msgs - first : kMergeMsgs;
        for (int r = 0; r < kMergeMsgs; ++r)
            list.msg[r] = r < cnt ? static_cast<const unsigned*>(msgs[first + r]) : nullptr;
        const bool acc = accumulate || first > 0;
#define CX_MERGED(OP, ACC)                                                                                          \
    do {                                                                                                            \
        typedef MergeCfg<T, ACC> Cfg;                                                                               \
        const unsigned ntiles = (unsigned)(((long long)out_n + Cfg::tile - 1) / Cfg::tile);                          \
        unsigned tiles_per_block = (ntiles + want_blocks - 1u) / want_blocks;                                       \
        if (tiles_per_block < 1u) tiles_per_block = 1u;                                                             \
        const unsigned grid = (ntiles + tiles_per_block - 1u) / tiles_per_block;                                    \
        hipLaunchKernelGGL((merge_kernel<T, OP, ACC>), dim3(grid), dim3(Cfg::block), 0, h->stream, out, out_n, list, \
                           cnt > 0 ? cnt : 0, ntiles, tiles_per_block, h->d_status);                                \
    } while (0)
        if (op == 0) {
            CX_MERGED(0, false);
        } else if (!acc) {
            CX_MERGED(1, false);
        } else {
            CX_MERGED(1, true);
        }
#undef CX_MERGED
        if (n_msgs == 0) break;
    }
    CX_HIP(hipGetLastError());
    return CX_OK;
}

// first pair of each message in each dense tile, for the tiled reduce
int ensure_bounds(cx_handle h, size_t need) {
    if (need > h->reduce_bounds_cap) {
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->reduce_bounds) CX_HIP(hipFree(h->reduce_bounds));
        h->reduce_bounds = nullptr;
        h->reduce_bounds_cap = 0;
        CX_HIP(hipMalloc(reinterpret_cast<void**>(&h->reduce_bounds), need * sizeof(unsigned)));
        h->reduce_bounds_cap = need;
    }
    return CX_OK;
}

template <typename T>
int launch_tiled(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int op, int accumulate,
                 const unsigned* skip_if) {
    if (out_n == 0) return check_headers(h, msgs, n_msgs);
    constexpr int kReduceTile = ReduceTile<T>::value;
    const unsigned ntiles = (unsigned)(((long long)out_n + kReduceTile - 1) / kReduceTile);
    int rc_bounds = ensure_bounds(h, (size_t)kMaxMsgs * (ntiles + 1));
    if (rc_bounds != CX_OK) return rc_bounds;
    for (int first = 0; first < n_msgs || first == 0; first += kMaxMsgs) {
        MsgList list;
        const int cnt = n_msgs - first < kMaxMsgs ? n_msgs - first : kMaxMsgs;
        for (int r = 0; r < kMaxMsgs; ++r) list.msg[r] = r < cnt ? static_cast<const unsigned*>(msgs[first + r]) : nullptr;
        if (cnt > 0) {
            unsigned grid = (unsigned)(((long long)out_n / 64 + kBlock - 1) / kBlock);  // k <= n: ~1 thread per 64 elements
            if (grid < 1) grid = 1;
            if (grid > 1024) grid = 1024;
            hipLaunchKernelGGL(bounds_kernel<T>, dim3(grid, cnt), dim3(kBlock), 0, h->stream, list, out_n, ntiles,
                               h->reduce_bounds, h->d_status, skip_if);
        }
        const bool acc = accumulate || first > 0;
#define CX_TILED(OP, ACC, RMAX)                                                                                     \
    hipLaunchKernelGGL((tiled_kernel<T, OP, ACC, RMAX>), dim3(ntiles), dim3(kBlock), 0, h->stream, out, out_n, list, \
                       cnt, ntiles, h->reduce_bounds, h->d_status, skip_if)
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
__global__ __launch_bounds__(kBlock) void zero_kernel(T* __restrict__ v, long long n,
                                                      const unsigned* __restrict__ run_if = nullptr) {
    if (run_if && *run_if == 0u) return;
    const long long stride = (long long)gridDim.x * kBlock;
    const long long nvec = n / VEC;
    Pack<T, VEC> z;
#pragma unroll
    for (int c = 0; c < VEC; ++c) z.x[c] = (T)0;
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += stride)
        reinterpret_cast<Pack<T, VEC>*>(v)[i] = z;
    for (long long i = nvec * VEC + (long long)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) v[i] = (T)0;
}

// data[i] += rests[i].  A block owns kAddUnroll * kBlock consecutive 16-byte vectors; every load of a
// thread is issued before the first add.  `rests` is read once and `data` rewritten once per call:
// both go past the caches (nontemporal); the reads of `data` stay cacheable.
constexpr int kAddUnroll = 4;
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void add_vec_kernel(T* __restrict__ data, const T* __restrict__ rests,
                                                         long long n) {
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const long long nvec = n / VEC;
    const long long first = (long long)blockIdx.x * (kBlock * kAddUnroll) + threadIdx.x;
    if (VEC > 1 && first + (long long)(kAddUnroll - 1) * kBlock < nvec) {
        vec_t a[kAddUnroll], b[kAddUnroll];
#pragma unroll
        for (int q = 0; q < kAddUnroll; ++q) {
            a[q] = reinterpret_cast<const vec_t*>(data)[first + q * kBlock];
            b[q] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(rests) + first + q * kBlock);
        }
#pragma unroll
        for (int q = 0; q < kAddUnroll; ++q) {
#pragma unroll
            for (int c = 0; c < VEC; ++c) a[q][c] = (T)(a[q][c] + b[q][c]);
            __builtin_nontemporal_store(a[q], reinterpret_cast<vec_t*>(data) + first + q * kBlock);
        }
    } else {
        for (int q = 0; q < kAddUnroll; ++q) {
            const long long v = first + (long long)q * kBlock;
            if (v < nvec) {
#pragma unroll
                for (int c = 0; c < VEC; ++c) data[v * VEC + c] = (T)(data[v * VEC + c] + rests[v * VEC + c]);
            }
        }
    }
    // elements behind the last whole vector
    if (blockIdx.x == 0)
        for (long long i = nvec * VEC + threadIdx.x; i < n; i += kBlock) data[i] = (T)(data[i] + rests[i]);
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

// dst[0 .. min(*d_bytes, capacity)) = src[..]: the count is read on the device
__global__ __launch_bounds__(kBlock) void copy_counted_kernel(unsigned char* __restrict__ dst,
                                                              const unsigned char* __restrict__ src,
                                                              const int* __restrict__ d_bytes, long long capacity,
                                                              int words_ok) {
    long long bytes = *d_bytes;
    if (bytes < 0) bytes = 0;
    if (bytes > capacity) bytes = capacity;
    const long long stride = (long long)gridDim.x * kBlock;
    const long long first = (long long)blockIdx.x * kBlock + threadIdx.x;
    long long done = 0;
    if (words_ok) {  // both pointers 4-byte aligned
        const long long nwords = bytes / 4;
        for (long long i = first; i < nwords; i += stride)
            reinterpret_cast<unsigned*>(dst)[i] = reinterpret_cast<const unsigned*>(src)[i];
        done = nwords * 4;
    }
    for (long long i = done + first; i < bytes; i += stride) dst[i] = src[i];
}

int launch_copy_counted(cx_handle h, void* dst, const void* src, const int* d_bytes, long long capacity) {
    if (!dst || !src || !d_bytes || capacity < 0) return fail(CX_ERR_INVALID, "copy_counted: bad arguments");
    if (capacity == 0) return CX_OK;
    const int words_ok = ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 3u) == 0 ? 1 : 0;
    hipLaunchKernelGGL(copy_counted_kernel, dim3(grid_for(capacity / 4 + 1, 4)), dim3(kBlock), 0, h->stream,
                       static_cast<unsigned char*>(dst), static_cast<const unsigned char*>(src), d_bytes, capacity,
                       words_ok);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

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
    if (((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(rests)) & 15u) == 0) {
        const long long per_block = (long long)kBlock * kAddUnroll * kVec;
        hipLaunchKernelGGL((add_vec_kernel<T, kVec>), dim3((unsigned)(((long long)n + per_block - 1) / per_block)),
                           dim3(kBlock), 0, h->stream, data, rests, (long long)n);
    } else {
        const long long per_block = (long long)kBlock * kAddUnroll;
        hipLaunchKernelGGL((add_vec_kernel<T, 1>), dim3((unsigned)(((long long)n + per_block - 1) / per_block)),
                           dim3(kBlock), 0, h->stream, data, rests, (long long)n);
    }
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

template <typename T> int launch_sequential(cx_handle h, T* out, int out_n, const void* msg, int add) {
    if ((!out && out_n > 0) || !msg || out_n < 0) return fail(CX_ERR_INVALID, "decompress: bad arguments");
    if (!add) {
        int rc = launch_zero<T>(h, out, out_n);
        if (rc != CX_OK) return rc;
        hipLaunchKernelGGL((sequential_kernel<T, 0>), dim3(1), dim3(64), 0, h->stream, out, out_n,
                           static_cast<const unsigned*>(msg), h->d_status);
    } else {
        hipLaunchKernelGGL((sequential_kernel<T, 1>), dim3(1), dim3(64), 0, h->stream, out, out_n,
                           static_cast<const unsigned*>(msg), h->d_status);
    }
    CX_HIP(hipGetLastError());
    return CX_OK;
}

// add_strategy for a message in ANY index order without the host in between: the order check, the
// fast kernel (which does nothing when the check found disorder) and the pair-after-pair kernel (which
// does nothing otherwise) are enqueued one behind the other.
template <typename T> int launch_add_any_order(cx_handle h, T* out, int out_n, const void* msg) {
    if ((!out && out_n > 0) || !msg || out_n < 0) return fail(CX_ERR_INVALID, "add: bad arguments");
    if (out_n == 0) return check_headers(h, &msg, 1);
    unsigned* flag = reinterpret_cast<unsigned*>(h->d_status) + 16;
    const unsigned* words = static_cast<const unsigned*>(msg);
    MsgHeaders list;
    for (int r = 0; r < MsgHeaders::kMax; ++r) list.msg[r] = r == 0 ? words : nullptr;
    hipLaunchKernelGGL(order_check_kernel, dim3(256, 1), dim3(kBlock), 0, h->stream, list, flag, (int)Elem<T>::pair_words);
    hipLaunchKernelGGL((scatter_kernel<T, 1>), dim3(grid_for(out_n, 1)), dim3(kBlock), 0, h->stream, out, out_n, words,
                       h->d_status, flag);
    hipLaunchKernelGGL((sequential_kernel<T, 1>), dim3(1), dim3(64), 0, h->stream, out, out_n, words, h->d_status, flag);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

// decompression_strategy for a message in ANY index order without the host in between: order check, the
// tiled kernels (which do nothing when the check found disorder), then zero fill and the pair-after-pair
// kernel (which do nothing otherwise).
template <typename T> int launch_decompress_any_order(cx_handle h, T* out, int out_n, const void* msg) {
    if ((!out && out_n > 0) || !msg || out_n < 0) return fail(CX_ERR_INVALID, "decompress: bad arguments");
    if (out_n == 0) return check_headers(h, &msg, 1);
    unsigned* flag = reinterpret_cast<unsigned*>(h->d_status) + 16;
    const unsigned* words = static_cast<const unsigned*>(msg);
    MsgHeaders list;
    for (int r = 0; r < MsgHeaders::kMax; ++r) list.msg[r] = r == 0 ? words : nullptr;
    hipLaunchKernelGGL(order_check_kernel, dim3(256, 1), dim3(kBlock), 0, h->stream, list, flag, (int)Elem<T>::pair_words);
    int rc = launch_tiled<T>(h, out, out_n, &msg, 1, 0, 0, flag);
    if (rc != CX_OK) return rc;
    constexpr int kVec = 16 / (int)sizeof(T);
    if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0)
        hipLaunchKernelGGL((zero_kernel<T, kVec>), dim3(grid_for(out_n, 4 * kVec)), dim3(kBlock), 0, h->stream, out,
                           (long long)out_n, flag);
    else
        hipLaunchKernelGGL((zero_kernel<T, 1>), dim3(grid_for(out_n, 4)), dim3(kBlock), 0, h->stream, out, (long long)out_n, flag);
    hipLaunchKernelGGL((sequential_kernel<T, 0>), dim3(1), dim3(64), 0, h->stream, out, out_n, words, h->d_status, flag);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

// Are all the messages index-sorted?  One pass over their indices and one wait for the stream.
template <typename T>
int messages_sorted(cx_handle h, const void* const* msgs, int n_msgs, int* sorted, long long* total_pairs) {
    *sorted = 1;
    if (total_pairs) *total_pairs = 0;
    unsigned* flag = reinterpret_cast<unsigned*>(h->d_status) + 16;  // two words of the status block: flag, pair count
    for (int first = 0; first < n_msgs; first += MsgHeaders::kMax) {
        MsgHeaders list;
        const int cnt = n_msgs - first < MsgHeaders::kMax ? n_msgs - first : MsgHeaders::kMax;
        for (int r = 0; r < MsgHeaders::kMax; ++r)
            list.msg[r] = r < cnt ? static_cast<const unsigned*>(msgs[first + r]) : nullptr;
        hipLaunchKernelGGL(order_check_kernel, dim3(256, cnt), dim3(kBlock), 0, h->stream, list, flag,
                           (int)Elem<T>::pair_words);
    }
    CX_HIP(hipGetLastError());
    CX_HIP(hipMemcpyAsync(h->h_pinned + 13, flag, 2 * sizeof(unsigned), hipMemcpyDeviceToHost, h->stream));
    CX_HIP(hipStreamSynchronize(h->stream));
    if (h->h_pinned[13] != 0) *sorted = 0;
    if (total_pairs) *total_pairs = (long long)(unsigned)h->h_pinned[14];
    if (h->h_pinned[13] != 0 || h->h_pinned[14] != 0) CX_HIP(hipMemsetAsync(flag, 0, 2 * sizeof(unsigned), h->stream));
    return CX_OK;
}

template <typename T> int launch_add(cx_handle h, T* out, int out_n, const void* msg, int atomic) {
    if ((!out && out_n > 0) || !msg || out_n < 0) return fail(CX_ERR_INVALID, "add: bad arguments");
    if (out_n == 0) return check_headers(h, &msg, 1);
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
    if ((!out && out_n > 0) || !msg || out_n < 0) return fail(CX_ERR_INVALID, "decompress: bad arguments");
    if (out_n == 0) return check_headers(h, &msg, 1);
    // one message: short-lived blocks, one per tile, reach the vector's write rate; the pipelined
    // kernel (reduce_variant 3 forces it) pays off from two messages on
    if (h->reduce_variant == 0 || h->reduce_variant == 2) return launch_tiled<T>(h, out, out_n, &msg, 1, 0, 0);
    if (h->reduce_variant == 3) return launch_merged<T>(h, out, out_n, &msg, 1, 0, 0);
    int rc = launch_zero<T>(h, out, out_n);  // the whole output, also when the size check fails afterwards
    if (rc != CX_OK) return rc;
    hipLaunchKernelGGL((scatter_kernel<T, 0>), dim3(grid_for(out_n, 1)), dim3(kBlock), 0, h->stream, out, out_n,
                       static_cast<const unsigned*>(msg), h->d_status);
    CX_HIP(hipGetLastError());
    return CX_OK;
}

template <typename T>
int launch_reduce(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int accumulate, int mode) {
    if ((!out && out_n > 0) || out_n < 0 || n_msgs < 0 || (n_msgs > 0 && !msgs)) return fail(CX_ERR_INVALID, "reduce: bad arguments");
    if (out_n == 0) return check_headers(h, msgs, n_msgs);
    if (mode == 0 && h->reduce_variant == 3) return launch_merged<T>(h, out, out_n, msgs, n_msgs, 1, accumulate);
    if (mode == 0 && h->reduce_variant == 0) {
        // Measured on 64 Mi fp32 elements with 1 %-dense messages, 1 / 2 / 3 / 4 / 8 messages (events around
        // the call).  Writing the vector from zeros: pipelined 61 / 57 / 62 / 62 / 57 us against one block
        // per tile 45 / 50 / 61 / 66 / 91 us.  Adding into it: pipelined 94 / 100 / 96 / 97 / 94 us against
        // 87 / 94 / 105 / 114 / 146 us.  32 Mi fp64 elements: from zeros 58 / 57 / 59 / 55 / 63 us against
        // 43 / 49 / 56 / 62 / 96 us, adding 97 / 101 / 99 / 103 / 97 us against 86 / 95 / 105 / 114 / 155 us.
        // Later batches of 8 messages add.
        if (n_msgs > (accumulate ? 2 : 3)) return launch_merged<T>(h, out, out_n, msgs, n_msgs, 1, accumulate);
    }
    if (mode == 0 && (h->reduce_variant == 0 || h->reduce_variant == 2))
        return launch_tiled<T>(h, out, out_n, msgs, n_msgs, 1, accumulate);
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

template <typename T> int reserve_reduce(cx_handle h, int n) {
    constexpr int kReduceTile = ReduceTile<T>::value;
    const size_t ntiles = (size_t)(((long long)n + kReduceTile - 1) / kReduceTile);
    return ensure_bounds(h, (size_t)kMaxMsgs * (ntiles + 1));
}
template int reserve_reduce<float>(cx_handle, int);
template int reserve_reduce<double>(cx_handle, int);
template int reserve_reduce<int>(cx_handle, int);

#define CX_INSTANTIATE(T)                                                                         \
    template int launch_zero<T>(cx_handle, T*, int);                                              \
    template int launch_add_vec<T>(cx_handle, T*, const T*, int);                                 \
    template int launch_threshold_apply<T>(cx_handle, T*, T*, const T*, int, const T*, const T*); \
    template int launch_add<T>(cx_handle, T*, int, const void*, int);                             \
    template int launch_sequential<T>(cx_handle, T*, int, const void*, int);                      \
    template int messages_sorted<T>(cx_handle, const void* const*, int, int*, long long*);     \
    template int launch_add_any_order<T>(cx_handle, T*, int, const void*);                        \
    template int launch_decompress_any_order<T>(cx_handle, T*, int, const void*);                    \
    template int launch_decompress<T>(cx_handle, T*, int, const void*);                           \
    template int launch_reduce<T>(cx_handle, T*, int, const void* const*, int, int, int);
CX_INSTANTIATE(float)
CX_INSTANTIATE(double)
CX_INSTANTIATE(int)

}  // namespace cx
