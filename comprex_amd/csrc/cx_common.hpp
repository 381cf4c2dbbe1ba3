// Shared host-side declarations of the gfx950 library: handle layout, error plumbing,
// element-type traits.  Device code lives in the k_*.hip files.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>

#include "../../include/comprex_gfx950.h"

namespace cx {

// ---- error plumbing --------------------------------------------------------
std::string& last_error();
int fail(int code, const char* fmt, ...);

#define CX_HIP(call)                                                                         \
    do {                                                                                     \
        hipError_t e__ = (call);                                                             \
        if (e__ != hipSuccess)                                                               \
            return ::cx::fail(CX_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e__), \
                              __FILE__, __LINE__);                                           \
    } while (0)

// ---- per-element-type traits -----------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<float> {
    using key_t = uint32_t;
    static constexpr int key_bits = 31;  // sign stripped
    static constexpr int pair_words = 2;
};
template <> struct Elem<int> {
    using key_t = uint32_t;
    static constexpr int key_bits = 32;  // |INT_MIN| needs bit 31
    static constexpr int pair_words = 2;
};
template <> struct Elem<double> {
    using key_t = uint64_t;
    static constexpr int key_bits = 63;
    static constexpr int pair_words = 3;
};

// ---- device-side scratch layouts -------------------------------------------
constexpr int kRadixBits = 11;
constexpr int kRadixBins = 1 << kRadixBits;

// What is fixed of the wanted key after some passes.
struct PickState {
    unsigned long long prefix;     // key bits fixed so far
    unsigned long long mask;       // which bits of `prefix` are fixed
    unsigned long long rank;       // descending rank still to find among matching keys
};
constexpr int kMaxRadixPasses = 6; // 63-bit keys, 11 bits per pass

// State of one radix-select run; lives in device memory.
struct SelectState {
    unsigned int hist[kRadixBins]; // two-launch select: top-digit counts of all keys; zero between runs
    unsigned int short_count;      // two-launch select: keys in the short list; zero between runs
    unsigned int short_digit;      // ... and the largest cut of a block: the leading two digits of its short_k-th key
    // chained passes (no pick launch in between): one histogram per pass, all zero between runs,
    // and the state entering each pass.  The slot behind a key type's last pass holds the top-digit
    // counts of a candidate list, made by the kernel that collects the list.
    unsigned int pass_hist[kMaxRadixPasses + 1][kRadixBins];
    PickState pass_state[kMaxRadixPasses];
};

// Device status: `code` = the first error a kernel recorded (first wins); bit 0 of `detail` = a
// compressed message was cut short for lack of room (not an error of the message: see collect_status).
struct DeviceStatus {
    int code;
    int detail;
};

}  // namespace cx

// The handle: stream + scratch of one compressor clone.
struct cx_handle_s {
    int device = 0;
    hipStream_t stream = nullptr;

    // compaction scratch: per-tile staging slots, counts and final offsets
    unsigned* staging = nullptr;
    size_t staging_cap = 0;            // 32-bit words allocated
    unsigned* tile_counts = nullptr;
    unsigned* tile_offsets = nullptr;
    unsigned* block_sums = nullptr;    // survivors per streaming block
    size_t tiles_cap = 0;              // tiles allocated
    unsigned* redo_flag = nullptr;     // holds the launch number of the last launch that deferred a tile
    unsigned epoch = 0;                // launch number
    unsigned parity = 0;               // flips with every full pass over the vectors: 1 = the next one walks from the end

    unsigned* static_scratch = nullptr; // this device's copy of the library's static scratch array (not owned)

    unsigned* reduce_bounds = nullptr;  // tiled reduce: first pair of each message in each dense tile
    size_t reduce_bounds_cap = 0;

    cx::SelectState* sel = nullptr;
    void* cand = nullptr;              // candidates of the one-pass whole-vector select (keys) / fused top-k (pairs)
    size_t cand_bytes = 0;
    void* sel_keys = nullptr;          // gathered sample keys of the two-launch select
    size_t sel_keys_bytes = 0;
    void* rle_pairs = nullptr;         // run-length codec: the (index, value) pairs its compress starts from
    size_t rle_pairs_bytes = 0;
    unsigned* rle_scan = nullptr;      // run-length codec: per-block counts / prefix sums over the runs
    size_t rle_scan_bytes = 0;
    cx::DeviceStatus* d_status = nullptr;
    void* d_thr = nullptr;             // 256 bytes: threshold slot at 0, sampled lower bound at 64,
                                       // small result words at 128, a codec's derived threshold at 192
    int* h_pinned = nullptr;           // 64-byte pinned read-back area

    // optional timing of the streaming pass: HIP events recorded around stage_kernel
    static constexpr int kProfileRing = 1024;
    int profile = 0;                   // N > 0: events around every N-th streaming launch
    unsigned profile_tick = 0;
    int profile_count = 0;             // launches recorded since the last read
    hipEvent_t* profile_events = nullptr;  // 2 * kProfileRing events, created on first use

    // options
    int compact_items = 0;             // 16-byte loads per lane and tile: 2, 4, 8, or 0 = by the vector's length
    int stage_alternate = 1;           // 1 = every other launch walks the tiles from the end
    int stage_cached_tail_mb = 192;    // residual read cacheably over the last so many MB of a walk (-1: all of it)
    int select_bracket = 1;            // 1 = one-pass whole-vector select with a sampled lower bound
    int select_short_list = 1;         // 1 = the two-launch select passes a short list of top keys to its second launch
    int fused_topk = 1;                // cx_ip_compress_topk's single-pass route: 0 never, 1 from 20 Mi elements, 2 from 2^23
    int fused_topk_taken = 0;          // how the last cx_ip_compress_topk ran: 0 two calls, 1 single pass, 2 single pass abandoned
    // A chained whole-vector selection whose last pick is left to the compress pass that follows it
    // (launch_compress_topk asks for this with defer_pick): that pass's blocks pick from the last
    // histogram themselves, which spares the launch of a one-block kernel.
    bool defer_pick = false;
    struct {
        bool active = false;
        unsigned long long rank = 0;
        int plus_one = 0;
        void* thr_out = nullptr;
    } pending_pick;
    int reduce_variant = 0;            // 0 = rank-ordered, kernel chosen by message count; 1 = per-message scatter;
                                       // 2 = always one block per tile behind a bounds pass; 3 = always the pipelined kernel
    int reduce_blocks_per_cu = 1;      // persistent blocks per compute unit of the merged reduce
    int cu_count = 0;                  // compute units of the device
};

namespace cx {

// sample_mode of launch_topk_threshold
enum { kSampleFull = 0, kSampleStrided = 1, kSampleIndexed = 2 };

// ---- launchers implemented in the k_*.hip files -----------------------------
template <typename T>
int launch_compact(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                   const T* thr_host, const T* d_thr, int* d_size_prefix, bool no_alloc = false);
// allocation-free variant: this device's copy of the static scratch array, and its size limit
int locate_static_scratch(unsigned** out);
// Pre-size a module's scratch for vectors of up to n elements of T, so that later calls find it large enough.
template <typename T> int reserve_compact(cx_handle h, int n);
template <typename T> int reserve_select(cx_handle h, int n);
// makes the pick a selection left pending (handle's pending_pick) with a launch of its own
template <typename T> int launch_pending_pick(cx_handle h);
template <typename T> int reserve_reduce(cx_handle h, int n);
template <typename T> int reserve_rle(cx_handle h, int n);
long long noalloc_max_elements();

template <typename T>
int launch_topk_threshold(cx_handle h, const T* vec, const T* add_vec, int n, const int* d_idx, int m,
                          int sample_mode, float stepsize, float topK, T* d_thr_out);

// fused exact top-k (whole-vector ThresholdTopK + compress_add_update in one pass over the vectors)
template <typename T>
int launch_candidates(cx_handle h, unsigned* cand_words, long long cap_pairs, const T* data, T* update, int n,
                      const T* d_bound);
template <typename T>
int launch_filter(cx_handle h, const unsigned* cand_words, unsigned cand_cap, unsigned long long rank, T* d_thr,
                  T* update, int n, unsigned* msg_words, long long cap_pairs, int* size_prefix, unsigned* d_result,
                  unsigned long long expected_candidates);
template <typename T>
int launch_compress_topk(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                         float topK, T* d_thr_out, int* d_size_prefix);

// run-length codec
template <typename T>
int launch_rle_compress(cx_handle h, void* out_msg, long long out_capacity, const T* data, T* update, int n,
                        const T* thr_host, const T* d_thr, int* d_size_prefix, int* d_result);
template <typename T> int launch_rle_decode(cx_handle h, T* out, int out_n, const void* msg, int add, int* n_out);

template <typename T> int launch_decompress(cx_handle h, T* out, int out_n, const void* msg);
template <typename T> int launch_add(cx_handle h, T* out, int out_n, const void* msg, int atomic);
template <typename T> int launch_add_any_order(cx_handle h, T* out, int out_n, const void* msg);
template <typename T> int launch_decompress_any_order(cx_handle h, T* out, int out_n, const void* msg);
// the reference's loop, pair after pair: any index order, indices repeated anywhere (slow)
template <typename T> int launch_sequential(cx_handle h, T* out, int out_n, const void* msg, int add);
// one pass over the messages' indices and one wait: *sorted = every message's indices ascend
template <typename T>
int messages_sorted(cx_handle h, const void* const* msgs, int n_msgs, int* sorted, long long* total_pairs = nullptr);
template <typename T>
int launch_reduce(cx_handle h, T* out, int out_n, const void* const* msgs, int n_msgs, int accumulate, int mode);
int launch_copy_counted(cx_handle h, void* dst, const void* src, const int* d_bytes, long long capacity);
template <typename T> int launch_zero(cx_handle h, T* v, int n);
template <typename T> int launch_add_vec(cx_handle h, T* data, const T* rests, int n);
template <typename T>
int launch_threshold_apply(cx_handle h, T* high, T* low, const T* in, int n, const T* thr_host, const T* d_thr);

}  // namespace cx
