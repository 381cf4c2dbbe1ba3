// extern "C" kernel-level boundary (cx_*): argument checks, element-type dispatch, handle
// life cycle.  Declarations and the reference interfaces they replace: include/comprex_gfx950.h.
#include "cx_common.hpp"

#include <cmath>

namespace cx {

std::string& last_error() {
    static thread_local std::string msg;
    return msg;
}

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    last_error() = buf;
    return code;
}

namespace {

const char* status_text(int code) {
    switch (code) {
        case CX_ERR_MSG_TOO_LARGE: return "Decompression vector size is bigger than output buffer!";
        case CX_ERR_CAPACITY: return "compressed message does not fit the buffer it was given";
        case CX_ERR_INDEX: return "a message index lies outside the output vector";
        case CX_ERR_INTERNAL: return "a bounded device-side wait expired";
        default: return "device-side error";
    }
}

// Reads and clears the device status; waits for the stream.  `code` holds the first error a kernel
// recorded; a message cut short for lack of room is noted apart from it (bit 0 of `detail`: the
// message is valid and error feedback sends the rest later), so that it neither hides a real
// error nor is hidden by one: a real error is reported first, the note with the next call.
int collect_status(cx_handle h) {
    CX_HIP(hipMemcpyAsync(h->h_pinned, h->d_status, sizeof(DeviceStatus), hipMemcpyDeviceToHost, h->stream));
    CX_HIP(hipStreamSynchronize(h->stream));
    const int code = h->h_pinned[0], cut_short = h->h_pinned[1] & 1;
    if (code != 0) {
        CX_HIP(hipMemsetAsync(&h->d_status->code, 0, sizeof(int), h->stream));
        CX_HIP(hipStreamSynchronize(h->stream));
        return fail(code, "%s", status_text(code));
    }
    if (cut_short) {
        CX_HIP(hipMemsetAsync(&h->d_status->detail, 0, sizeof(int), h->stream));
        CX_HIP(hipStreamSynchronize(h->stream));
        return fail(CX_ERR_CAPACITY, "%s", status_text(CX_ERR_CAPACITY));
    }
    return CX_OK;
}

bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

}  // namespace
}  // namespace cx

using namespace cx;

namespace {

template <typename T>
int finish_threshold(cx_handle h, T* d_thr_out, void* h_thr_out) {
    if (!h_thr_out) return CX_OK;
    const T* src = d_thr_out ? d_thr_out : static_cast<const T*>(h->d_thr);
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, src, sizeof(T), hipMemcpyDeviceToHost, h->stream));
    int rc = collect_status(h);
    memcpy(h_thr_out, h->h_pinned + 8, sizeof(T));
    return rc;
}

template <typename T>
int topk_threshold_impl(cx_handle h, const void* vec, const void* add_vec, int n, int add_n, float topK,
                        int default_subsamples, float subsample_factor, void* d_thr_out, void* h_thr_out) {
    if (add_vec && n != add_n) return fail(CX_ERR_SIZE_MISMATCH, "vector sizes must be the same!");
    int subsamples = cx_topk_subsamples(topK, default_subsamples, subsample_factor);
    if (subsamples < 0) subsamples = 0x7fffffff;  // undefined in the reference: use the whole vector
    int rc;
    if (n < subsamples) {
        rc = launch_topk_threshold<T>(h, static_cast<const T*>(vec), static_cast<const T*>(add_vec), n, nullptr, n,
                                      kSampleFull, 1.0f, topK, static_cast<T*>(d_thr_out));
    } else {
        const float stepsize = (float)n / (float)subsamples;
        rc = launch_topk_threshold<T>(h, static_cast<const T*>(vec), static_cast<const T*>(add_vec), n, nullptr,
                                      subsamples, kSampleStrided, stepsize, topK, static_cast<T*>(d_thr_out));
    }
    if (rc != CX_OK) return rc;
    return finish_threshold<T>(h, static_cast<T*>(d_thr_out), h_thr_out);
}

template <typename T>
int topk_threshold_indexed_impl(cx_handle h, const void* vec, const void* add_vec, int n, const int* d_idx, int m,
                                float topK, void* d_thr_out, void* h_thr_out) {
    int rc = launch_topk_threshold<T>(h, static_cast<const T*>(vec), static_cast<const T*>(add_vec), n, d_idx, m,
                                      kSampleIndexed, 1.0f, topK, static_cast<T*>(d_thr_out));
    if (rc != CX_OK) return rc;
    return finish_threshold<T>(h, static_cast<T*>(d_thr_out), h_thr_out);
}

template <typename T>
int compress_impl(cx_handle h, void* out_msg, long long out_capacity, const void* data, void* update, int n,
                  const void* thr_host, const void* d_thr, int* d_size_prefix, int* h_bytes) {
    int rc = launch_compact<T>(h, out_msg, out_capacity, static_cast<const T*>(data), static_cast<T*>(update), n,
                               static_cast<const T*>(thr_host), static_cast<const T*>(d_thr), d_size_prefix);
    if (rc != CX_OK || !h_bytes) return rc;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, out_msg, 8, hipMemcpyDeviceToHost, h->stream));
    rc = collect_status(h);
    const int k = h->h_pinned[9];
    *h_bytes = 8 + k * 4 * Elem<T>::pair_words;
    return rc;
}

template <typename T>
int compress_topk_impl(cx_handle h, void* out_msg, long long out_capacity, const void* data, void* update, int n,
                       float topK, void* d_thr_out, int* d_size_prefix, int* h_bytes) {
    int rc = launch_compress_topk<T>(h, out_msg, out_capacity, static_cast<const T*>(data), static_cast<T*>(update), n,
                                     topK, static_cast<T*>(d_thr_out), d_size_prefix);
    if (rc != CX_OK || !h_bytes) return rc;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, out_msg, 8, hipMemcpyDeviceToHost, h->stream));
    rc = collect_status(h);
    *h_bytes = 8 + h->h_pinned[9] * 4 * Elem<T>::pair_words;
    return rc;
}

// ThresholdTopK::prepare_with + compress_add_update in one call
template <typename T>
int write_step_impl(cx_handle h, void* out_msg, long long out_capacity, const void* data, void* update, int n, float topK,
                    int default_subsamples, float subsample_factor, const int* d_idx, int m, void* d_thr_out,
                    int* d_size_prefix, int* h_bytes) {
    const T* d = static_cast<const T*>(data);
    T* u = static_cast<T*>(update);
    T* thr = static_cast<T*>(d_thr_out);
    int mode, keys;
    float stepsize = 1.0f;
    if (d_idx && m > 0) {
        mode = kSampleIndexed;
        keys = m;
    } else {
        int subsamples = cx_topk_subsamples(topK, default_subsamples, subsample_factor);
        if (subsamples < 0) subsamples = 0x7fffffff;  // undefined in the reference: use the whole vector
        if (n < subsamples) {
            mode = kSampleFull;
            keys = n;
        } else {
            mode = kSampleStrided;
            keys = subsamples;
            stepsize = (float)n / (float)subsamples;
        }
    }
    int rc;
    if (mode == kSampleFull) {
        rc = launch_compress_topk<T>(h, out_msg, out_capacity, d, u, n, topK, thr, d_size_prefix);
    } else {
        rc = launch_topk_threshold<T>(h, u, d, n, d_idx, keys, mode, stepsize, topK, thr);
        if (rc == CX_OK) rc = launch_compact<T>(h, out_msg, out_capacity, d, u, n, nullptr, thr, d_size_prefix);
    }
    if (rc != CX_OK || !h_bytes) return rc;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, out_msg, 8, hipMemcpyDeviceToHost, h->stream));
    rc = collect_status(h);
    *h_bytes = 8 + h->h_pinned[9] * 4 * Elem<T>::pair_words;
    return rc;
}

template <typename T>
int rle_compress_impl(cx_handle h, void* out_msg, long long out_capacity, const void* data, void* update, int n,
                      const void* thr_host, const void* d_thr, int* d_size_prefix, int* h_bytes) {
    int* d_result = reinterpret_cast<int*>(static_cast<char*>(h->d_thr) + 128);
    int rc = launch_rle_compress<T>(h, out_msg, out_capacity, static_cast<const T*>(data), static_cast<T*>(update), n,
                                    static_cast<const T*>(thr_host), static_cast<const T*>(d_thr), d_size_prefix,
                                    d_result);
    if (rc != CX_OK || !h_bytes) return rc;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, d_result, 4, hipMemcpyDeviceToHost, h->stream));
    rc = collect_status(h);
    *h_bytes = h->h_pinned[8];
    return rc;
}

template <typename T>
int decompress_impl(cx_handle h, void* out, int out_n, const void* msg, int* h_bytes) {
    if (h_bytes && (h->reduce_variant == 0 || h->reduce_variant == 2)) {
        // the reporting form takes any index order, as the reference does (src/compressor.hxx:613-633):
        // decided on the device, one wait at the end
        int rc_any = launch_decompress_any_order<T>(h, static_cast<T*>(out), out_n, msg);
        if (rc_any != CX_OK) return rc_any;
        CX_HIP(hipMemcpyAsync(h->h_pinned + 8, msg, 8, hipMemcpyDeviceToHost, h->stream));
        rc_any = collect_status(h);
        *h_bytes = 8 + h->h_pinned[9] * 4 * Elem<T>::pair_words;
        return rc_any;
    }
    if (h_bytes) {
        // what earlier calls left behind is reported now, so that the status read below belongs to
        // this message alone (a message cut short by an earlier compress is not this call's business)
        const int pending = collect_status(h);
        if (pending != CX_OK && pending != CX_ERR_CAPACITY) return pending;
    }
    int rc = launch_decompress<T>(h, static_cast<T*>(out), out_n, msg);
    if (rc != CX_OK || !h_bytes) return rc;
    CX_HIP(hipMemcpyAsync(h->h_pinned + 8, msg, 8, hipMemcpyDeviceToHost, h->stream));
    rc = collect_status(h);
    if (rc == CX_ERR_INDEX) {
        // the fast path wants ascending indices; the reference takes any order (src/compressor.hxx:613-633):
        // once more, pair after pair.  An index outside the vector is reported again.
        rc = launch_sequential<T>(h, static_cast<T*>(out), out_n, msg, 0);
        if (rc != CX_OK) return rc;
        rc = collect_status(h);
    }
    *h_bytes = 8 + h->h_pinned[9] * 4 * Elem<T>::pair_words;
    return rc;
}

}  // namespace

namespace {
template <typename T> int reserve_impl(cx_handle h, int n, unsigned paths) {
    int rc = CX_OK;
    if (rc == CX_OK && (paths & CX_RESERVE_COMPRESS)) rc = reserve_compact<T>(h, n);
    if (rc == CX_OK && (paths & CX_RESERVE_THRESHOLD)) rc = reserve_select<T>(h, n);
    if (rc == CX_OK && (paths & CX_RESERVE_REDUCE)) rc = reserve_reduce<T>(h, n);
    if (rc == CX_OK && (paths & CX_RESERVE_RLE)) rc = reserve_rle<T>(h, n);
    return rc;
}
}  // namespace


extern "C" {

const char* cx_last_error(void) { return last_error().c_str(); }

int cx_abi_version(void) { return 1; }

int cx_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int cx_pointer_on_device(const void* p) {
    if (!p) return 0;
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();  // pageable host memory is reported as an error
        return 0;
    }
    return (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged ||
            attr.type == hipMemoryTypeHost)
               ? 1
               : 0;
}

int cx_device_alloc(void** out, size_t bytes) {
    if (!out) return fail(CX_ERR_INVALID, "cx_device_alloc: null output");
    *out = nullptr;
    if (bytes == 0) return CX_OK;
    CX_HIP(hipMalloc(out, bytes));
    return CX_OK;
}

int cx_device_free(void* p) {
    if (p) CX_HIP(hipFree(p));
    return CX_OK;
}

int cx_copy(cx_handle h, void* dst, const void* src, size_t bytes) {
    if (!h || ((!dst || !src) && bytes > 0)) return fail(CX_ERR_INVALID, "cx_copy: bad arguments");
    if (bytes == 0) return CX_OK;
    CX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, h->stream));
    // a pageable host buffer may be reused by the caller right away
    if (!cx_pointer_on_device(dst) || !cx_pointer_on_device(src)) CX_HIP(hipStreamSynchronize(h->stream));
    return CX_OK;
}

int cx_copy_counted(cx_handle h, void* dst, const void* src, const int* d_bytes, long long capacity) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    return launch_copy_counted(h, dst, src, d_bytes, capacity);
}

int cx_create(cx_handle* out, void* hip_stream) {
    if (!out) return fail(CX_ERR_INVALID, "cx_create: null output");
    *out = nullptr;
    if (cx_device_count() < 1) return fail(CX_ERR_HIP, "cx_create: no HIP device available");
    cx_handle h = new cx_handle_s();
    h->stream = static_cast<hipStream_t>(hip_stream);
    hipError_t e = hipGetDevice(&h->device);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&h->cu_count, hipDeviceAttributeMultiprocessorCount, h->device);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&h->redo_flag), 256);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&h->sel), sizeof(SelectState));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&h->d_status), 256);
    if (e == hipSuccess) e = hipMalloc(&h->d_thr, 256);
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void**>(&h->h_pinned), 64, hipHostMallocDefault);
    // cleared ON THE HANDLE'S STREAM and waited for: a plain hipMemset runs on the null stream, with
    // which a non-blocking stream is not ordered, so a first kernel could see (or a late memset wipe)
    // the state of whoever held this memory before
    if (e == hipSuccess) e = hipMemsetAsync(h->redo_flag, 0, 256, h->stream);
    if (e == hipSuccess) e = hipMemsetAsync(h->sel, 0, sizeof(SelectState), h->stream);
    if (e == hipSuccess) e = hipMemsetAsync(h->d_status, 0, 256, h->stream);
    if (e == hipSuccess) e = hipMemsetAsync(h->d_thr, 0, 256, h->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(h->stream);
    if (e != hipSuccess) {
        cx_destroy(h);
        return fail(CX_ERR_HIP, "cx_create: %s", hipGetErrorString(e));
    }
    // where this device keeps the static scratch array of cx_ip_compress_noalloc
    const int rc = locate_static_scratch(&h->static_scratch);
    if (rc != CX_OK) {
        cx_destroy(h);
        return rc;
    }
    *out = h;
    return CX_OK;
}

int cx_destroy(cx_handle h) {
    if (!h) return CX_OK;
    (void)hipStreamSynchronize(h->stream);
    if (h->staging) (void)hipFree(h->staging);
    if (h->tile_counts) (void)hipFree(h->tile_counts);
    if (h->tile_offsets) (void)hipFree(h->tile_offsets);
    if (h->block_sums) (void)hipFree(h->block_sums);
    if (h->redo_flag) (void)hipFree(h->redo_flag);
    if (h->reduce_bounds) (void)hipFree(h->reduce_bounds);
    if (h->sel) (void)hipFree(h->sel);
    if (h->sel_keys) (void)hipFree(h->sel_keys);
    if (h->cand) (void)hipFree(h->cand);
    if (h->rle_pairs) (void)hipFree(h->rle_pairs);
    if (h->rle_scan) (void)hipFree(h->rle_scan);
    if (h->d_status) (void)hipFree(h->d_status);
    if (h->d_thr) (void)hipFree(h->d_thr);
    if (h->h_pinned) (void)hipHostFree(h->h_pinned);
    if (h->profile_events) {
        for (int i = 0; i < 2 * cx_handle_s::kProfileRing; ++i) (void)hipEventDestroy(h->profile_events[i]);
        delete[] h->profile_events;
    }
    delete h;
    return CX_OK;
}

int cx_set_stream(cx_handle h, void* hip_stream) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (h->stream != static_cast<hipStream_t>(hip_stream)) {
        CX_HIP(hipStreamSynchronize(h->stream));  // scratch is shared between launches of one handle
        h->stream = static_cast<hipStream_t>(hip_stream);
    }
    return CX_OK;
}

void* cx_get_stream(cx_handle h) { return h ? static_cast<void*>(h->stream) : nullptr; }

int cx_stream_create(void** out_stream) {
    if (!out_stream) return fail(CX_ERR_INVALID, "cx_stream_create: null output");
    *out_stream = nullptr;
    if (cx_device_count() < 1) return fail(CX_ERR_HIP, "cx_stream_create: no HIP device available");
    hipStream_t s = nullptr;
    CX_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *out_stream = static_cast<void*>(s);
    return CX_OK;
}

int cx_stream_create_blocking(void** out_stream) {
    if (!out_stream) return fail(CX_ERR_INVALID, "cx_stream_create_blocking: null output");
    *out_stream = nullptr;
    if (cx_device_count() < 1) return fail(CX_ERR_HIP, "cx_stream_create_blocking: no HIP device available");
    hipStream_t s = nullptr;
    CX_HIP(hipStreamCreateWithFlags(&s, hipStreamDefault));  // default priority
    *out_stream = static_cast<void*>(s);
    return CX_OK;
}

int cx_stream_destroy(void* hip_stream) {
    if (hip_stream) CX_HIP(hipStreamDestroy(static_cast<hipStream_t>(hip_stream)));
    return CX_OK;
}

int cx_stream_synchronize(void* hip_stream) {
    CX_HIP(hipStreamSynchronize(static_cast<hipStream_t>(hip_stream)));
    return CX_OK;
}

int cx_event_create(void** out_event) {
    if (!out_event) return fail(CX_ERR_INVALID, "cx_event_create: null output");
    *out_event = nullptr;
    hipEvent_t e = nullptr;
    CX_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    *out_event = static_cast<void*>(e);
    return CX_OK;
}

int cx_event_destroy(void* hip_event) {
    if (hip_event) CX_HIP(hipEventDestroy(static_cast<hipEvent_t>(hip_event)));
    return CX_OK;
}

int cx_event_record(void* hip_event, void* hip_stream) {
    if (!hip_event) return fail(CX_ERR_INVALID, "cx_event_record: null event");
    CX_HIP(hipEventRecord(static_cast<hipEvent_t>(hip_event), static_cast<hipStream_t>(hip_stream)));
    return CX_OK;
}

int cx_stream_wait_event(void* hip_stream, void* hip_event) {
    if (!hip_event) return fail(CX_ERR_INVALID, "cx_stream_wait_event: null event");
    CX_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(hip_stream), static_cast<hipEvent_t>(hip_event), 0));
    return CX_OK;
}

int cx_synchronize(cx_handle h) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    return collect_status(h);
}

int cx_set_option(cx_handle h, const char* key, int value) {
    if (!h || !key) return fail(CX_ERR_INVALID, "null handle or key");
    if (!strcmp(key, "compact_items")) {
        if (value != 0 && value != 2 && value != 4 && value != 8) return fail(CX_ERR_INVALID, "compact_items must be 0 (by length), 2, 4 or 8");
        h->compact_items = value;
    } else if (!strcmp(key, "profile_stage")) {
        if (value && !h->profile_events) {
            h->profile_events = new hipEvent_t[2 * cx_handle_s::kProfileRing];
            for (int i = 0; i < 2 * cx_handle_s::kProfileRing; ++i) CX_HIP(hipEventCreate(&h->profile_events[i]));
        }
        h->profile = value > 0 ? value : 0;
        h->profile_count = 0;
        h->profile_tick = 0;
    } else if (!strcmp(key, "stage_alternate")) {
        h->stage_alternate = value ? 1 : 0;
    } else if (!strcmp(key, "stage_cached_tail_mb")) {
        h->stage_cached_tail_mb = value < 0 ? -1 : value;
    } else if (!strcmp(key, "select_bracket")) {
        h->select_bracket = value ? 1 : 0;
    } else if (!strcmp(key, "reduce_variant")) {
        h->reduce_variant = value;
    } else if (!strcmp(key, "reduce_blocks_per_cu")) {
        if (value < 1 || value > 32) return fail(CX_ERR_INVALID, "reduce_blocks_per_cu must be 1..32");
        h->reduce_blocks_per_cu = value;
    } else if (!strcmp(key, "fused_topk")) {
        h->fused_topk = value < 0 ? 0 : (value > 2 ? 2 : value);  // 2: from 2^23 elements on, whatever is faster
    } else if (!strcmp(key, "select_short_list")) {
        h->select_short_list = value ? 1 : 0;

    } else {
        return fail(CX_ERR_INVALID, "unknown option '%s'", key);
    }
    return CX_OK;
}

int cx_get_option(cx_handle h, const char* key, int* value) {
    if (!h || !key || !value) return fail(CX_ERR_INVALID, "null handle, key or output");
    if (!strcmp(key, "compact_items")) *value = h->compact_items;
    else if (!strcmp(key, "profile_stage")) *value = h->profile;
    else if (!strcmp(key, "stage_alternate")) *value = h->stage_alternate;
    else if (!strcmp(key, "stage_cached_tail_mb")) *value = h->stage_cached_tail_mb;
    else if (!strcmp(key, "select_bracket")) *value = h->select_bracket;
    else if (!strcmp(key, "reduce_variant")) *value = h->reduce_variant;
    else if (!strcmp(key, "reduce_blocks_per_cu")) *value = h->reduce_blocks_per_cu;
    else if (!strcmp(key, "fused_topk")) *value = h->fused_topk;
    else if (!strcmp(key, "select_short_list")) *value = h->select_short_list;
    else if (!strcmp(key, "fused_topk_taken")) *value = h->fused_topk_taken;
    else return fail(CX_ERR_INVALID, "unknown option '%s'", key);
    return CX_OK;
}

int cx_profile_read(cx_handle h, float* ms_out, int max_out, int* n_out) {
    if (!h || !n_out || (max_out > 0 && !ms_out)) return fail(CX_ERR_INVALID, "cx_profile_read: bad arguments");
    *n_out = 0;
    CX_HIP(hipStreamSynchronize(h->stream));
    const int n = h->profile_count < max_out ? h->profile_count : max_out;
    for (int i = 0; i < n; ++i)
        CX_HIP(hipEventElapsedTime(&ms_out[i], h->profile_events[2 * i], h->profile_events[2 * i + 1]));
    *n_out = n;
    h->profile_count = 0;
    return CX_OK;
}

void* cx_threshold_slot(cx_handle h) { return h ? h->d_thr : nullptr; }

// ---- host arithmetic of ThresholdTopK (must reproduce the reference's fp32 steps) ----

int cx_topk_subsamples(float topK, int default_subsamples, float subsample_factor) {
    // `cond ? float : int` has type float: default_subsamples is rounded to fp32 first
    const float req = subsample_factor / topK;
    const float chosen = (req > (float)default_subsamples) ? req : (float)default_subsamples;
    if (!(chosen < 2147483648.0f) || !(chosen > -2147483904.0f)) return -1;
    return (int)chosen;
}

int cx_topk_pos(size_t m, float topK) {
    const float prod = (float)m * topK;
    const float up = std::ceil(prod);
    const float minus = up - 1.0f;
    return (int)minus;
}

#define CX_DISPATCH(dt, CALL)                                          \
    switch (dt) {                                                      \
        case CX_F32: { using T = float; return CALL; }                 \
        case CX_F64: { using T = double; return CALL; }                \
        case CX_I32: { using T = int; return CALL; }                   \
        default: return fail(CX_ERR_INVALID, "unknown element type %d", (int)dt); \
    }

// as CX_DISPATCH, but goes on when the call succeeds
#define CX_DISPATCH_RC(dt, CALL)                                                   \
    do {                                                                           \
        int rc__;                                                                  \
        switch (dt) {                                                              \
            case CX_F32: { using T = float; rc__ = CALL; break; }                  \
            case CX_F64: { using T = double; rc__ = CALL; break; }                 \
            case CX_I32: { using T = int; rc__ = CALL; break; }                    \
            default: return fail(CX_ERR_INVALID, "unknown element type %d", (int)dt); \
        }                                                                          \
        if (rc__ != CX_OK) return rc__;                                            \
    } while (0)

int cx_topk_threshold(cx_handle h, cx_dtype dt, const void* vec, const void* add_vec, int n, int add_n, float topK,
                      int default_subsamples, float subsample_factor, void* d_thr_out, void* h_thr_out) {
    if (!h || n < 0 || (!vec && n > 0)) return fail(CX_ERR_INVALID, "topk_threshold: bad arguments");
    if (topK > 1.0f || topK < 0.0f) return fail(CX_ERR_TOPK, "topK value must be between 0.0 and 1.0!");
    CX_DISPATCH(dt, topk_threshold_impl<T>(h, vec, add_vec, n, add_n, topK, default_subsamples, subsample_factor,
                                           d_thr_out, h_thr_out));
}

int cx_topk_threshold_indexed(cx_handle h, cx_dtype dt, const void* vec, const void* add_vec, int n, const int* d_idx,
                              int m, float topK, void* d_thr_out, void* h_thr_out) {
    if (!h || n < 0 || m < 0 || (!vec && n > 0) || (!d_idx && m > 0))
        return fail(CX_ERR_INVALID, "topk_threshold_indexed: bad arguments");
    if (topK > 1.0f || topK < 0.0f) return fail(CX_ERR_TOPK, "topK value must be between 0.0 and 1.0!");
    CX_DISPATCH(dt, topk_threshold_indexed_impl<T>(h, vec, add_vec, n, d_idx, m, topK, d_thr_out, h_thr_out));
}

int cx_ip_compress(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity, const void* data, void* update,
                   int n, const void* thr_host, const void* d_thr, int* d_size_prefix, int* h_bytes) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    CX_DISPATCH(dt, compress_impl<T>(h, out_msg, out_capacity, data, update, n, thr_host, d_thr, d_size_prefix, h_bytes));
}

int cx_ip_compress_noalloc(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity, const void* data,
                           void* update, int n, const void* thr_host, const void* d_thr, int* d_size_prefix) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    CX_DISPATCH(dt, launch_compact<T>(h, out_msg, out_capacity, static_cast<const T*>(data), static_cast<T*>(update), n,
                                      static_cast<const T*>(thr_host), static_cast<const T*>(d_thr), d_size_prefix,
                                      true));
}

long long cx_noalloc_max_elements(void) { return noalloc_max_elements(); }

int cx_reserve(cx_handle h, cx_dtype dt, int n, unsigned paths) {
    if (!h || n < 0) return fail(CX_ERR_INVALID, "cx_reserve: null handle or negative size");
    if (paths == 0u || (paths & ~(unsigned)CX_RESERVE_ALL)) return fail(CX_ERR_INVALID, "cx_reserve: unknown path bits %#x", paths);
    CX_DISPATCH(dt, reserve_impl<T>(h, n, paths));
}

int cx_ip_compress_topk(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity, const void* data, void* update,
                        int n, float topK, void* d_thr_out, int* d_size_prefix, int* h_bytes) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (n < 0 || !update || !data) return fail(CX_ERR_INVALID, "compress_topk: needs both vectors and a size >= 0");
    if (topK > 1.0f || topK < 0.0f) return fail(CX_ERR_TOPK, "topK value must be between 0.0 and 1.0!");
    CX_DISPATCH(dt, compress_topk_impl<T>(h, out_msg, out_capacity, data, update, n, topK, d_thr_out, d_size_prefix,
                                          h_bytes));
}

int cx_ip_write_step(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity, const void* data, void* update,
                     int n, float topK, int default_subsamples, float subsample_factor, const int* d_idx, int m,
                     void* d_thr_out, int* d_size_prefix, int* h_bytes) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (n < 0 || !update || !data || m < 0) return fail(CX_ERR_INVALID, "write_step: needs both vectors and sizes >= 0");
    if (topK > 1.0f || topK < 0.0f) return fail(CX_ERR_TOPK, "topK value must be between 0.0 and 1.0!");
    CX_DISPATCH(dt, write_step_impl<T>(h, out_msg, out_capacity, data, update, n, topK, default_subsamples,
                                       subsample_factor, d_idx, m, d_thr_out, d_size_prefix, h_bytes));
}

int cx_rle_compress(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity, const void* data, void* update,
                    int n, const void* thr_host, const void* d_thr, int* d_size_prefix, int* h_bytes) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    CX_DISPATCH(dt, rle_compress_impl<T>(h, out_msg, out_capacity, data, update, n, thr_host, d_thr, d_size_prefix,
                                         h_bytes));
}

int cx_rle_decompress(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg, int* h_n) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (!aligned4(msg)) return fail(CX_ERR_INVALID, "message must be 4-byte aligned");
    CX_DISPATCH(dt, launch_rle_decode<T>(h, static_cast<T*>(out), out_n, msg, 0, h_n));
}

int cx_rle_add(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (!msg || !aligned4(msg)) return fail(CX_ERR_INVALID, "message must be a 4-byte aligned device pointer");
    CX_DISPATCH(dt, launch_rle_decode<T>(h, static_cast<T*>(out), out_n, msg, 1, nullptr));
}

int cx_ip_decompress(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg, int* h_bytes) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (!aligned4(msg)) return fail(CX_ERR_INVALID, "message must be 4-byte aligned");
    CX_DISPATCH(dt, decompress_impl<T>(h, out, out_n, msg, h_bytes));
}

int cx_ip_add(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg, int check) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    if (!msg || !aligned4(msg)) return fail(CX_ERR_INVALID, "message must be a 4-byte aligned device pointer");
    // any index order: decided on the device, nothing waits (a message made for a longer vector is
    // refused by the kernels themselves and reported with the status, like every other device-side error)
    if (check == CX_ADD_ANY_ORDER) CX_DISPATCH(dt, launch_add_any_order<T>(h, static_cast<T*>(out), out_n, msg));
    if (check) {
        CX_HIP(hipMemcpyAsync(h->h_pinned + 8, msg, 8, hipMemcpyDeviceToHost, h->stream));
        CX_HIP(hipStreamSynchronize(h->stream));
        if (h->h_pinned[8] > out_n)
            return fail(CX_ERR_MSG_TOO_LARGE, "Decompression vector size is bigger than output buffer!");
    }
    CX_DISPATCH(dt, launch_add<T>(h, static_cast<T*>(out), out_n, msg, 0));
}

int cx_ip_reduce(cx_handle h, cx_dtype dt, void* out, int out_n, const void* const* msgs, int n_msgs, int accumulate,
                 int mode) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    for (int r = 0; r < n_msgs; ++r)
        if (!msgs || !msgs[r] || !aligned4(msgs[r]))
            return fail(CX_ERR_INVALID, "message %d must be a 4-byte aligned device pointer", r);
    if ((mode & CX_REDUCE_ANY_ORDER) && n_msgs > 0) {
        int sorted = 1;
        long long pairs = 0;
        CX_DISPATCH_RC(dt, messages_sorted<T>(h, msgs, n_msgs, &sorted, &pairs));
        if (!sorted) {
            // the reference's loop, message after message, pair after pair (src/compressor.hxx:640-658)
            if (!accumulate) CX_DISPATCH_RC(dt, launch_zero<T>(h, static_cast<T*>(out), out_n));
            for (int r = 0; r < n_msgs; ++r)
                CX_DISPATCH_RC(dt, launch_sequential<T>(h, static_cast<T*>(out), out_n, msgs[r], 1));
            return CX_OK;
        }
        // Adding sparse messages into a long vector: one scatter per message touches the pairs' elements
        // only, a pass over the vector reads and writes all of it.  Measured, fp32, 1 %-dense messages added
        // into 64 Mi elements, 1 / 2 / 4 / 8 messages: 20.5 / 40.9 / 84.0 / 200 us as scatters against 83 /
        // 88 / 93 / 94 us as one pass; into 16 Mi elements 4.7 / 10.2 / 23.2 / 45.6 against 24.0 / 25.6 /
        // 28.4 / 33.6 us; into 1 Mi elements 4.5 / 7.0 / 12.5 / 23.1 against 7.0 / 7.1 / 8.1 / 10.3 us.  The
        // model below (4.5 us a launch, 0.03 us per thousand pairs; 7 us + the vector's bytes twice at
        // 6.5 TB/s) follows those figures; the pair count is known here because the order check read it.
        if (accumulate && (mode & ~CX_REDUCE_ANY_ORDER) == 0 && h->reduce_variant == 0) {
            const double elem_bytes = dt == CX_F64 ? 8.0 : 4.0;
            const double scatter_us = 4.5 * n_msgs + 0.03e-3 * (double)pairs;
            const double pass_us = 7.0 + 2.0 * elem_bytes * (double)out_n / 6.5e6;
            if (scatter_us < pass_us) {
                for (int r = 0; r < n_msgs; ++r)
                    CX_DISPATCH_RC(dt, launch_add<T>(h, static_cast<T*>(out), out_n, msgs[r], 0));
                return CX_OK;
            }
        }
    }
    mode &= ~CX_REDUCE_ANY_ORDER;
    CX_DISPATCH(dt, launch_reduce<T>(h, static_cast<T*>(out), out_n, msgs, n_msgs, accumulate, mode));
}

int cx_zero(cx_handle h, cx_dtype dt, void* v, int n) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    CX_DISPATCH(dt, launch_zero<T>(h, static_cast<T*>(v), n));
}

int cx_add_vec(cx_handle h, cx_dtype dt, void* data, const void* rests, int n) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    CX_DISPATCH(dt, launch_add_vec<T>(h, static_cast<T*>(data), static_cast<const T*>(rests), n));
}

int cx_threshold_apply(cx_handle h, cx_dtype dt, void* high, void* low, const void* in, int n, const void* thr_host,
                       const void* d_thr) {
    if (!h) return fail(CX_ERR_INVALID, "null handle");
    CX_DISPATCH(dt, launch_threshold_apply<T>(h, static_cast<T*>(high), static_cast<T*>(low), static_cast<const T*>(in),
                                              n, static_cast<const T*>(thr_host), static_cast<const T*>(d_thr)));
}

}  // extern "C"
