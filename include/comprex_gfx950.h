/*
 * comprex_gfx950.h -- C ABI of the MI355X (gfx950) implementation of ComprEx's
 * gradient-compression hot path.
 *
 * Two groups of entry points live in libcomprex_gfx950.so:
 *
 *  1. cx_*  : the kernel-level boundary.  Plain pointers and sizes, no C++ or torch
 *             types.  Vectors and messages are DEVICE pointers (anything the GPU can
 *             dereference); scalars are passed by value or through small host
 *             pointers.  Each function cites the reference interface it replaces
 *             (paths relative to the reference tree).  Calls are enqueued on the
 *             handle's HIP stream and return without waiting unless a host output
 *             pointer is given.
 *
 *  2. The reference's own float-only symbol set (src/comprEx_C.cpp:17-87,
 *     src/GPI_C.cpp:41-73, src/allreduce_C.cpp:26-122), so that the reference's
 *     ctypes wrappers bind unchanged; declared at the end of this file.
 *
 * Element types: the reference's templates are instantiated for float in its C ABI
 * (src/comprEx_C.cpp:12) and for int in its tests (test/compressor.cpp:8); double is
 * allowed by the templates.  All three are supported here (cx_dtype).
 *
 * Message layout (src/compressor.hxx:559-565,606), unchanged:
 *     int32 n (uncompressed length) | int32 k (pairs) | k x { int32 index, T value }
 * pairs packed without padding, indices strictly ascending.
 */
#ifndef COMPREX_GFX950_H
#define COMPREX_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cx_handle_s* cx_handle;

typedef enum { CX_F32 = 0, CX_F64 = 1, CX_I32 = 2 } cx_dtype;

typedef enum {
    CX_OK = 0,
    CX_ERR_INVALID = 1,        /* bad argument (null pointer, negative size, unknown dtype) */
    CX_ERR_SIZE_MISMATCH = 2,  /* vector sizes differ (reference: throws, compressor.hxx:45-49, threshold.hxx:161-163) */
    CX_ERR_MSG_TOO_LARGE = 3,  /* message's vector length exceeds the output (compressor.hxx:620-624,645-647) */
    CX_ERR_CAPACITY = 4,       /* message would not fit the caller's buffer (the reference overruns silently) */
    CX_ERR_INDEX = 5,          /* a pair's index lies outside the output vector (the reference overruns silently) */
    CX_ERR_HIP = 6,            /* a HIP runtime call failed */
    CX_ERR_INTERNAL = 7,       /* a bounded device-side wait expired */
    CX_ERR_TOPK = 8            /* topK outside [0,1] (threshold.hxx:131-133) */
} cx_status;

/* Text of the last error raised on the calling thread. */
const char* cx_last_error(void);
/* ABI version of this header. */
int cx_abi_version(void);
/* Number of HIP devices visible (0 when there is no GPU); never throws. */
int cx_device_count(void);
/* 1 when `p` is device (or managed/host-registered) memory, 0 for pageable host memory. */
int cx_pointer_on_device(const void* p);

/* Device memory for callers without a HIP runtime of their own (the C++ classes of this
 * library's headers keep the residual and their staging buffers in it).  cx_copy moves bytes
 * between any two pointers (host or device) in stream order and waits when a pageable host
 * buffer is involved.  They stand in for the std::vector / memcpy of src/comprEx.tpp:149-157. */
int cx_device_alloc(void** out, size_t bytes);
int cx_device_free(void* p);
int cx_copy(cx_handle h, void* dst, const void* src, size_t bytes);

/* The handle's scratch buffers grow on demand, which makes a call that finds them too small wait for
 * the stream and allocate.  cx_reserve sizes them ahead of time for vectors of up to n elements of
 * type `dt`, for the paths named in `paths` (an OR of the bits below), so that none of those calls
 * allocates afterwards.  It plays the part of the constructors' allocations in the reference
 * (ComprEx's restsVector and buffers, src/comprEx.tpp:40-60): memory is taken when the object is set
 * up, not in the exchange.  CX_RESERVE_RLE takes 8 + n * (4 + sizeof(T)) bytes (the pairs its
 * encoder starts from); the others take about n/2 bytes or less. */
enum {
    CX_RESERVE_COMPRESS = 1,   /* cx_ip_compress, the compaction of cx_ip_compress_topk */
    CX_RESERVE_THRESHOLD = 2,  /* cx_topk_threshold*, the candidate list of cx_ip_compress_topk */
    CX_RESERVE_REDUCE = 4,     /* cx_ip_decompress, cx_ip_add, cx_ip_reduce on vectors of n elements */
    CX_RESERVE_RLE = 8,        /* cx_rle_compress */
    CX_RESERVE_ALL = 15
};
int cx_reserve(cx_handle h, cx_dtype dt, int n, unsigned paths);

/* No counterpart in the reference, whose transports take a host-side byte count
 * (initTransferPart(sizeBytes, offset), src/comprEx.tpp:442): copies *d_bytes bytes (a device
 * int32, e.g. the size prefix a compressor wrote; clamped to [0, capacity]) from src to dst, device
 * memory both, in stream order, without the host ever reading the count. */
int cx_copy_counted(cx_handle h, void* dst, const void* src, const int* d_bytes, long long capacity);

/* A handle owns one HIP stream reference and the scratch memory of one compressor
 * clone (tile descriptors, histograms, a device-side threshold slot, a status word).
 * It replaces the per-object state of Compressor<T>/ThresholdFunction<T> clones
 * (src/comprEx.tpp:94-112).  Not thread safe, like the reference's objects. */
int cx_create(cx_handle* out, void* hip_stream /* hipStream_t, NULL = default stream */);
int cx_destroy(cx_handle h);
int cx_set_stream(cx_handle h, void* hip_stream);
void* cx_get_stream(cx_handle h);

/* Streams and events for callers that hold no HIP headers (the C++ classes of include/ (.hxx) are
 * plain host code).  The reference's RDMA put is asynchronous and its receiver waits for a
 * notification (src/comprEx.tpp:190,231,243): here every ComprEx object works on a stream of its
 * own and a message's hand-over is an event the sender records and the receiver's stream waits
 * for.  cx_stream_create makes a non-blocking stream (no implicit ordering with the null stream),
 * cx_stream_create_blocking one the runtime orders with the null stream (what the objects use);
 * both at the default priority; events carry no timing.  A NULL stream argument names the null stream. */
int cx_stream_create(void** out_stream);
/* A stream that IS ordered with the null stream, both ways, by the runtime (a "blocking" stream): what an
 * object whose caller works on the null stream needs, without an event join around every call. */
int cx_stream_create_blocking(void** out_stream);
int cx_stream_destroy(void* hip_stream);
int cx_stream_synchronize(void* hip_stream);
int cx_event_create(void** out_event);
int cx_event_destroy(void* hip_event);
int cx_event_record(void* hip_event, void* hip_stream);
int cx_stream_wait_event(void* hip_stream, void* hip_event);
/* Waits for the handle's stream and returns the first device-side error seen since the
 * last call (CX_OK if none), clearing it. */
int cx_synchronize(cx_handle h);
/* Tuning switches: "compact_items" (16-byte loads per lane and tile: 2, 4 or 8; 0 = by the vector's length, the default),
 * "stage_alternate" (1 = every other compress walks the vector from its end, so that it starts on
 * what the previous one left in the memory-side cache), "profile_stage" (see cx_profile_read),
 * "reduce_variant", "select_bracket" (1 = whole-vector thresholds try a one-pass selection first),
 * "fused_topk" (0 = cx_ip_compress_topk never takes its single-pass route, 1 = where it is the
 * faster one, from 20 Mi elements on, 2 = from 2^23 elements on).  Unknown keys return
 * CX_ERR_INVALID. */
int cx_set_option(cx_handle h, const char* key, int value);
/* Reads an option back; also "fused_topk_taken": how the last cx_ip_compress_topk ran
 * (0 = threshold and compress as two steps, 1 = single pass, 2 = single pass abandoned). */
int cx_get_option(cx_handle h, const char* key, int* value);

/* No counterpart in the reference: a measurement aid.  After cx_set_option(h, "profile_stage", N)
 * every N-th cx_ip_compress records a HIP event before and after its streaming kernel, on the
 * handle's stream (at most 1024 recorded launches between reads; the two events cost a few
 * microseconds per recorded launch).  This call waits for the stream and returns the
 * elapsed milliseconds of those launches, oldest first, and forgets them. */
int cx_profile_read(cx_handle h, float* ms_out, int max_out, int* n_out);

/* ---- thresholds ----------------------------------------------------------- */

/* ThresholdTopK<T>::calc_subsamples (src/threshold.hxx:182-186).  -1 where the
 * reference's float->int conversion is undefined. */
int cx_topk_subsamples(float topK, int default_subsamples, float subsample_factor);
/* topk_pos of ThresholdTopK<T>::calc_threshold (src/threshold.hxx:190). */
int cx_topk_pos(size_t m, float topK);

/* ThresholdTopK<T>::prepare_with(vec, n, add_vec, n) / prepare(vec, n) when add_vec is
 * NULL (src/threshold.hxx:152-167): strided sub-sample (or the whole vector when
 * n < subsamples) of vec[p] + add_vec[p], then the (topk_pos+1)-th largest magnitude
 * (or max+1 when topk_pos <= 0).  The threshold is written to `d_thr_out` (device, T;
 * NULL = the handle's own slot, see cx_threshold_slot) and, when `h_thr_out` is not
 * NULL, also copied to the host (this waits for the stream). */
int cx_topk_threshold(cx_handle h, cx_dtype dt, const void* vec, const void* add_vec, int n, int add_n,
                      float topK, int default_subsamples, float subsample_factor,
                      void* d_thr_out, void* h_thr_out);
/* Same order statistic over m host-chosen sample positions d_idx[0..m) (device int32):
 * keys are vec[idx] (+ add_vec[idx]); a position outside [0, n) counts as a key of magnitude 0
 * and is never dereferenced.  No counterpart in the reference, whose sampling is always strided
 * (src/threshold.hxx:224-240); calc_threshold (:189-205) is unchanged. */
int cx_topk_threshold_indexed(cx_handle h, cx_dtype dt, const void* vec, const void* add_vec,
                              int n, const int* d_idx, int m, float topK, void* d_thr_out, void* h_thr_out);
/* Device address of the handle's threshold slot (8 bytes, holds a T). */
void* cx_threshold_slot(cx_handle h);

/* ---- IndexPairs codec ------------------------------------------------------ */

/* CompressorIndexPairs<T>::compression_strategy (src/compressor.hxx:556-611) behind
 * Compressor<T>::compress / compress_update / compress_add_update (:36-51):
 *   data != NULL, update != NULL : update += data; emit |update| > thr; zero emitted
 *   data == NULL                 : emit |update| > thr; zero emitted
 *   update == NULL               : emit |data| > thr
 * `out_msg` needs 4-byte alignment only.  The threshold comes from `thr_host`
 * (pointer to a host T) or, when that is NULL, from `d_thr` (device T; NULL = the
 * handle's slot).  `out_capacity` is the size in bytes of out_msg: pairs beyond it are
 * not written and CX_ERR_CAPACITY is recorded.  `d_size_prefix` (device int32, may be
 * NULL) receives the message's byte count (the send_sizeBytes prefix of
 * src/comprEx.tpp:184-188).  When `h_bytes` is not NULL the call waits and stores the
 * bytes written (8 + k*(4+sizeof(T))), as the reference returns them. */
int cx_ip_compress(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity,
                   const void* data, void* update, int n,
                   const void* thr_host, const void* d_thr,
                   int* d_size_prefix, int* h_bytes);

/* No counterpart in the reference.  cx_ip_compress for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * same kernels, same message, residual and size prefix, but the compaction's scratch (staging
 * slots, per-tile counts and offsets, per-block sums) lives in a static device array of about
 * 26 MB that each GPU holds from the moment the library's code is loaded there until the process
 * ends, instead of in buffers the handle grows on demand.  No hipMalloc, hipFree or other
 * allocating call is made and the call never waits; the byte count is delivered through
 * d_size_prefix and the message header only.  n may not exceed cx_noalloc_max_elements()
 * (16 777 216, any element type): larger vectors are refused with CX_ERR_INVALID.  All handles on
 * one GPU share that array: calls that overlap in time on one GPU (different streams) race;
 * calls in stream order do not.  The handle itself (cx_create) is made beforehand. */
int cx_ip_compress_noalloc(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity,
                           const void* data, void* update, int n,
                           const void* thr_host, const void* d_thr, int* d_size_prefix);
long long cx_noalloc_max_elements(void);

/* ComprEx<T>::writeRemote with a whole-vector ThresholdTopK (src/comprEx.tpp:176-191 calling
 * src/threshold.hxx:160-167 in its `n < subsamples` mode, :224-231, and src/compressor.hxx:44-51):
 * the exact top-k threshold of |update + data| and the fused compress_add_update of
 * cx_ip_compress, same message, residual and threshold as cx_topk_threshold followed by
 * cx_ip_compress, but with ONE pass over the two vectors when n >= 2^23 and topK is small
 * (a sampled lower bound of the threshold selects candidates during the accumulate pass; the
 * exact threshold is found among them; if the bound turns out unusable the result is
 * computed from the accumulated vector instead).  The threshold is left in `d_thr_out`
 * (device T; NULL = the handle's slot).  Waits for the stream once.  Other arguments as
 * cx_ip_compress. */
int cx_ip_compress_topk(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity,
                        const void* data, void* update, int n, float topK,
                        void* d_thr_out, int* d_size_prefix, int* h_bytes);

/* ComprEx<T>::writeRemote with ANY ThresholdTopK (src/comprEx.tpp:183-185): ThresholdTopK(topK,
 * default_subsamples, subsample_factor)::prepare_with(update, data) (src/threshold.hxx:160-167,
 * 182-240: the whole vector when n < subsamples, else `subsamples` strided positions) followed by
 * compress_add_update with that threshold, as one call.  d_idx / m (device int32 positions, m > 0)
 * replace the strided rule by the caller's sample positions.  A whole-vector threshold takes
 * cx_ip_compress_topk's route, a sampled one cx_topk_threshold[_indexed] + cx_ip_compress: the same
 * kernels, message, residual and threshold as the separate calls, enqueued by one call that never
 * waits unless asked to (so that a caller may capture it in a HIP graph: short vectors are all
 * launch latency, and a replayed graph halves it).  The threshold is left in d_thr_out (device T;
 * NULL = the handle's slot).  h_bytes != NULL waits and returns the byte count. */
int cx_ip_write_step(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity,
                     const void* data, void* update, int n, float topK, int default_subsamples,
                     float subsample_factor, const int* d_idx, int m, void* d_thr_out,
                     int* d_size_prefix, int* h_bytes);

/* CompressorRLE<T> (src/compressor.hxx:158-532), the run-length codec: message
 * int32 n | int32 c | c values | int32 runs | int32 signum | runs x int32 run lengths, an element
 * is sent when |x| >= threshold.  cx_rle_compress = compression_strategy (:167-390) in its three
 * modes (arguments as cx_ip_compress), with the sent values stored densely: the reference's
 * encoder indexes them by vector position (:238,277,316) and only produces a decodable message
 * when every element is sent.  cx_rle_decompress = decompression_strategy (:393-470): writes
 * the message's n elements (nothing beyond), *h_n receives n, which is what the reference
 * returns; CX_ERR_MSG_TOO_LARGE when n > out_n.  cx_rle_add = add_strategy (:473-530).
 * The two decoders read the message's header on the host (they wait for the stream). */
int cx_rle_compress(cx_handle h, cx_dtype dt, void* out_msg, long long out_capacity,
                    const void* data, void* update, int n,
                    const void* thr_host, const void* d_thr,
                    int* d_size_prefix, int* h_bytes);
int cx_rle_decompress(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg, int* h_n);
int cx_rle_add(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg);

/* CompressorIndexPairs<T>::decompression_strategy (src/compressor.hxx:613-638): zero
 * all out_n elements, then out[index] = value.  A message whose n exceeds out_n leaves
 * `out` zeroed and records CX_ERR_MSG_TOO_LARGE.  h_bytes as above (bytes consumed).
 * Index order: the compressors of this library and of the reference emit ascending indices, and
 * the fast path requires them (an index below its predecessor records CX_ERR_INDEX).  The
 * reference's decoder takes any order, repeats anywhere, last value wins: with h_bytes != NULL
 * a pass over the indices runs first and the device decides between the fast kernels and the
 * pair-after-pair kernel, with exactly that result (one wait, at the end, for the byte count and
 * the status); with h_bytes == NULL the fast path runs alone and the error stands.  Indices outside
 * [0, out_n) are CX_ERR_INDEX either way (the reference writes out of bounds). */
int cx_ip_decompress(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg, int* h_bytes);

/* CompressorIndexPairs<T>::add_strategy (src/compressor.hxx:640-658): out[index] += value
 * in message order.  A message whose n exceeds out_n changes nothing and records
 * CX_ERR_MSG_TOO_LARGE.  `check` == 1 reads the header first and returns that error
 * synchronously, as the reference throws before touching `out`.
 * Index order: the kernel applies a run of equal NEIGHBOURING indices in message order, which is
 * all an index-sorted message (what the compressors emit) needs; an index below its predecessor
 * records CX_ERR_INDEX, because equal indices may then lie apart and `out` is no longer what the
 * reference's loop gives.  check == CX_ADD_ANY_ORDER takes any order, exactly as the reference does,
 * and waits for nothing: a pass over the indices, the fast kernel and the pair-after-pair kernel are
 * enqueued one behind the other and the device decides which of the two does the work; errors
 * (the oversize message included) come with the status, as from any asynchronous call. */
enum { CX_ADD_ANY_ORDER = 2 };
int cx_ip_add(cx_handle h, cx_dtype dt, void* out, int out_n, const void* msg, int check);

/* The chief's reduce loop of Comprex_AllToOneAllreduce::apply (src/allreduce.tpp:183-189):
 * out (+)= sum over messages in the order given.  `msgs` is a HOST array of n_msgs device
 * pointers.  accumulate == 0 starts from zeros (every message is added, the first one to
 * 0), != 0 adds into `out`.  mode 0 = rank-ordered, bit-exact, needs every message's indices
 * ascending (CX_ERR_INDEX otherwise; option reduce_variant = 1 only needs equal indices to be
 * neighbours); mode 1 = one launch of floating-point atomics per message, in the order given:
 * the additions to an element are reordered only among pairs of ONE message that share its
 * index.  An empty `out` (out_n == 0) writes nothing and still refuses messages made for a
 * longer vector (CX_ERR_MSG_TOO_LARGE).  mode | CX_REDUCE_ANY_ORDER: the call first looks at the
 * indices (one pass, one wait for the stream) and, when a message is not index-sorted, applies the
 * messages one after the other, pair after pair, as the reference's loop does: any order, equal
 * indices anywhere; without it such a message records CX_ERR_INDEX and leaves `out` undefined. */
enum { CX_REDUCE_ANY_ORDER = 4 };
int cx_ip_reduce(cx_handle h, cx_dtype dt, void* out, int out_n, const void* const* msgs, int n_msgs,
                 int accumulate, int mode);

/* ---- residual maintenance -------------------------------------------------- */

/* ComprEx<T>::resetRests (src/comprEx.tpp:121-126): v[0..n) = 0. */
int cx_zero(cx_handle h, cx_dtype dt, void* v, int n);
/* ComprEx<T>::addRests (src/comprEx.tpp:159-169): data[i] += rests[i]. */
int cx_add_vec(cx_handle h, cx_dtype dt, void* data, const void* rests, int n);
/* ThresholdFunction<T>::apply with a given threshold (src/threshold.hxx:19-27):
 * out = |in| >= thr ? in : 0, and apply_split (:30-50) when `low` is not NULL. */
int cx_threshold_apply(cx_handle h, cx_dtype dt, void* high, void* low, const void* in, int n,
                       const void* thr_host, const void* d_thr);

/* ---- the reference's C ABI (float only) ------------------------------------- */
/* src/GPI_C.cpp:41-73.  One process stands for `ranks` simulated ranks that exchange
 * messages through device buffers; segment_size is accepted and ignored. */
void* GaspiEnvironment_new(int segment_size);
void GaspiEnvironment_del(void* self);
int GaspiEnvironment_get_rank(void* self);
int GaspiEnvironment_get_ranks(void* self);
void GaspiEnvironment_barrier(void* self);
void GaspiEnvironment_flush(void* self);
void Gaspi_Printf(const char* msg);
/* Not in the reference: selects which simulated rank the next calls act as, and how many
 * there are (the reference gets both from gaspi_run). */
void GaspiEnvironment_set_rank(void* self, int rank, int ranks);

/* src/comprEx_C.cpp:17-87 */
void* Comprex_new(void* gaspi_env, int size, float size_factor);
void Comprex_del(void* self);
void Comprex_setThreshold(void* self, const void* threshold);
void Comprex_setCompressor(void* self, const void* compressor);
void Comprex_resetRests(void* self);
void Comprex_flushRests(void* self);
void Comprex_getRests(void* self, float* vector, int size);
void Comprex_writeRemote(void* self, const float* vector, int size);
void Comprex_readRemote(void* self, float* vector, int size);
void Comprex_readRemote_add(void* self, float* vector, int size);
void Comprex_connectTo(void* self, int srcRank, int targRank, int tag);
void Comprex_connectTx(void* self, int targRank, int tag);
void Comprex_connectRx(void* self, int srcRank, int tag);
void* ThresholdNone_new(void);
void ThresholdNone_del(void* self);
void* ThresholdConst_new(float thr);
void ThresholdConst_del(void* self);
float ThresholdConst_getThreshold(void* self);
void* ThresholdTopK_new(float topK);
void ThresholdTopK_del(void* self);
float ThresholdTopK_getThreshold(void* self);
void* CompressorNone_new(void);
void CompressorNone_del(void* self);
void* CompressorRLE_new(void);
void CompressorRLE_del(void* self);
void* CompressorIndexPairs_new(void);
void CompressorIndexPairs_del(void* self);
/* src/allreduce_C.cpp:26-122, the three compressed schedules.  One object per simulated rank, driven
 * from that rank's own host thread (GaspiEnvironment_set_rank, then GaspiEnvironment_set_blocking so
 * that receives wait for their message); apply/flush work in place on `data`, host or device. */
void GaspiEnvironment_set_blocking(void* self, int blocking, double timeout_s);
/* No counterpart in the reference (its vectors are host memory).  The HIP stream on which the
 * calling thread's device vectors are produced and consumed (NULL, the default, = the null stream):
 * every exchange call joins its object's own stream with it on entry and on exit. */
void GaspiEnvironment_set_user_stream(void* self, void* hip_stream);
void* Comprex_AllToOneAllreduce_new(void* gaspi_env);
void Comprex_AllToOneAllreduce_del(void* self);
void Comprex_AllToOneAllreduce_setupConnections(void* self, int size, int tag, int chiefRank, float compression_ratio,
                                                float size_factor);
void Comprex_AllToOneAllreduce_apply(void* self, float* data, int size);
void Comprex_AllToOneAllreduce_flush(void* self, float* data, int size);
void Comprex_AllToOneAllreduce_reset(void* self);
void Comprex_AllToOneAllreduce_set_compression_ratio(void* self, float compression_ratio);
void* Comprex_RingAllreduce_new(void* gaspi_env);
void Comprex_RingAllreduce_del(void* self);
void Comprex_RingAllreduce_setupConnections(void* self, int size, int tag, float compression_ratio, float size_factor);
void Comprex_RingAllreduce_apply(void* self, float* data, int size);
void Comprex_RingAllreduce_flush(void* self, float* data, int size);
void Comprex_RingAllreduce_reset(void* self);
void Comprex_RingAllreduce_set_compression_ratio(void* self, float compression_ratio);
void* Comprex_BigRingAllreduce_new(void* gaspi_env);
void Comprex_BigRingAllreduce_del(void* self);
void Comprex_BigRingAllreduce_setupConnections(void* self, int size, int tag, float compression_ratio,
                                               float size_factor);
void Comprex_BigRingAllreduce_apply(void* self, float* data, int size);
void Comprex_BigRingAllreduce_flush(void* self, float* data, int size);
void Comprex_BigRingAllreduce_reset(void* self);
void Comprex_BigRingAllreduce_set_compression_ratio(void* self, float compression_ratio);

/* Error text of the last reference-ABI call that failed on this thread ("" if none).  The
 * reference lets std::runtime_error escape through extern "C"; here it is caught. */
const char* Comprex_lastError(void);

#ifdef __cplusplus
}
#endif
#endif
