// The reference's float-only C ABI (libPyGPI.so: src/comprEx_C.cpp:17-87, src/GPI_C.cpp:41-73)
// on top of this library's C++ classes, so that the reference's ctypes wrappers
// (ComprEx.py, gpi.py) bind to libcomprex_gfx950.so unchanged.
//
// The reference lets std::runtime_error escape through extern "C" (which ends the process
// under ctypes).  Here every call catches, remembers the text for Comprex_lastError() and
// returns; Comprex_lastError() is cleared by the next successful call.
#include <cstdio>
#include <string>

#include "../../include/allreduce.hxx"
#include "../../include/comprEx.hxx"
#include "../../include/compressor.hxx"
#include "../../include/gaspiEnvironment.hxx"
#include "../../include/threshold.hxx"

typedef float data_t;

namespace {

std::string& abi_error() {
    static thread_local std::string msg;
    return msg;
}

template <class F> void guarded(F&& f) {
    try {
        f();
        abi_error().clear();
    } catch (const std::exception& e) {
        abi_error() = e.what();
    }
}

template <class R, class F> R guarded_value(R fallback, F&& f) {
    try {
        R r = f();
        abi_error().clear();
        return r;
    } catch (const std::exception& e) {
        abi_error() = e.what();
        return fallback;
    }
}

}  // namespace

extern "C" {

const char* Comprex_lastError(void) { return abi_error().c_str(); }

// ---- GaspiEnvironment (src/GPI_C.cpp:41-73) --------------------------------------------
void* GaspiEnvironment_new(int segment_size) {
    return guarded_value<void*>(nullptr, [&] { return (void*)new GaspiEnvironment((unsigned long)segment_size); });
}
void GaspiEnvironment_del(void* self) { delete static_cast<GaspiEnvironment*>(self); }
int GaspiEnvironment_get_rank(void* self) { return static_cast<GaspiEnvironment*>(self)->get_rank(); }
int GaspiEnvironment_get_ranks(void* self) { return static_cast<GaspiEnvironment*>(self)->get_ranks(); }
void GaspiEnvironment_barrier(void* self) { static_cast<GaspiEnvironment*>(self)->barrier(); }
void GaspiEnvironment_flush(void* self) { static_cast<GaspiEnvironment*>(self)->flush(); }
void GaspiEnvironment_set_rank(void* self, int rank, int ranks) {
    guarded([&] { static_cast<GaspiEnvironment*>(self)->set_rank(rank, ranks); });
}
void GaspiEnvironment_set_blocking(void* self, int blocking, double timeout_s) {
    static_cast<GaspiEnvironment*>(self)->set_blocking(blocking != 0, timeout_s);
}
void GaspiEnvironment_set_user_stream(void* self, void* hip_stream) {
    static_cast<GaspiEnvironment*>(self)->set_user_stream(hip_stream);
}
void Gaspi_Printf(const char* msg) {
    printf("%s\n", msg);
    fflush(stdout);
}

// ---- ComprEx (src/comprEx_C.cpp:17-53) ---------------------------------------------------
void* Comprex_new(void* gaspi_env, int size, float size_factor) {
    return guarded_value<void*>(nullptr, [&] {
        return (void*)new ComprEx<data_t>(static_cast<GaspiEnvironment*>(gaspi_env)->get_segment(), size, size_factor);
    });
}
void Comprex_del(void* self) { delete static_cast<ComprEx<data_t>*>(self); }
void Comprex_setThreshold(void* self, const void* threshold) {
    guarded([&] {
        static_cast<ComprEx<data_t>*>(self)->setThreshold(static_cast<const ThresholdFunction<data_t>*>(threshold));
    });
}
void Comprex_setCompressor(void* self, const void* compressor) {
    guarded(
        [&] { static_cast<ComprEx<data_t>*>(self)->setCompressor(static_cast<const Compressor<data_t>*>(compressor)); });
}
void Comprex_resetRests(void* self) { guarded([&] { static_cast<ComprEx<data_t>*>(self)->resetRests(); }); }
void Comprex_flushRests(void* self) { guarded([&] { static_cast<ComprEx<data_t>*>(self)->flushRests(); }); }
void Comprex_getRests(void* self, float* vector, int size) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->getRests(vector, size); });
}
void Comprex_writeRemote(void* self, const float* vector, int size) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->writeRemote(vector, size); });
}
void Comprex_readRemote(void* self, float* vector, int size) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->readRemote(vector, size); });
}
void Comprex_readRemote_add(void* self, float* vector, int size) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->readRemote_add(vector, size); });
}
void Comprex_connectTo(void* self, int srcRank, int targRank, int tag) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->connectTo(srcRank, targRank, tag); });
}
void Comprex_connectTx(void* self, int targRank, int tag) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->connectTx(targRank, tag); });
}
void Comprex_connectRx(void* self, int srcRank, int tag) {
    guarded([&] { static_cast<ComprEx<data_t>*>(self)->connectRx(srcRank, tag); });
}

// ---- thresholds (src/comprEx_C.cpp:58-71) ------------------------------------------------
void* ThresholdNone_new(void) { return new ThresholdNone<data_t>(); }
void ThresholdNone_del(void* self) { delete static_cast<ThresholdNone<data_t>*>(self); }
void* ThresholdConst_new(float thr) {
    return guarded_value<void*>(nullptr, [&] { return (void*)new ThresholdConst<data_t>(thr); });
}
void ThresholdConst_del(void* self) { delete static_cast<ThresholdConst<data_t>*>(self); }
float ThresholdConst_getThreshold(void* self) { return static_cast<ThresholdConst<data_t>*>(self)->get_threshold(); }
void* ThresholdTopK_new(float topK) {
    return guarded_value<void*>(nullptr, [&] { return (void*)new ThresholdTopK<data_t>(topK); });
}
void ThresholdTopK_del(void* self) { delete static_cast<ThresholdTopK<data_t>*>(self); }
float ThresholdTopK_getThreshold(void* self) {
    return guarded_value<float>(0.0f, [&] { return static_cast<ThresholdTopK<data_t>*>(self)->get_threshold(); });
}

// ---- compressors (src/comprEx_C.cpp:76-87) ----------------------------------------------------
void* CompressorNone_new(void) { return new CompressorNone<data_t>(); }
void CompressorNone_del(void* self) { delete static_cast<CompressorNone<data_t>*>(self); }
void* CompressorRLE_new(void) { return new CompressorRLE<data_t>(); }
void CompressorRLE_del(void* self) { delete static_cast<CompressorRLE<data_t>*>(self); }
void* CompressorIndexPairs_new(void) { return new CompressorIndexPairs<data_t>(); }
void CompressorIndexPairs_del(void* self) { delete static_cast<CompressorIndexPairs<data_t>*>(self); }

// ---- compressed allreduce schedules (src/allreduce_C.cpp:26-122) ----------------------------
// One object per simulated rank, used from that rank's own thread (GaspiEnvironment_set_rank +
// GaspiEnvironment_set_blocking); apply/flush work in place on `data` (host or device pointer).
#define CX_ALLREDUCE_COMMON(NAME)                                                                        \
    void* NAME##_new(void* gaspi_env) {                                                                  \
        return guarded_value<void*>(nullptr, [&] { return (void*)new NAME<data_t>(static_cast<GaspiEnvironment*>(gaspi_env)); }); \
    }                                                                                                    \
    void NAME##_del(void* self) { delete static_cast<NAME<data_t>*>(self); }                             \
    void NAME##_apply(void* self, float* data, int size) {                                               \
        guarded([&] { static_cast<NAME<data_t>*>(self)->apply(data, size); });                           \
    }                                                                                                    \
    void NAME##_flush(void* self, float* data, int size) {                                               \
        guarded([&] { static_cast<NAME<data_t>*>(self)->flush(data, size); });                           \
    }                                                                                                    \
    void NAME##_reset(void* self) { guarded([&] { static_cast<NAME<data_t>*>(self)->reset(); }); }       \
    void NAME##_set_compression_ratio(void* self, float compression_ratio) {                             \
        guarded([&] { static_cast<NAME<data_t>*>(self)->set_compression_ratio(compression_ratio); });    \
    }
CX_ALLREDUCE_COMMON(Comprex_AllToOneAllreduce)
CX_ALLREDUCE_COMMON(Comprex_RingAllreduce)
CX_ALLREDUCE_COMMON(Comprex_BigRingAllreduce)
void Comprex_AllToOneAllreduce_setupConnections(void* self, int size, int tag, int chiefRank, float compression_ratio,
                                                float size_factor) {
    guarded([&] {
        static_cast<Comprex_AllToOneAllreduce<data_t>*>(self)->setupConnections(size, tag, chiefRank, compression_ratio,
                                                                                 size_factor);
    });
}
void Comprex_RingAllreduce_setupConnections(void* self, int size, int tag, float compression_ratio, float size_factor) {
    guarded([&] {
        static_cast<Comprex_RingAllreduce<data_t>*>(self)->setupConnections(size, tag, compression_ratio, size_factor);
    });
}
void Comprex_BigRingAllreduce_setupConnections(void* self, int size, int tag, float compression_ratio,
                                               float size_factor) {
    guarded([&] {
        static_cast<Comprex_BigRingAllreduce<data_t>*>(self)->setupConnections(size, tag, compression_ratio, size_factor);
    });
}

}  // extern "C"
