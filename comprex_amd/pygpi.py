"""Python classes with the names and methods of the reference's ctypes wrappers
(ComprEx.py:100-199, gpi.py: GaspiEnvironment), bound to the same C symbols
(src/comprEx_C.cpp, src/GPI_C.cpp) that libcomprex_gfx950.so exports.

Vectors may be float32 numpy arrays (as in the reference) or 1-D float32 CUDA tensors, in
which case nothing leaves the device.  A C++ exception that the reference would let escape
through extern "C" is raised here as RuntimeError.
"""
import ctypes as C

import numpy as np

from . import _lib

data_t = C.c_float
_vp, _i, _f = C.c_void_p, C.c_int, C.c_float
_PROTOS = {
    "Comprex_lastError": (C.c_char_p, []),
    "GaspiEnvironment_new": (_vp, [_i]), "GaspiEnvironment_del": (None, [_vp]),
    "GaspiEnvironment_get_rank": (_i, [_vp]), "GaspiEnvironment_get_ranks": (_i, [_vp]),
    "GaspiEnvironment_barrier": (None, [_vp]), "GaspiEnvironment_flush": (None, [_vp]),
    "GaspiEnvironment_set_rank": (None, [_vp, _i, _i]), "Gaspi_Printf": (None, [C.c_char_p]),
    "Comprex_new": (_vp, [_vp, _i, _f]), "Comprex_del": (None, [_vp]),
    "Comprex_setThreshold": (None, [_vp, _vp]), "Comprex_setCompressor": (None, [_vp, _vp]),
    "Comprex_resetRests": (None, [_vp]), "Comprex_flushRests": (None, [_vp]),
    "Comprex_getRests": (None, [_vp, _vp, _i]), "Comprex_writeRemote": (None, [_vp, _vp, _i]),
    "Comprex_readRemote": (None, [_vp, _vp, _i]), "Comprex_readRemote_add": (None, [_vp, _vp, _i]),
    "Comprex_connectTo": (None, [_vp, _i, _i, _i]), "Comprex_connectTx": (None, [_vp, _i, _i]),
    "Comprex_connectRx": (None, [_vp, _i, _i]),
    "ThresholdNone_new": (_vp, []), "ThresholdNone_del": (None, [_vp]),
    "ThresholdConst_new": (_vp, [_f]), "ThresholdConst_del": (None, [_vp]),
    "ThresholdConst_getThreshold": (_f, [_vp]),
    "ThresholdTopK_new": (_vp, [_f]), "ThresholdTopK_del": (None, [_vp]),
    "ThresholdTopK_getThreshold": (_f, [_vp]),
    "GaspiEnvironment_set_blocking": (None, [_vp, _i, C.c_double]),
    "GaspiEnvironment_set_user_stream": (None, [_vp, _vp]),
    "CompressorNone_new": (_vp, []), "CompressorNone_del": (None, [_vp]),
    "CompressorRLE_new": (_vp, []), "CompressorRLE_del": (None, [_vp]),
    "CompressorIndexPairs_new": (_vp, []), "CompressorIndexPairs_del": (None, [_vp]),
}
for _fam, _setup in (("Comprex_AllToOneAllreduce", [_vp, _i, _i, _i, _f, _f]),
                     ("Comprex_RingAllreduce", [_vp, _i, _i, _f, _f]),
                     ("Comprex_BigRingAllreduce", [_vp, _i, _i, _f, _f])):
    _PROTOS.update({
        _fam + "_new": (_vp, [_vp]), _fam + "_del": (None, [_vp]), _fam + "_setupConnections": (None, _setup),
        _fam + "_apply": (None, [_vp, _vp, _i]), _fam + "_flush": (None, [_vp, _vp, _i]),
        _fam + "_reset": (None, [_vp]), _fam + "_set_compression_ratio": (None, [_vp, _f]),
    })
_bound = None


def libcomprex():
    global _bound
    if _bound is None:
        L = _lib.lib()
        for name, (res, args) in _PROTOS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _bound = L
    return _bound


def _raise_if_failed():
    msg = libcomprex().Comprex_lastError()
    if msg:
        raise RuntimeError(msg.decode())


def _ptr_size(vector):
    """(address, element count) of a float32 numpy array or CUDA tensor."""
    if isinstance(vector, np.ndarray):
        assert vector.dtype == np.float32 and vector.flags["C_CONTIGUOUS"] and vector.ndim == 1
        return vector.ctypes.data, vector.size
    assert vector.dtype.is_floating_point and vector.element_size() == 4 and vector.is_contiguous()
    return vector.data_ptr(), vector.numel()


class Getable(object):
    def get(self):
        return self.obj

    def _release(self, symbol):
        """Calls the C destructor once; silent when the interpreter is already tearing the module down."""
        obj = getattr(self, "obj", None)
        if not obj:
            return
        self.obj = None
        try:
            getattr(libcomprex(), symbol)(obj)
        except TypeError:  # module globals are gone at interpreter exit
            pass


class GaspiEnvironment(Getable):
    def __init__(self, segment_size=1 << 20):
        self.obj = libcomprex().GaspiEnvironment_new(int(segment_size))
        _raise_if_failed()

    def __del__(self):
        self._release("GaspiEnvironment_del")

    def get_rank(self):
        return libcomprex().GaspiEnvironment_get_rank(self.obj)

    def get_ranks(self):
        return libcomprex().GaspiEnvironment_get_ranks(self.obj)

    def set_rank(self, rank, ranks):
        """Not in the reference: which simulated rank the following calls act as."""
        libcomprex().GaspiEnvironment_set_rank(self.obj, rank, ranks)
        _raise_if_failed()

    def set_blocking(self, blocking, timeout_s=60.0):
        """Not in the reference: one host thread per rank; receives wait for their message."""
        libcomprex().GaspiEnvironment_set_blocking(self.obj, int(blocking), float(timeout_s))

    def set_user_stream(self, stream):
        """Not in the reference: the stream the calling thread's device vectors live on (a
        torch.cuda.Stream, a raw hipStream_t as an int, or None for the null stream).  Every exchange
        call joins its object's own stream with it on entry and on exit."""
        raw = getattr(stream, "cuda_stream", stream)
        libcomprex().GaspiEnvironment_set_user_stream(self.obj, C.c_void_p(raw or None))

    def barrier(self):
        libcomprex().GaspiEnvironment_barrier(self.obj)

    def flush(self):
        libcomprex().GaspiEnvironment_flush(self.obj)


class Comprex(Getable):
    def __init__(self, gaspi_env, size, size_factor=1.0):
        self.size = size
        self.env = gaspi_env  # keeps the channel registry alive
        self.obj = libcomprex().Comprex_new(gaspi_env.get(), size, size_factor)
        _raise_if_failed()

    def __del__(self):
        self._release("Comprex_del")

    def setThreshold(self, threshold):
        libcomprex().Comprex_setThreshold(self.obj, threshold.get())
        _raise_if_failed()

    def setCompressor(self, compressor):
        libcomprex().Comprex_setCompressor(self.obj, compressor.get())
        _raise_if_failed()

    def getSize(self):
        return self.size

    def resetRests(self):
        libcomprex().Comprex_resetRests(self.obj)
        _raise_if_failed()

    def flushRests(self):
        libcomprex().Comprex_flushRests(self.obj)
        _raise_if_failed()

    def getRests(self, out=None):
        res = np.ndarray([self.size], dtype=np.float32) if out is None else out
        p, n = _ptr_size(res)
        libcomprex().Comprex_getRests(self.obj, p, n)
        _raise_if_failed()
        return res

    def writeRemote(self, vector):
        if isinstance(vector, np.ndarray) and vector.dtype != np.float32:
            vector = np.array(vector, dtype=np.float32)
        p, n = _ptr_size(vector)
        libcomprex().Comprex_writeRemote(self.obj, p, n)
        _raise_if_failed()

    def readRemote(self, out=None):
        res = np.ndarray([self.size], dtype=np.float32) if out is None else out
        p, n = _ptr_size(res)
        libcomprex().Comprex_readRemote(self.obj, p, n)
        _raise_if_failed()
        return res

    def readRemote_add(self, vector):
        p, n = _ptr_size(vector)
        libcomprex().Comprex_readRemote_add(self.obj, p, n)
        _raise_if_failed()
        return vector

    def connectTo(self, srcRank, targRank, tag):
        libcomprex().Comprex_connectTo(self.obj, srcRank, targRank, tag)
        _raise_if_failed()

    def connectTx(self, Rank, tag):
        libcomprex().Comprex_connectTx(self.obj, Rank, tag)
        _raise_if_failed()

    def connectRx(self, Rank, tag):
        libcomprex().Comprex_connectRx(self.obj, Rank, tag)
        _raise_if_failed()


class ThresholdNone(Getable):
    def __init__(self):
        self.obj = libcomprex().ThresholdNone_new()

    def __del__(self):
        self._release("ThresholdNone_del")


class ThresholdConst(Getable):
    def __init__(self, thresh):
        self.obj = libcomprex().ThresholdConst_new(thresh)
        _raise_if_failed()

    def __del__(self):
        self._release("ThresholdConst_del")

    def getThreshold(self):
        return libcomprex().ThresholdConst_getThreshold(self.obj)


class ThresholdTopK(Getable):
    def __init__(self, topK):
        self.obj = libcomprex().ThresholdTopK_new(topK)
        _raise_if_failed()

    def __del__(self):
        self._release("ThresholdTopK_del")

    def getThreshold(self):
        return libcomprex().ThresholdTopK_getThreshold(self.obj)


class CompressorNone(Getable):
    def __init__(self):
        self.obj = libcomprex().CompressorNone_new()

    def __del__(self):
        self._release("CompressorNone_del")


class CompressorRLE(Getable):
    def __init__(self):
        self.obj = libcomprex().CompressorRLE_new()

    def __del__(self):
        self._release("CompressorRLE_del")


class CompressorIndexPairs(Getable):
    def __init__(self):
        self.obj = libcomprex().CompressorIndexPairs_new()

    def __del__(self):
        self._release("CompressorIndexPairs_del")


###########################
# Compressed allreduce schedules (allreduce.py:175-355 of the reference)
###########################
class _ComprexAllreduce(Getable):
    _family = None

    def __init__(self, gaspi_env):
        self.env = gaspi_env
        self.size = None
        self.obj = getattr(libcomprex(), self._family + "_new")(gaspi_env.get())
        _raise_if_failed()

    def __del__(self):
        self._release(self._family + "_del")

    def apply(self, vector):
        """In place on `vector` (float32 numpy array or CUDA tensor); returns it."""
        p, n = _ptr_size(vector)
        getattr(libcomprex(), self._family + "_apply")(self.obj, p, n)
        _raise_if_failed()
        return vector

    def flush(self, vector):
        p, n = _ptr_size(vector)
        getattr(libcomprex(), self._family + "_flush")(self.obj, p, n)
        _raise_if_failed()
        return vector

    def reset(self):
        getattr(libcomprex(), self._family + "_reset")(self.obj)
        _raise_if_failed()

    def set_compression_ratio(self, compression_ratio):
        getattr(libcomprex(), self._family + "_set_compression_ratio")(self.obj, compression_ratio)
        _raise_if_failed()

    def getSize(self):
        return self.size


class Comprex_AllToOneAllreduce(_ComprexAllreduce):
    _family = "Comprex_AllToOneAllreduce"

    def setup_connections(self, size, tag, chiefRank, compression_ratio, size_factor=1.0):
        self.size = size
        libcomprex().Comprex_AllToOneAllreduce_setupConnections(self.obj, size, tag, chiefRank, compression_ratio,
                                                               size_factor)
        _raise_if_failed()


class Comprex_RingAllreduce(_ComprexAllreduce):
    _family = "Comprex_RingAllreduce"

    def setup_connections(self, size, tag, compression_ratio, size_factor=1.0):
        self.size = size
        libcomprex().Comprex_RingAllreduce_setupConnections(self.obj, size, tag, compression_ratio, size_factor)
        _raise_if_failed()


class Comprex_BigRingAllreduce(_ComprexAllreduce):
    _family = "Comprex_BigRingAllreduce"

    def setup_connections(self, size, tag, compression_ratio, size_factor=1.0):
        self.size = size
        libcomprex().Comprex_BigRingAllreduce_setupConnections(self.obj, size, tag, compression_ratio, size_factor)
        _raise_if_failed()
