"""ctypes doorway onto the CPU checker libraries.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``; the product package never imports it.

``Oracle()``      -> liboracle.so, the plain-C restatement (``cxo_*`` symbols)
``Oracle(ref=True)`` -> _ref/libref.so, the reference's own headers behind an
                     extern "C" shim (``cxr_*`` symbols); present only where it was
                     built from the reference tree.

Both expose the same methods; arrays are 1-D contiguous numpy arrays of dtype
float32 / float64 / int32, messages are ``np.uint8`` buffers.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SFX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64", np.dtype(np.int32): "i32"}
_CT = {"f32": C.c_float, "f64": C.c_double, "i32": C.c_int}


def build():
    """Compile liboracle.so (and _ref/libref.so when the reference tree is here)."""
    subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)


def ref_available():
    return os.path.exists(os.path.join(_HERE, "_ref", "libref.so"))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self, ref=False):
        self.ref = ref
        path = os.path.join(_HERE, "_ref", "libref.so") if ref else os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            if ref:
                raise FileNotFoundError(path)
            build()
        self.lib = C.CDLL(path)
        self.p = "cxr_" if ref else "cxo_"
        self.kind = "reference" if ref else "port"

    # ---- helpers -------------------------------------------------------
    def _f(self, name, restype, *argtypes):
        fn = getattr(self.lib, self.p + name)
        fn.restype = restype
        fn.argtypes = list(argtypes)
        return fn

    @staticmethod
    def _sfx(a):
        a = np.asarray(a)
        assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
        return _SFX[a.dtype]

    # ---- host arithmetic ----------------------------------------------
    def calc_subsamples(self, topK, default_subsamples=1000, subsample_factor=10.0):
        return self._f("calc_subsamples", C.c_int, C.c_float, C.c_int, C.c_float)(
            topK, default_subsamples, subsample_factor)

    def topk_pos(self, m, topK):
        assert not self.ref
        return self._f("topk_pos", C.c_int, C.c_size_t, C.c_float)(m, topK)

    def strided_pos(self, i, n, subsamples):
        assert not self.ref
        return self._f("strided_pos", C.c_int, C.c_int, C.c_int, C.c_int)(i, n, subsamples)

    # ---- thresholds ---------------------------------------------------
    def calc_threshold(self, vec, topK):
        s = self._sfx(vec)
        scratch = vec.copy()
        return self._f("calc_threshold_" + s, _CT[s], C.c_void_p, C.c_size_t, C.c_float)(
            _ptr(scratch), scratch.size, topK)

    def topk_prepare(self, vec, topK, default_subsamples=1000, subsample_factor=10.0):
        s = self._sfx(vec)
        return self._f("topk_prepare_" + s, _CT[s], C.c_void_p, C.c_int, C.c_float, C.c_int, C.c_float)(
            _ptr(vec), vec.size, topK, default_subsamples, subsample_factor)

    def topk_prepare_with(self, vec, add_vec, topK, default_subsamples=1000, subsample_factor=10.0):
        s = self._sfx(vec)
        err = C.c_int(0)
        thr = self._f("topk_prepare_with_" + s, _CT[s], C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                      C.c_float, C.c_int, C.c_float, C.POINTER(C.c_int))(
            _ptr(vec), vec.size, _ptr(add_vec), add_vec.size, topK, default_subsamples,
            subsample_factor, C.byref(err))
        if err.value:
            raise RuntimeError("vector sizes must be the same!")
        return thr

    def topk_prepare_indexed(self, vec, add_vec, idx, topK):
        assert not self.ref
        s = self._sfx(vec)
        idx = np.ascontiguousarray(idx, dtype=np.int32)
        return self._f("topk_prepare_indexed_" + s, _CT[s], C.c_void_p, C.c_void_p, C.c_void_p,
                       C.c_int, C.c_float)(_ptr(vec), _ptr(add_vec), _ptr(idx), idx.size, topK)

    def threshold_apply(self, vec, thr):
        s = self._sfx(vec)
        out = np.empty_like(vec)
        self._f("threshold_apply_" + s, None, C.c_void_p, C.c_void_p, C.c_int, _CT[s])(
            _ptr(out), _ptr(vec), vec.size, thr)
        return out

    def threshold_apply_split(self, vec, thr):
        s = self._sfx(vec)
        hi, lo = np.empty_like(vec), np.empty_like(vec)
        self._f("threshold_apply_split_" + s, None, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, _CT[s])(
            _ptr(hi), _ptr(lo), _ptr(vec), vec.size, thr)
        return hi, lo

    def topk_apply(self, vec, topK):
        """ThresholdTopK(topK).apply (reference shim only): (masked copy, threshold)."""
        assert self.ref
        s = self._sfx(vec)
        out = np.empty_like(vec)
        thr = self._f("topk_apply_" + s, _CT[s], C.c_void_p, C.c_void_p, C.c_int, C.c_float)(
            _ptr(out), _ptr(vec), vec.size, topK)
        return out, thr

    # ---- IndexPairs codec --------------------------------------------
    @staticmethod
    def message_capacity(n, dtype):
        return 8 + n * (4 + np.dtype(dtype).itemsize)

    def ip_compress(self, data, update, thr, out=None):
        """data and/or update (update is modified in place).  Returns the message bytes."""
        ref_arr = data if data is not None else update
        s = self._sfx(ref_arr)
        n = ref_arr.size
        if out is None:
            out = np.zeros(self.message_capacity(n, ref_arr.dtype), dtype=np.uint8)
        nbytes = self._f("ip_compress_" + s, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, _CT[s])(
            _ptr(out), _ptr(data), _ptr(update), n, thr)
        return out[:nbytes]

    def ip_compress_add_update(self, update, data, thr):
        s = self._sfx(update)
        out = np.zeros(self.message_capacity(max(update.size, data.size), update.dtype), dtype=np.uint8)
        nbytes = self._f("ip_compress_add_update_" + s, C.c_int, C.c_void_p, C.c_void_p, C.c_int,
                         C.c_void_p, C.c_int, _CT[s])(
            _ptr(out), _ptr(update), update.size, _ptr(data), data.size, thr)
        if nbytes == -2:
            raise RuntimeError("Compressor: Update vector size (%d) is not equal data vector size (%d)!"
                               % (update.size, data.size))
        return out[:nbytes]

    def ip_decompress(self, msg, out):
        s = self._sfx(out)
        msg = np.ascontiguousarray(msg, dtype=np.uint8)
        r = self._f("ip_decompress_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p)(
            _ptr(out), out.size, _ptr(msg))
        if r < 0:
            raise RuntimeError("Decompression vector size is bigger than output buffer!")
        return r

    def ip_add(self, msg, out):
        s = self._sfx(out)
        msg = np.ascontiguousarray(msg, dtype=np.uint8)
        r = self._f("ip_add_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p)(_ptr(out), out.size, _ptr(msg))
        if r < 0:
            raise RuntimeError("Decompression vector size is bigger than output buffer!")

    # ---- run-length codec ---------------------------------------------
    @staticmethod
    def rle_capacity(n, dtype):
        return 16 + n * np.dtype(dtype).itemsize + 4 * (n + 1)

    def rle_compress(self, data, update, thr, out=None):
        """data and/or update (update is modified in place).  Returns the message bytes.  With
        ref=True this is the reference's encoder, which is only sound when every element is sent."""
        ref_arr = data if data is not None else update
        s = self._sfx(ref_arr)
        n = ref_arr.size
        if out is None:
            out = np.zeros(self.rle_capacity(n, ref_arr.dtype) + 8 * n, dtype=np.uint8)
        nbytes = self._f("rle_compress_" + s, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, _CT[s])(
            _ptr(out), _ptr(data), _ptr(update), n, thr)
        return out[:nbytes]

    def rle_decompress(self, msg, out):
        s = self._sfx(out)
        msg = np.ascontiguousarray(msg, dtype=np.uint8)
        r = self._f("rle_decompress_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p)(
            _ptr(out), out.size, _ptr(msg))
        if r < 0:
            raise RuntimeError("Decompression vector size is bigger than output buffer!")
        return r

    def rle_add(self, msg, out):
        s = self._sfx(out)
        msg = np.ascontiguousarray(msg, dtype=np.uint8)
        r = self._f("rle_add_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p)(_ptr(out), out.size, _ptr(msg))
        if r < 0:
            raise RuntimeError("Decompression vector size is bigger than output buffer!")

    # ---- dense codec ---------------------------------------------------
    def none_compress(self, data, update):
        """CompressorNone: int32 n, then the values (update is modified in place)."""
        ref_arr = data if data is not None else update
        s = self._sfx(ref_arr)
        out = np.zeros(4 + ref_arr.size * ref_arr.itemsize, dtype=np.uint8)
        nbytes = self._f("none_compress_" + s, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int)(
            _ptr(out), _ptr(data), _ptr(update), ref_arr.size)
        return out[:nbytes]

    def none_decompress(self, msg, out):
        s = self._sfx(out)
        msg = np.ascontiguousarray(msg, dtype=np.uint8)
        r = self._f("none_decompress_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p)(_ptr(out), out.size, _ptr(msg))
        if r < 0:
            raise RuntimeError("Decompression vector size is bigger than output buffer!")
        return r

    def none_add(self, msg, out):
        s = self._sfx(out)
        msg = np.ascontiguousarray(msg, dtype=np.uint8)
        r = self._f("none_add_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p)(_ptr(out), out.size, _ptr(msg))
        if r < 0:
            raise RuntimeError("Decompression vector size is bigger than output buffer!")

    def fast_comprex(self, n, dtype, codec="ip", size_factor=3.0, topK=0.01, default_subsamples=1000,
                     subsample_factor=10.0):
        """A FastComprEx sender (restatement only): see FastChannel."""
        assert not self.ref
        return FastChannel(self, n, dtype, codec, size_factor, topK, default_subsamples, subsample_factor)

    # ---- channel level (restatement only) ----------------------------
    def add_rests(self, data, rests):
        assert not self.ref
        s = self._sfx(data)
        self._f("add_rests_" + s, None, C.c_void_p, C.c_void_p, C.c_int)(_ptr(data), _ptr(rests), data.size)

    def write_remote(self, rests, vec, topK, default_subsamples=1000, subsample_factor=10.0,
                     send_size_bytes=False):
        """Returns (buffer bytes incl. optional prefix, threshold)."""
        assert not self.ref
        s = self._sfx(vec)
        buf = np.zeros(4 + self.message_capacity(vec.size, vec.dtype), dtype=np.uint8)
        thr = _CT[s]()
        nbytes = self._f("write_remote_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                         C.c_int, C.c_float, C.c_int, C.c_float, C.c_void_p)(
            _ptr(buf), int(send_size_bytes), _ptr(rests), _ptr(vec), vec.size, topK,
            default_subsamples, subsample_factor, C.byref(thr))
        return buf[:nbytes + (4 if send_size_bytes else 0)], thr.value

    def write_remote_noresidual(self, vec, topK, default_subsamples=1000, subsample_factor=10.0,
                                send_size_bytes=False):
        assert not self.ref
        s = self._sfx(vec)
        buf = np.zeros(4 + self.message_capacity(vec.size, vec.dtype), dtype=np.uint8)
        thr = _CT[s]()
        nbytes = self._f("write_remote_noresidual_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p,
                         C.c_int, C.c_float, C.c_int, C.c_float, C.c_void_p)(
            _ptr(buf), int(send_size_bytes), _ptr(vec), vec.size, topK, default_subsamples,
            subsample_factor, C.byref(thr))
        return buf[:nbytes + (4 if send_size_bytes else 0)], thr.value

    def flush_rests(self, rests, send_size_bytes=False):
        assert not self.ref
        s = self._sfx(rests)
        buf = np.zeros(4 + self.message_capacity(rests.size, rests.dtype), dtype=np.uint8)
        nbytes = self._f("flush_rests_" + s, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int)(
            _ptr(buf), int(send_size_bytes), _ptr(rests), rests.size)
        return buf[:nbytes + (4 if send_size_bytes else 0)]


class FastChannel:
    """Sender side of FastComprEx (comprEx.tpp:366-493) on the restatement: residual, the two
    halves of the send buffer, sizeBytes / phase / is_first and the threshold's current value.
    Every call returns the bytes it hands to the transport."""
    CODECS = {"ip": 0, "rle": 1, "none": 2}

    def __init__(self, oracle, n, dtype, codec, size_factor, topK, ds, sf):
        self.o, self.n, self.dt, self.codec = oracle, n, np.dtype(dtype), self.CODECS[codec]
        self.s = _SFX[self.dt]
        self.rests = np.zeros(n, self.dt)
        # doublebuffer_offset of the reference is size*size_factor*sizeof(T); the restatement's
        # buffers are sized for the largest message of any codec
        self.half_bytes = max(int(n * size_factor * self.dt.itemsize), 64 + n * (8 + self.dt.itemsize))
        self.halves = np.zeros(2 * self.half_bytes, np.uint8)
        self.st = np.array([0, 0, 1], np.int32)  # sizeBytes, phase, is_first
        self.thr = _CT[self.s](0)
        self.topK, self.ds, self.sf = topK, ds, sf

    def write_remote(self, vec):
        sent = np.zeros(self.half_bytes, np.uint8)
        nb = self.o._f("fast_write_remote_" + self.s, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                       C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_float, C.c_void_p)(
            self.codec, _ptr(self.rests), self.n, _ptr(vec), _ptr(self.halves), self.half_bytes, _ptr(self.st),
            C.byref(self.thr), self.topK, self.ds, self.sf, _ptr(sent))
        return sent[:nb]

    def flush_rests(self):
        sent = np.zeros(self.half_bytes, np.uint8)
        nb = self.o._f("fast_flush_rests_" + self.s, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                       C.c_void_p, C.c_void_p)(
            self.codec, _ptr(self.rests), self.n, _ptr(self.halves), self.half_bytes, _ptr(self.st), _ptr(sent))
        return sent[:nb]

    def write_remote_same_as(self, other):
        sent = np.zeros(self.half_bytes, np.uint8)
        nb = self.o._f("fast_write_remote_same_as_" + self.s, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p,
                       C.c_int, C.c_void_p, _CT[self.s], C.c_void_p, C.c_void_p, C.c_void_p)(
            self.codec, _ptr(self.rests), self.n, _ptr(self.halves), self.half_bytes, _ptr(self.st), self.thr,
            _ptr(other.halves), _ptr(other.st), _ptr(sent))
        return sent[:nb]


def parse_message(msg, dtype):
    """Split an IndexPairs message into (n, k, indices int32[k], values dtype[k])."""
    msg = np.ascontiguousarray(msg, dtype=np.uint8)
    n, k = np.frombuffer(msg[:8].tobytes(), dtype=np.int32)
    dt = np.dtype(dtype)
    rec = np.dtype([("i", np.int32), ("v", dt)], align=False)
    body = np.frombuffer(msg[8:8 + int(k) * rec.itemsize].tobytes(), dtype=rec)
    return int(n), int(k), body["i"].copy(), body["v"].copy()


def reorder_bound(msgs, dtype, n, base=None):
    """How far two floating-point sums of the same contributions can lie apart when only the ORDER
    of the additions differs (rank order against whatever order atomics take), per element.

    Element i receives c_i contributions v_1..v_c (plus base[i] when given), summed from a start
    that is one of the terms (or from zero, whose first addition is exact): c_i - 1 (with a base:
    c_i) rounded additions.  Each ordering's result differs from the exact sum by at most
    gamma_m * sum|v|, gamma_m = m*u / (1 - m*u), m the number of rounded additions, u = eps/2 the unit
    roundoff (Higham, Accuracy and Stability of Numerical Algorithms, section 4.2); two orderings
    differ by at most twice that.  An element with a single contribution and no base has bound 0:
    both paths must give the same bits there.  Computed in float64 from the messages alone."""
    dt = np.dtype(dtype)
    u = float(np.finfo(dt).eps) / 2.0
    mass = np.zeros(n, np.float64)
    count = np.zeros(n, np.int64)
    for m in msgs:
        _, _, idx, val = parse_message(np.asarray(m), dt)
        np.add.at(mass, idx, np.abs(val.astype(np.float64)))
        np.add.at(count, idx, 1)
    rounded = np.maximum(count - 1, 0)
    if base is not None:
        mass += np.abs(np.asarray(base, np.float64))
        rounded = count
    gamma = rounded * u / (1.0 - rounded * u)
    # the bound itself is evaluated in float64: one part in 2^40 of slack covers its own rounding
    return 2.0 * gamma * mass * (1.0 + 2.0 ** -40)
