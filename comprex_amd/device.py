"""Thin torch-tensor front end of the cx_* C ABI (include/comprex_gfx950.h).

PyTorch only supplies device memory and the current HIP stream; every operation
below is one call into libcomprex_gfx950.so.  Messages are uint8/int32 CUDA tensors
in the reference's IndexPairs layout (src/compressor.hxx:559-565).
"""
import ctypes as C

import numpy as np
import torch

from . import _lib
from ._lib import CX_F32, CX_F64, CX_I32, ComprexError, check  # noqa: F401

_DT = {torch.float32: CX_F32, torch.float64: CX_F64, torch.int32: CX_I32}
_CT = {torch.float32: C.c_float, torch.float64: C.c_double, torch.int32: C.c_int}


def pair_bytes(dtype):
    return 4 + torch.empty((), dtype=dtype).element_size()


def message_capacity(n, dtype):
    """Bytes of the largest message a vector of n elements can produce."""
    return 8 + n * pair_bytes(dtype)


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _dt(t):
    assert t.is_cuda and t.is_contiguous() and t.dim() == 1, "need 1-D contiguous device tensors"
    return _DT[t.dtype]


class Handle:
    """One compressor clone's scratch + stream (cx_create / cx_destroy)."""

    def __init__(self, stream=None):
        self.lib = _lib.lib()
        self._h = C.c_void_p()
        if stream is None:
            stream = torch.cuda.current_stream()
        self.stream = stream
        check(self.lib.cx_create(C.byref(self._h), C.c_void_p(stream.cuda_stream)))

    def close(self):
        if self._h:
            self.lib.cx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    RESERVE_COMPRESS, RESERVE_THRESHOLD, RESERVE_REDUCE, RESERVE_RLE, RESERVE_ALL = 1, 2, 4, 8, 15

    def reserve(self, n, dtype, paths=7):
        """Sizes the handle's scratch for vectors of up to n elements of `dtype` so that later calls
        on the named paths (an OR of the RESERVE_* bits; default: all but the run-length codec) never
        allocate (cx_reserve)."""
        check(self.lib.cx_reserve(self._h, _DT[dtype], int(n), int(paths)))

    def set_option(self, key, value):
        check(self.lib.cx_set_option(self._h, key.encode(), int(value)))

    def profile_read(self, max_out=1024):
        """Milliseconds of the streaming kernel of each compress since the last read
        (needs set_option("profile_stage", 1)); waits for the stream."""
        buf = (C.c_float * max_out)()
        n = C.c_int(0)
        check(self.lib.cx_profile_read(self._h, buf, max_out, C.byref(n)))
        return [buf[i] for i in range(n.value)]

    def synchronize(self):
        """Waits for the stream; raises the first device-side error recorded since the last call."""
        check(self.lib.cx_synchronize(self._h))

    # ---- thresholds ------------------------------------------------------
    def topk_threshold(self, vec, add_vec, topK, default_subsamples=1000, subsample_factor=10.0,
                       out=None, to_host=True):
        """ThresholdTopK.prepare_with (add_vec given) / prepare (add_vec None)."""
        dt = _dt(vec)
        host = _CT[vec.dtype]() if to_host else None
        check(self.lib.cx_topk_threshold(
            self._h, dt, _p(vec), _p(add_vec), vec.numel(), 0 if add_vec is None else add_vec.numel(),
            C.c_float(topK), int(default_subsamples), C.c_float(subsample_factor), _p(out),
            C.byref(host) if to_host else None))
        return host.value if to_host else None

    def topk_threshold_indexed(self, vec, add_vec, idx, topK, out=None, to_host=True):
        dt = _dt(vec)
        assert idx.dtype == torch.int32 and idx.is_cuda
        host = _CT[vec.dtype]() if to_host else None
        check(self.lib.cx_topk_threshold_indexed(
            self._h, dt, _p(vec), _p(add_vec), vec.numel(), _p(idx), idx.numel(), C.c_float(topK), _p(out),
            C.byref(host) if to_host else None))
        return host.value if to_host else None

    def threshold_slot(self):
        """Raw device address of the handle's own threshold slot."""
        return self.lib.cx_threshold_slot(self._h)

    # ---- codec -------------------------------------------------------------
    def compress(self, out_msg, data, update, thr=None, d_thr=None, size_prefix=None, sync=True):
        """compress / compress_update / compress_add_update by which of data/update is None.
        thr: host scalar; else d_thr: 1-element device tensor; else the handle's slot.
        Returns bytes written when sync, else None."""
        ref = data if data is not None else update
        dt = _DT[ref.dtype] if ref is not None else CX_F32
        n = ref.numel() if ref is not None else 0
        if data is not None and update is not None and data.numel() != update.numel():
            raise ComprexError(_lib.CX_ERR_SIZE_MISMATCH,
                               "Compressor: Update vector size (%d) is not equal data vector size (%d)!"
                               % (update.numel(), data.numel()))
        hthr = None
        if thr is not None:
            hthr = _CT[ref.dtype](thr)
        nbytes = C.c_int(0)
        check(self.lib.cx_ip_compress(
            self._h, dt, _p(out_msg), out_msg.numel() * out_msg.element_size(), _p(data), _p(update), n,
            C.byref(hthr) if hthr is not None else None, _p(d_thr), _p(size_prefix),
            C.byref(nbytes) if sync else None))
        return nbytes.value if sync else None

    def compress_topk(self, out_msg, data, update, topk, d_thr=None, size_prefix=None):
        """Whole-vector ThresholdTopK(topk) on update + data and compress_add_update in one call
        (a single pass over the vectors when they are large).  The threshold is left in d_thr
        (1-element device tensor) or the handle's slot.  Returns bytes written."""
        if data.numel() != update.numel():
            raise ComprexError(_lib.CX_ERR_SIZE_MISMATCH, "vector sizes must be the same!")
        nbytes = C.c_int(0)
        check(self.lib.cx_ip_compress_topk(
            self._h, _dt(update), _p(out_msg), out_msg.numel() * out_msg.element_size(), _p(data), _p(update),
            update.numel(), float(topk), _p(d_thr), _p(size_prefix), C.byref(nbytes)))
        return nbytes.value

    def write_step(self, out_msg, data, update, topk, default_subsamples=1000, subsample_factor=10.0, idx=None,
                   d_thr=None, size_prefix=None, sync=True):
        """ThresholdTopK(topk, default_subsamples, subsample_factor).prepare_with(update, data) and
        compress_add_update in one call (cx_ip_write_step); idx: int32 device tensor of sample
        positions instead of the strided rule.  Returns bytes written when sync."""
        if data.numel() != update.numel():
            raise ComprexError(_lib.CX_ERR_SIZE_MISMATCH, "vector sizes must be the same!")
        nbytes = C.c_int(0)
        check(self.lib.cx_ip_write_step(
            self._h, _dt(update), _p(out_msg), out_msg.numel() * out_msg.element_size(), _p(data), _p(update),
            update.numel(), float(topk), int(default_subsamples), float(subsample_factor), _p(idx),
            0 if idx is None else idx.numel(), _p(d_thr), _p(size_prefix), C.byref(nbytes) if sync else None))
        return nbytes.value if sync else None

    def get_option(self, key):
        v = C.c_int(0)
        check(self.lib.cx_get_option(self._h, key.encode(), C.byref(v)))
        return v.value

    # ---- run-length codec -------------------------------------------------
    def rle_compress(self, out_msg, data, update, thr=None, d_thr=None, size_prefix=None, sync=True):
        """CompressorRLE: as compress(), but |x| >= thr is sent and the message carries values
        and run lengths instead of (index, value) pairs.  Returns bytes written when sync."""
        ref = data if data is not None else update
        if ref is None:
            raise ComprexError(_lib.CX_ERR_INVALID, "Compression needs a valid input vector!")
        if data is not None and update is not None and data.numel() != update.numel():
            raise ComprexError(_lib.CX_ERR_SIZE_MISMATCH,
                               "Compressor: Update vector size (%d) is not equal data vector size (%d)!"
                               % (update.numel(), data.numel()))
        hthr = _CT[ref.dtype](thr) if thr is not None else None
        nbytes = C.c_int(0)
        check(self.lib.cx_rle_compress(
            self._h, _DT[ref.dtype], _p(out_msg), out_msg.numel() * out_msg.element_size(), _p(data), _p(update),
            ref.numel(), C.byref(hthr) if hthr is not None else None, _p(d_thr), _p(size_prefix),
            C.byref(nbytes) if sync else None))
        return nbytes.value if sync else None

    def rle_decompress(self, out, msg):
        """Returns the vector length the message carries (what the reference's decoder returns)."""
        n = C.c_int(0)
        check(self.lib.cx_rle_decompress(self._h, _dt(out), _p(out), out.numel(), _p(msg), C.byref(n)))
        return n.value

    def rle_add(self, out, msg):
        check(self.lib.cx_rle_add(self._h, _dt(out), _p(out), out.numel(), _p(msg)))

    def decompress(self, out, msg, sync=True):
        nbytes = C.c_int(0)
        check(self.lib.cx_ip_decompress(self._h, _dt(out), _p(out), out.numel(), _p(msg),
                                        C.byref(nbytes) if sync else None))
        return nbytes.value if sync else None

    def add(self, out, msg, check_header=True, any_order=False):
        """any_order: look at the indices first (one more wait) and apply a message that is not
        index-sorted pair after pair, as the reference's loop does (CX_ADD_ANY_ORDER)."""
        check(self.lib.cx_ip_add(self._h, _dt(out), _p(out), out.numel(), _p(msg),
                                 2 if any_order else (1 if check_header else 0)))

    def reduce(self, out, msgs, accumulate=False, mode=0, any_order=False):
        arr = (C.c_void_p * len(msgs))(*[m.data_ptr() for m in msgs])
        check(self.lib.cx_ip_reduce(self._h, _dt(out), _p(out), out.numel(), arr, len(msgs),
                                    1 if accumulate else 0, int(mode) | (4 if any_order else 0)))

    # ---- residual maintenance ---------------------------------------------
    def zero(self, v):
        check(self.lib.cx_zero(self._h, _dt(v), _p(v), v.numel()))

    def add_vec(self, data, rests):
        if data.numel() != rests.numel():
            raise ComprexError(_lib.CX_ERR_SIZE_MISMATCH, "Vector of size %d does not match Rests Vector of size %d!"
                               % (data.numel(), rests.numel()))
        check(self.lib.cx_add_vec(self._h, _dt(data), _p(data), _p(rests), data.numel()))

    def threshold_apply(self, vec, thr, split=False):
        high = torch.empty_like(vec)
        low = torch.empty_like(vec) if split else None
        hthr = _CT[vec.dtype](thr)
        check(self.lib.cx_threshold_apply(self._h, _dt(vec), _p(high), _p(low), _p(vec), vec.numel(),
                                          C.byref(hthr), None))
        return (high, low) if split else high


def message_to_numpy(msg, nbytes):
    """First nbytes of a device message tensor as a uint8 numpy array."""
    raw = msg.view(torch.uint8) if msg.dtype != torch.uint8 else msg
    return raw[:nbytes].cpu().numpy()
