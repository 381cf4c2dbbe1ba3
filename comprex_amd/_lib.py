"""Loads libcomprex_gfx950.so (built in-tree by comprex_amd/csrc/Makefile) and declares
the cx_* prototypes of include/comprex_gfx950.h.  There is no fallback: a missing
library is an error."""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# COMPREX_GFX950_LIB selects another build of the same library (e.g. one made with other flags)
LIB_PATH = os.environ.get("COMPREX_GFX950_LIB") or os.path.join(_HERE, "lib", "libcomprex_gfx950.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

CX_F32, CX_F64, CX_I32 = 0, 1, 2
(CX_OK, CX_ERR_INVALID, CX_ERR_SIZE_MISMATCH, CX_ERR_MSG_TOO_LARGE, CX_ERR_CAPACITY, CX_ERR_INDEX,
 CX_ERR_HIP, CX_ERR_INTERNAL, CX_ERR_TOPK) = range(9)


class ComprexError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("[cx status %d] %s" % (code, text))
        self.code = code


def build(jobs=8):
    """Compile the HIP library for gfx950 (hipcc cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", CSRC_DIR, "-j%d" % jobs, "all"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `make -C comprex_amd/csrc` "
                          "(or __graft_entry__.build()); there is no CPU fallback" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    vp, i, f, ll = C.c_void_p, C.c_int, C.c_float, C.c_longlong
    protos = {
        "cx_last_error": (C.c_char_p, []),
        "cx_abi_version": (i, []),
        "cx_device_count": (i, []),
        "cx_pointer_on_device": (i, [vp]),
        "cx_device_alloc": (i, [C.POINTER(vp), C.c_size_t]),
        "cx_device_free": (i, [vp]),
        "cx_copy": (i, [vp, vp, vp, C.c_size_t]),
        "cx_copy_counted": (i, [vp, vp, vp, vp, ll]),
        "cx_create": (i, [C.POINTER(vp), vp]),
        "cx_destroy": (i, [vp]),
        "cx_set_stream": (i, [vp, vp]),
        "cx_synchronize": (i, [vp]),
        "cx_get_stream": (vp, [vp]),
        "cx_stream_create": (i, [C.POINTER(vp)]),
        "cx_stream_create_blocking": (i, [C.POINTER(vp)]),
        "cx_stream_destroy": (i, [vp]),
        "cx_stream_synchronize": (i, [vp]),
        "cx_event_create": (i, [C.POINTER(vp)]),
        "cx_event_destroy": (i, [vp]),
        "cx_event_record": (i, [vp, vp]),
        "cx_stream_wait_event": (i, [vp, vp]),
        "cx_set_option": (i, [vp, C.c_char_p, i]),
        "cx_profile_read": (i, [vp, C.POINTER(C.c_float), i, C.POINTER(i)]),
        "cx_topk_subsamples": (i, [f, i, f]),
        "cx_topk_pos": (i, [C.c_size_t, f]),
        "cx_topk_threshold": (i, [vp, i, vp, vp, i, i, f, i, f, vp, vp]),
        "cx_topk_threshold_indexed": (i, [vp, i, vp, vp, i, vp, i, f, vp, vp]),
        "cx_threshold_slot": (vp, [vp]),
        "cx_ip_compress": (i, [vp, i, vp, ll, vp, vp, i, vp, vp, vp, C.POINTER(i)]),
        "cx_ip_compress_noalloc": (i, [vp, i, vp, ll, vp, vp, i, vp, vp, vp]),
        "cx_noalloc_max_elements": (ll, []),
        "cx_reserve": (i, [vp, i, i, C.c_uint]),
        "cx_ip_compress_topk": (i, [vp, i, vp, ll, vp, vp, i, C.c_float, vp, vp, C.POINTER(i)]),
        "cx_ip_write_step": (i, [vp, i, vp, ll, vp, vp, i, C.c_float, i, C.c_float, vp, i, vp, vp, C.POINTER(i)]),
        "cx_get_option": (i, [vp, C.c_char_p, C.POINTER(i)]),
        "cx_rle_compress": (i, [vp, i, vp, ll, vp, vp, i, vp, vp, vp, C.POINTER(i)]),
        "cx_rle_decompress": (i, [vp, i, vp, i, vp, C.POINTER(i)]),
        "cx_rle_add": (i, [vp, i, vp, i, vp]),
        "cx_ip_decompress": (i, [vp, i, vp, i, vp, C.POINTER(i)]),
        "cx_ip_add": (i, [vp, i, vp, i, vp, i]),
        "cx_ip_reduce": (i, [vp, i, vp, i, C.POINTER(vp), i, i, i]),
        "cx_zero": (i, [vp, i, vp, i]),
        "cx_add_vec": (i, [vp, i, vp, vp, i]),
        "cx_threshold_apply": (i, [vp, i, vp, vp, vp, i, vp, vp]),
    }
    for name, (res, args) in protos.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def check(rc):
    if rc != CX_OK:
        raise ComprexError(rc, lib().cx_last_error().decode())
