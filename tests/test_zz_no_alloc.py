"""cx_ip_compress_noalloc (scratch in a static device array) against cx_ip_compress (scratch the
handle allocates) AND against the CPU checker, through the C ABI: same message bytes, size prefix
and residual, bit for bit, on calls in a row, the later ones with smaller inputs, so that the static
array still holds an earlier call's contents when they run; for every tile shape, for sub-vectors at
odd offsets (the scalar path) and at the largest size the entry point takes."""
import ctypes as C

import numpy as np
import pytest
import torch

from comprex_amd import _lib

pytestmark = pytest.mark.gpu

_DT = {torch.float32: _lib.CX_F32, torch.float64: _lib.CX_F64, torch.int32: _lib.CX_I32}
_CT = {torch.float32: C.c_float, torch.float64: C.c_double, torch.int32: C.c_int}


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _inputs(rng, n, dtype):
    if dtype == torch.int32:
        g = rng.integers(-1000, 1000, n).astype(np.int32)
        r = rng.integers(-300, 300, n).astype(np.int32)
    else:
        np_dt = np.float32 if dtype == torch.float32 else np.float64
        g = rng.standard_normal(n).astype(np_dt)
        r = (0.3 * rng.standard_normal(n)).astype(np_dt)
    return torch.from_numpy(g).cuda(), torch.from_numpy(r).cuda()


def _run(L, h, entry, dtype, data, update, thr, cap_bytes):
    """One compress through `entry`; returns (message bytes, prefix, residual bytes)."""
    msg = torch.full((cap_bytes,), 0xEE, dtype=torch.uint8, device="cuda")
    prefix = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    hthr = _CT[dtype](thr)
    n = (data if data is not None else update).numel()
    args = [h, _DT[dtype], _p(msg), cap_bytes, _p(data), _p(update), n, C.byref(hthr), None, _p(prefix)]
    if entry == "cx_ip_compress":
        args.append(None)
    _lib.check(getattr(L, entry)(*args))
    _lib.check(L.cx_synchronize(h))
    nbytes = int(prefix.item())
    hdr = msg[:8].view(torch.int32).cpu().numpy()
    esize = (data if data is not None else update).element_size()
    assert int(hdr[0]) == n and nbytes == 8 + int(hdr[1]) * (4 + esize)
    return msg[:nbytes].cpu().numpy().tobytes(), nbytes, None if update is None else update.cpu().numpy().tobytes()


def _checker(oracle, data, update, thr):
    """The same compress through the CPU checker: (message bytes, byte count, residual bytes)."""
    d = None if data is None else data.cpu().numpy()
    u = None if update is None else update.cpu().numpy().copy()
    msg = oracle.ip_compress(d, u, thr)
    return msg.tobytes(), msg.size, None if u is None else u.tobytes()


@pytest.mark.parametrize("offset", [0, 1])
@pytest.mark.parametrize("items", [2, 4, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.int32])
def test_noalloc_matches_allocating_entry_point_and_checker_on_consecutive_calls(oracle, dtype, items, offset):
    """offset 1: the vectors start one element behind an aligned address (scalar loads, the tile
    shape of that path); items: 16-byte loads per lane and tile of the vector path."""
    L = _lib.lib()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    h = C.c_void_p()
    _lib.check(L.cx_create(C.byref(h), C.c_void_p(stream.cuda_stream)))
    try:
        _lib.check(L.cx_set_option(h, b"compact_items", items))
        rng = np.random.default_rng(5)
        esize = torch.empty((), dtype=dtype).element_size()
        # a large call, then a smaller one (odd length: ragged last tile), then a dense flush-like call
        cases = [(3_000_017, 2.2, "fused"), (70_001, 1.5, "fused"), (70_001, 0.0, "update"), (4_099, 0.7, "data")]
        for n, thr, mode in cases:
            if dtype == torch.int32:
                thr = int(thr * 400)
            g, r = _inputs(rng, n + offset, dtype)
            g, r = g[offset:], r[offset:]
            cap = 8 + n * (4 + esize)
            want_in = (g if mode != "update" else None, r.clone() if mode != "data" else None)
            got_in = (g if mode != "update" else None, r.clone() if mode != "data" else None)
            if offset:  # clone() realigns: keep the odd start
                hold_w, hold_g = torch.empty(n + 1, dtype=dtype, device="cuda"), torch.empty(n + 1, dtype=dtype, device="cuda")
                if want_in[1] is not None:
                    hold_w[1:].copy_(r), hold_g[1:].copy_(r)
                    want_in, got_in = (want_in[0], hold_w[1:]), (got_in[0], hold_g[1:])
            check_in = (want_in[0], None if want_in[1] is None else want_in[1].clone())
            want = _run(L, h, "cx_ip_compress", dtype, want_in[0], want_in[1], thr, cap)
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            got = _run(L, h, "cx_ip_compress_noalloc", dtype, got_in[0], got_in[1], thr, cap)
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
            ref = _checker(oracle, check_in[0], check_in[1], thr)
            assert got[1] == want[1] == ref[1], (n, mode, got[1], want[1], ref[1])
            assert got[0] == want[0], "message differs from the allocating entry point (n=%d, %s)" % (n, mode)
            assert got[0] == ref[0], "message differs from the checker (n=%d, %s)" % (n, mode)
            assert got[2] == want[2] == ref[2], "residual differs (n=%d, %s)" % (n, mode)
            assert want[1] > 8 or thr > 100, "the case selects nothing"
    finally:
        L.cx_destroy(h)


def test_noalloc_largest_fp64_vector_smallest_tiles(oracle):
    """fp64 at exactly cx_noalloc_max_elements() with the smallest tile shape: the case that needs the
    most of the static array (staging slots of 3 words per pair, the most tiles)."""
    L = _lib.lib()
    torch.cuda.set_device(0)
    h = C.c_void_p()
    _lib.check(L.cx_create(C.byref(h), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    try:
        _lib.check(L.cx_set_option(h, b"compact_items", 2))
        n = int(L.cx_noalloc_max_elements())
        rng = np.random.default_rng(6)
        g = torch.from_numpy(rng.standard_normal(n)).cuda()
        r = torch.from_numpy(0.3 * rng.standard_normal(n)).cuda()
        cap = 8 + 12 * (n // 20)
        ref = _checker(oracle, g, r, 2.4)
        got = _run(L, h, "cx_ip_compress_noalloc", torch.float64, g, r, 2.4, cap)
        assert 8 < got[1] == ref[1] and got[0] == ref[0] and got[2] == ref[2]
    finally:
        L.cx_destroy(h)


def test_noalloc_refuses_vectors_beyond_its_limit():
    L = _lib.lib()
    torch.cuda.set_device(0)
    h = C.c_void_p()
    _lib.check(L.cx_create(C.byref(h), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    try:
        limit = L.cx_noalloc_max_elements()
        assert limit == 1 << 24
        n = limit + 1
        g = torch.zeros(n, device="cuda")
        r = torch.ones(n, device="cuda")
        msg = torch.zeros(64, dtype=torch.uint8, device="cuda")
        thr = C.c_float(0.5)
        rc = L.cx_ip_compress_noalloc(h, _lib.CX_F32, _p(msg), 64, _p(g), _p(r), n, C.byref(thr), None, None)
        assert rc == _lib.CX_ERR_INVALID and b"exceed the limit" in L.cx_last_error()
        _lib.check(L.cx_synchronize(h))
        assert bool((r == 1).all()), "a refused call must not touch the residual"
        # exactly at the limit it runs (all ones above 0.5: every element is sent and cleared)
        n = limit
        cap = 8 + 8 * n
        msg = torch.zeros(cap, dtype=torch.uint8, device="cuda")
        prefix = torch.zeros(1, dtype=torch.int32, device="cuda")
        _lib.check(L.cx_ip_compress_noalloc(h, _lib.CX_F32, _p(msg), cap, None, _p(r[:n]), n, C.byref(thr), None,
                                            _p(prefix)))
        _lib.check(L.cx_synchronize(h))
        assert int(prefix.item()) == cap and not bool(r[:n].any()) and float(r[n].item()) == 1.0
        pairs = msg[8:].view(torch.int32).view(-1, 2)
        assert bool((pairs[:, 0] == torch.arange(n, dtype=torch.int32, device="cuda")).all())
    finally:
        L.cx_destroy(h)
