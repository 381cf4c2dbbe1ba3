"""Parity of the HIP path with the CPU checker, through the C ABI, on one MI355X.

Bit-exact bar: thresholds, index sets, pair order, residuals, dense outputs of the
rank-ordered reduce.  Tolerance bar (stated where used): the atomic reduce variant.
"""
import sys

import numpy as np
import pytest
import torch

from oracle.pyoracle import parse_message, reorder_bound

pytestmark = pytest.mark.gpu

NP2T = {np.float32: torch.float32, np.float64: torch.float64, np.int32: torch.int32}
DTYPES = [np.float32, np.float64, np.int32]


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def dev():
    from comprex_amd.device import Handle
    assert torch.cuda.is_available(), "these tests need the GPU"
    h = Handle()
    yield h
    h.synchronize()
    h.close()


def _rand(rng, n, dtype, scale=1.0):
    if dtype == np.int32:
        return rng.integers(-1000, 1001, n).astype(np.int32)
    return (rng.standard_normal(n) * scale).astype(dtype)


def _gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _msgbuf(n, dtype, extra=0):
    from comprex_amd.device import message_capacity
    return torch.zeros(message_capacity(n, NP2T[dtype]) + extra, dtype=torch.uint8, device="cuda")


def test_reserve_takes_the_scratch_up_front(oracle):
    """cx_reserve sizes a handle's scratch once; the calls that follow, on vectors up to the reserved
    length, leave the device's free memory where it was (they would otherwise grow their buffers on
    first use) and give the checker's results."""
    from comprex_amd.device import Handle, message_capacity
    n = 9_000_000          # above 2^23: the one-pass exact top-k and its candidate list are in play
    rng = np.random.default_rng(12)
    g_h = rng.laplace(size=n).astype(np.float32)
    g, r = _gpu(g_h), torch.zeros(n, device="cuda")
    msg = torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")
    rle = torch.zeros(16 + 8 * n + 8, dtype=torch.uint8, device="cuda")
    idx = _gpu(np.sort(rng.integers(0, n, 50_000)).astype(np.int32))
    dense = torch.zeros(n, device="cuda")
    def calls(h, check):
        h.set_option("fused_topk", 2)   # the single pass from 2^23 elements on (by default only where it is faster)
        thr = h.topk_threshold_indexed(r, g, idx, np.float32(0.01))
        nbytes = h.compress(msg, g, r)
        if check:
            assert thr == oracle.topk_prepare_indexed(np.zeros(n, np.float32), g_h, idx.cpu().numpy(), np.float32(0.01))
            want = oracle.ip_compress(g_h, np.zeros(n, np.float32), np.float32(thr))
            assert msg[:nbytes].cpu().numpy().tobytes() == want.tobytes()
        h.decompress(dense, msg)
        h.reduce(dense, [msg, msg], accumulate=False, mode=0)
        h.reduce(dense, [msg, msg], accumulate=True, mode=0)
        h.reduce(dense, [msg] * 4, accumulate=False, mode=0)
        h.compress_topk(msg, g, r, np.float32(0.001))
        assert h.get_option("fused_topk_taken") == 1   # the one-pass route, whose candidate list was reserved
        h.rle_compress(rle, g, r, thr=np.float32(thr))
        h.synchronize()
        r.zero_()

    # the runtime places a source file's kernels in device memory on the first launch of one of them:
    # a first handle runs the same calls (growing its own buffers as it goes) and is closed again
    warm = Handle()
    try:
        calls(warm, False)
    finally:
        warm.close()
    h = Handle()
    try:
        with pytest.raises(RuntimeError):
            h.reserve(n, torch.float32, 0)
        with pytest.raises(RuntimeError):
            h.reserve(n, torch.float32, 32)
        h.reserve(n, torch.float32, Handle.RESERVE_ALL)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        calls(h, True)
        assert torch.cuda.mem_get_info()[0] == free_before
    finally:
        h.close()


def test_write_step_equals_prepare_with_then_compress(dev, oracle):
    """cx_ip_write_step = ThresholdTopK(topK, default_subsamples, factor).prepare_with(residual, gradient)
    followed by compress_add_update, in the reference's three sampling modes (strided sample, whole
    vector because the sample would cover it, and caller-given positions), three element types, over
    residual-carrying steps: threshold, message and residual equal the checker's."""
    from comprex_amd.device import message_capacity
    rng = np.random.default_rng(77)
    for dtype in DTYPES:
        tdt = NP2T[dtype]
        for n, topk, ds, indexed in ((100_003, 0.01, 1000, False), (100_003, 0.05, 1 << 20, False),
                                     (1_500_001, 0.002, 1 << 22, False), (300_000, 0.02, 1000, True),
                                     (5, 0.5, 1000, False), (1, 0.5, 1000, False)):
            say("write_step", dtype.__name__, n, topk, ds, indexed)
            r_h = np.zeros(n, dtype)
            r = torch.zeros(n, dtype=tdt, device="cuda")
            buf = torch.zeros(message_capacity(n, tdt), dtype=torch.uint8, device="cuda")
            thr_out = torch.zeros(1, dtype=tdt, device="cuda")
            idx_h = rng.integers(0, n, 20_000).astype(np.int32) if indexed else None
            idx = _gpu(idx_h) if indexed else None
            for step in range(3):
                g_h = (rng.standard_normal(n) * (1000 if dtype == np.int32 else 1)).astype(dtype)
                g = _gpu(g_h)
                nbytes = dev.write_step(buf, g, r, np.float32(topk), ds, 10.0, idx=idx, d_thr=thr_out)
                if indexed:
                    want_thr = oracle.topk_prepare_indexed(r_h, g_h, idx_h, np.float32(topk))
                else:
                    want_thr = oracle.topk_prepare_with(r_h, g_h, np.float32(topk), ds, 10.0)
                want = oracle.ip_compress(g_h, r_h, dtype(want_thr))
                assert thr_out.cpu().numpy()[0] == dtype(want_thr), (dtype.__name__, n, step)
                assert nbytes == want.size and buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
                assert r.cpu().numpy().tobytes() == r_h.tobytes()


# --------------------------------------------------------------------------- K2
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", ["fused", "update", "data"])
def test_compress_matches_oracle(dev, oracle, dtype, mode):
    rng = np.random.default_rng(11)
    sizes = [0, 1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 4095, 4096, 4097, 8193, 100_003, 1_000_003]
    for n in sizes:
        for q in [0.0, 0.9, 0.99, 1.0]:
            say("compress", dtype.__name__, mode, "n", n, "q", q)
            d = _rand(rng, n, dtype)
            u = _rand(rng, n, dtype, 0.5)
            s = u + d if mode == "fused" else (u if mode == "update" else d)
            thr = dtype(0) if (q == 0.0 or n == 0) else dtype(np.quantile(np.abs(s), q))
            dd = d.copy() if mode != "update" else None
            uu = u.copy() if mode != "data" else None
            want = oracle.ip_compress(dd, uu, thr)
            gd = _gpu(d) if mode != "update" else None
            gu = _gpu(u) if mode != "data" else None
            buf = _msgbuf(n, dtype)
            nbytes = dev.compress(buf, gd, gu, thr=thr)
            assert nbytes == want.size
            assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
            if uu is not None:
                assert gu.cpu().numpy().tobytes() == uu.tobytes()
            if gd is not None:
                assert gd.cpu().numpy().tobytes() == d.tobytes()  # data is read-only
    dev.synchronize()


@pytest.mark.parametrize("items", [2, 4, 8])
def test_compress_variants_agree(dev, oracle, items):
    """Every tile size of the compaction kernel gives the same bytes, at densities that stage
    every tile (sparse), defer some (around the 1/8 slot capacity) and defer all (dense)."""
    rng = np.random.default_rng(12)
    n = 3_000_017
    d, u = _rand(rng, n, np.float32), _rand(rng, n, np.float32, 0.3)
    try:
        dev.set_option("compact_items", items)
        for q in [0.0, 0.5, 0.85, 0.875, 0.9, 0.99, 0.9999]:
            say("variants items", items, "q", q)
            thr = np.float32(np.quantile(np.abs(u + d), q)) if q else np.float32(0)
            uu = u.copy()
            want = oracle.ip_compress(d.copy(), uu, thr)
            gu, buf = _gpu(u), _msgbuf(n, np.float32)
            nbytes = dev.compress(buf, _gpu(d), gu, thr=thr)
            assert nbytes == want.size
            assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
            assert gu.cpu().numpy().tobytes() == uu.tobytes()
    finally:
        dev.set_option("compact_items", 0)  # back to the choice by length


def test_compress_clustered_survivors(dev, oracle):
    """Survivors packed into a few tiles (spikes next to each other) while the rest is empty:
    dense tiles are deferred and redone, sparse ones staged, in one message."""
    rng = np.random.default_rng(21)
    n = 1_000_000
    for dtype in DTYPES:
        d = _rand(rng, n, dtype, 0.01) if dtype != np.int32 else rng.integers(-3, 4, n).astype(np.int32)
        for start in (0, 5000, 123_456, n - 3000):
            d[start:start + 3000] = dtype(50)
        d[rng.integers(0, n, 500)] = dtype(-60)
        u = np.zeros(n, dtype)
        uu = u.copy()
        want = oracle.ip_compress(d.copy(), uu, dtype(10))
        gu, buf = _gpu(u), _msgbuf(n, dtype)
        nbytes = dev.compress(buf, _gpu(d), gu, thr=dtype(10))
        assert nbytes == want.size and buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
        assert gu.cpu().numpy().tobytes() == uu.tobytes()


def test_compress_unaligned_pointers_and_prefix(dev, oracle):
    """Sub-vectors at odd offsets (ring segments, src/allreduce.tpp:436-437) and the 4-byte
    sizeBytes prefix (src/comprEx.tpp:184-188) that leaves pairs only 4-byte aligned."""
    rng = np.random.default_rng(13)
    n = 50_001
    for dtype in DTYPES:
        d, u = _rand(rng, n + 3, dtype), _rand(rng, n + 3, dtype, 0.3)
        for off in [1, 2, 3]:
            say("unaligned", dtype.__name__, off)
            thr = dtype(np.quantile(np.abs(u[off:off + n] + d[off:off + n]), 0.98))
            uu = u.copy()
            want = oracle.ip_compress(d[off:off + n].copy(), uu[off:off + n], thr)
            gd, gu = _gpu(d), _gpu(u)
            buf = _msgbuf(n, dtype, extra=8)
            prefix = buf[:4].view(torch.int32)
            nbytes = dev.compress(buf[4:], gd[off:off + n], gu[off:off + n], thr=thr, size_prefix=prefix)
            assert nbytes == want.size and int(prefix.item()) == want.size
            assert buf[4:4 + nbytes].cpu().numpy().tobytes() == want.tobytes()
            assert gu.cpu().numpy().tobytes() == uu.tobytes()  # elements outside the slice untouched too


def test_compress_special_values(dev, oracle):
    d = np.array([1, np.nan, -3, np.inf, -np.inf, 0.5, -0.0, 0.0] * 700, dtype=np.float32)
    u = np.zeros_like(d)
    uu = u.copy()
    want = oracle.ip_compress(d.copy(), uu, np.float32(0.75))
    gu, buf = _gpu(u), _msgbuf(d.size, np.float32)
    nbytes = dev.compress(buf, _gpu(d), gu, thr=0.75)
    assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
    assert gu.cpu().numpy().tobytes() == uu.tobytes()  # NaN stays in the residual, zeros are +0


def test_compress_capacity_and_size_errors(dev):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    d = torch.ones(1000, device="cuda")
    u = torch.zeros(1000, device="cuda")
    small = torch.zeros(8 + 8 * 10, dtype=torch.uint8, device="cuda")
    with pytest.raises(ComprexError) as e:
        dev.compress(small, d, u, thr=0.5)
    assert e.value.code == _lib.CX_ERR_CAPACITY
    # the header announces what was written, and what found no room is still in the residual
    assert small[:8].view(torch.int32).tolist() == [1000, 10]
    pairs = small[8:].view(torch.int32).view(-1, 2)
    assert pairs[:, 0].tolist() == list(range(10)) and small[8:].view(torch.float32).view(-1, 2)[:, 1].tolist() == [1.0] * 10
    assert u[:10].tolist() == [0.0] * 10 and u[10:].tolist() == [1.0] * 990
    big = _msgbuf(1000, np.float32)
    assert dev.compress(big, None, u, thr=0.5) == 8 + 8 * 990 and not bool(u.any())
    # the same through every route that places pairs: tiles deferred for their density (threshold 0:
    # the write pass of a flush), the single-call exact top-k, and the run-length codec
    for n, route in ((50_000, "flush"), (1 << 23, "topk"), (5000, "rle")):
        rng = np.random.default_rng(8)
        g_h = rng.integers(1, 100, n).astype(np.float32) * rng.choice([-1.0, 1.0], n).astype(np.float32)
        r_h = rng.integers(-20, 20, n).astype(np.float32)
        g, r = _gpu(g_h), _gpu(r_h)
        tiny = torch.zeros(8 + 8 * 100, dtype=torch.uint8, device="cuda")
        with pytest.raises(ComprexError) as e:
            if route == "flush":
                dev.compress(tiny, g, r, thr=0.0)
            elif route == "topk":
                dev.set_option("fused_topk", 2)  # the single pass at this length
                try:
                    dev.compress_topk(tiny, g, r, np.float32(0.001))
                finally:
                    dev.set_option("fused_topk", 1)
            else:
                dev.rle_compress(tiny, g, r, thr=1.0)
        assert e.value.code == _lib.CX_ERR_CAPACITY, route
        total = r_h + g_h
        if route == "rle":  # cannot be cut short: an empty message, everything stays behind
            assert tiny[:20].view(torch.int32).tolist() == [n, 0, 1, 0, n]
            sent = np.zeros(n, np.float32)
        else:
            hdr = tiny[:8].view(torch.int32).tolist()
            assert hdr[0] == n and 0 < hdr[1] <= 100
            sent = torch.zeros(n, device="cuda")
            dev.add(sent, tiny)
            sent = sent.cpu().numpy()
        assert np.array_equal(sent + r.cpu().numpy(), total), route  # nothing lost, nothing sent twice
    with pytest.raises(ComprexError) as e:
        dev.compress(_msgbuf(1000, np.float32), d, u[:999], thr=0.5)
    assert e.value.code == _lib.CX_ERR_SIZE_MISMATCH
    dev.synchronize()  # status is clean again


# --------------------------------------------------------------------------- thresholds
@pytest.mark.parametrize("dtype", DTYPES)
def test_topk_threshold_matches_oracle(dev, oracle, dtype):
    rng = np.random.default_rng(14)
    for n in [1, 2, 5, 999, 1000, 1001, 4096, 50_000, 300_001, 2_000_003]:
        for topk, ds, sf in [(0.01, 1000, 10.0), (0.1, 1000, 10.0), (0.001, 1000, 10.0), (0.01, 125, 4.0),
                             (0.02, 1 << 22, 10.0), (1.0, 10, 1.0), (0.5, 1 << 22, 10.0)]:
            say("threshold", dtype.__name__, n, topk, ds, sf)
            v, a = _rand(rng, n, dtype), _rand(rng, n, dtype, 0.3)
            if n > 100:
                v[rng.integers(0, n, n // 7)] = v[3]  # ties
            t = np.float32(topk)
            want_with = oracle.topk_prepare_with(v, a, t, ds, sf)
            want = oracle.topk_prepare(v, t, ds, sf)
            gv, ga = _gpu(v), _gpu(a)
            assert dev.topk_threshold(gv, ga, t, ds, sf) == want_with
            assert dev.topk_threshold(gv, None, t, ds, sf) == want


def test_exact_threshold_on_both_sides_of_the_candidate_pass_limit(dev, oracle):
    """Whole-vector thresholds just below and at the length from which one candidate pass replaces the
    three histogram passes (10 Mi elements): the checker's bits on both sides."""
    rng = np.random.default_rng(29)
    for n in ((10 << 20) - 1, 10 << 20, (10 << 20) + 3):
        v = rng.laplace(size=n).astype(np.float32)
        a = (0.1 * rng.standard_normal(n)).astype(np.float32)
        gv, ga = _gpu(v), _gpu(a)
        for topk in (0.0005, 0.02):
            say("candidate pass limit", n, topk)
            want = oracle.topk_prepare_with(v, a, np.float32(topk), 1 << 24, 10.0)
            assert dev.topk_threshold(gv, ga, np.float32(topk), 1 << 24, 10.0) == want


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_exact_threshold_one_pass_bracket_and_fallbacks(dev, oracle, dtype):
    """Whole-vector (exact top-k) thresholds on vectors large enough for the one-pass path
    (sampled lower bound + candidate collection), including inputs that defeat the bound:
    all-equal magnitudes (candidates overflow), a constant vector with a few outliers, and a
    large topK (bracket not attempted).  Same bits as the checker, with the path on and off."""
    rng = np.random.default_rng(19)
    n = 11_000_001
    ds = 1 << 24  # > n: exact mode
    base = (rng.standard_normal(n) * 3).astype(dtype)
    cases = {
        "gauss": (base, 0.01),
        "gauss_p0.001": (base, 0.001),
        "gauss_p0.3": (base, 0.3),
        "all_equal": (np.full(n, 2.5, dtype), 0.01),
        "two_levels": (np.where(rng.random(n) < 0.004, 7.0, 1.0).astype(dtype), 0.01),
        "ties_at_threshold": (np.round(base).astype(dtype), 0.02),
    }
    add = (rng.standard_normal(n) * 0.1).astype(dtype)
    try:
        for name, (v, topk) in cases.items():
            t = np.float32(topk)
            want_with = oracle.topk_prepare_with(v, add, t, ds, 10.0)
            want = oracle.topk_prepare(v, t, ds, 10.0)
            gv, ga = _gpu(v), _gpu(add)
            for bracket in (1, 0):
                say("exact threshold", dtype.__name__, name, "bracket", bracket)
                dev.set_option("select_bracket", bracket)
                assert dev.topk_threshold(gv, ga, t, ds, 10.0) == want_with
                assert dev.topk_threshold(gv, None, t, ds, 10.0) == want
    finally:
        dev.set_option("select_bracket", 1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_fused_exact_topk_single_pass_and_changes_of_plan(dev, oracle, dtype):
    """cx_ip_compress_topk = whole-vector ThresholdTopK + compress_add_update.  Inputs that let the
    single pass finish (route 1), inputs whose sampled bound is useless so that the answer is
    recomputed from the accumulated vector (route 2: every magnitude equal, ties at the
    threshold, small values exactly at the sampled positions), and parameters for which the
    single pass is not attempted (route 0).  Message, residual and threshold: the checker's bits."""
    rng = np.random.default_rng(23)
    n = 11_000_001
    ds = 1 << 24  # > n: whole-vector mode of the reference
    if dtype == np.int32:
        base = rng.integers(-100000, 100001, n).astype(np.int32)
        add = rng.integers(-50, 51, n).astype(np.int32)
        tie_vec = rng.integers(-9, 10, n).astype(np.int32)
        big, small = (rng.integers(500, 1000, n).astype(np.int32), np.ones(65536, np.int32))
    else:
        base = (rng.standard_normal(n) * 3).astype(dtype)
        add = (rng.standard_normal(n) * 0.1).astype(dtype)
        tie_vec = np.round(rng.standard_normal(n) * 3).astype(dtype)
        big, small = ((5 + rng.random(n)).astype(dtype), (rng.random(65536) * 1e-3).astype(dtype))
    zero = np.zeros(n, dtype)
    sample_pos = (np.arange(65536, dtype=np.float32) * (np.float32(n) / np.float32(65536))).astype(np.int64)
    hostile = big.copy()
    hostile[sample_pos] = small  # the strided sample only sees small values
    cases = {
        "random_p0.01": (base, add, 0.01, 1),
        "random_p0.001": (base, add, 0.001, 1),
        "random_p0.3": (base, add, 0.3, 0),
        "all_equal": (np.full(n, 3, dtype), zero, 0.01, 2),
        "ties_at_threshold": (tie_vec, zero, 0.02, 2 if dtype == np.int32 else None),
        "small_at_sampled_positions": (hostile, zero, 0.01, 2),
    }
    thr_out = torch.zeros(1, dtype=NP2T[dtype], device="cuda")
    try:
        for name, (u, d, topk, route) in cases.items():
            t = np.float32(topk)
            want_thr = oracle.topk_prepare_with(u, d, t, ds, 10.0)
            uu = u.copy()
            want_msg = oracle.ip_compress(d.copy(), uu, want_thr)
            for fused in (2, 0):  # 2: the single pass from 2^23 elements on
                say("fused exact top-k", dtype.__name__, name, "fused_topk", fused)
                dev.set_option("fused_topk", fused)
                gu, gd = _gpu(u), _gpu(d)
                buf = _msgbuf(n, dtype)
                prefix = torch.zeros(1, dtype=torch.int32, device="cuda")
                nbytes = dev.compress_topk(buf, gd, gu, t, d_thr=thr_out, size_prefix=prefix)
                taken = dev.get_option("fused_topk_taken")
                if fused and route is not None:
                    assert taken == route, (name, taken)
                if not fused:
                    assert taken == 0
                assert thr_out.cpu().numpy()[0] == want_thr, (name, taken)
                assert nbytes == want_msg.size and int(prefix.item()) == nbytes, (name, nbytes, want_msg.size)
                assert buf[:nbytes].cpu().numpy().tobytes() == want_msg.tobytes(), name
                assert gu.cpu().numpy().tobytes() == uu.tobytes(), name
                assert gd.cpu().numpy().tobytes() == d.tobytes(), name
    finally:
        dev.set_option("fused_topk", 1)


def test_fused_exact_topk_message_buffer_too_small_and_bad_arguments(dev, oracle):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rng = np.random.default_rng(24)
    n = (1 << 23) + 5
    u, d = _rand(rng, n, np.float32), _rand(rng, n, np.float32, 0.3)
    t = np.float32(0.01)
    want_thr = oracle.topk_prepare_with(u, d, t, 1 << 24, 10.0)
    uu = u.copy()
    want_msg = oracle.ip_compress(d.copy(), uu, want_thr)
    keep = 8 + 8 * 1000  # room for 1000 pairs
    buf = torch.zeros(keep, dtype=torch.uint8, device="cuda")
    gu, gd = _gpu(u), _gpu(d)
    say("fused exact top-k, message buffer too small")
    dev.set_option("fused_topk", 2)  # the single pass at this length
    try:
        with pytest.raises(ComprexError) as e:
            dev.compress_topk(buf, gd, gu, t)
    finally:
        dev.set_option("fused_topk", 1)
    assert e.value.code == _lib.CX_ERR_CAPACITY
    assert dev.get_option("fused_topk_taken") == 1
    got = buf.cpu().numpy()
    assert got[:8].view(np.int32).tolist() == [n, 1000]         # the header announces what was written
    assert got[8:].tobytes() == want_msg[8:keep].tobytes()      # the pairs that fit
    # what found no room is still in the residual: the sums of the pairs that were not written
    left = uu.copy()
    rest = want_msg[keep:].view(np.dtype([("i", np.int32), ("v", np.float32)]))
    left[rest["i"]] = rest["v"]
    assert gu.cpu().numpy().tobytes() == left.tobytes()
    with pytest.raises(ComprexError) as e:
        dev.compress_topk(_msgbuf(n, np.float32), gd, gu, 1.5)
    assert e.value.code == _lib.CX_ERR_TOPK
    with pytest.raises(ComprexError) as e:
        dev.compress_topk(_msgbuf(n, np.float32), gd[:-1], gu, 0.01)
    assert e.value.code == _lib.CX_ERR_SIZE_MISMATCH


def test_topk_threshold_indexed_and_device_slot(dev, oracle):
    rng = np.random.default_rng(15)
    n, m = 1_000_000, 10_000
    v, a = _rand(rng, n, np.float32), _rand(rng, n, np.float32, 0.5)
    idx = rng.integers(0, n, m).astype(np.int32)
    want = oracle.topk_prepare_indexed(v, a, idx, np.float32(0.01))
    gv, ga = _gpu(v), _gpu(a)
    assert dev.topk_threshold_indexed(gv, ga, _gpu(idx), np.float32(0.01)) == want
    # threshold left on the device and consumed from there by the compressor
    out = torch.zeros(1, device="cuda")
    dev.topk_threshold_indexed(gv, ga, _gpu(idx), np.float32(0.01), out=out, to_host=False)
    buf = _msgbuf(n, np.float32)
    nbytes = dev.compress(buf, ga, gv, d_thr=out)
    uu = v.copy()
    wmsg = oracle.ip_compress(a.copy(), uu, want)
    assert nbytes == wmsg.size and buf[:nbytes].cpu().numpy().tobytes() == wmsg.tobytes()
    assert gv.cpu().numpy().tobytes() == uu.tobytes()


@pytest.mark.parametrize("dtype", DTYPES)
def test_sampled_threshold_with_more_samples_than_the_two_launches_take(dev, oracle, dtype):
    """More than 2^18 sample positions, host-supplied or strided: radix passes over the sample.  On a
    vector long enough for the handle's candidate buffer the first pass leaves the gathered keys there
    and the later passes read them back; on a shorter one every pass follows the positions.  Ties,
    positions outside the vector (magnitude 0) and both orders of the positions: the checker's bits."""
    rng = np.random.default_rng(61)
    for n in (9_000_001, 3_000_000):
        v = _rand(rng, n, dtype)
        v[rng.integers(0, n, n // 50)] *= 40
        a = _rand(rng, n, dtype, 0.25)
        if dtype != np.int32:
            v = (np.round(v * 8) / 8).astype(dtype)  # ties
        v[0] = a[0] = 0  # where the checker looks for a position outside the vector (the reference would read out of bounds)
        gv, ga = _gpu(v), _gpu(a)
        for m, topk in ((300_000, 0.02), (600_001, 0.001), (262_145, 0.3)):
            idx = rng.integers(0, n, m).astype(np.int32)
            idx[::1000] = n + 5
            idx[1::1000] = -1
            for order in ("given", "sorted"):
                if order == "sorted":
                    idx = np.sort(idx)
                say("large sample", dtype.__name__, n, m, topk, order)
                inside = np.where((idx < 0) | (idx >= n), 0, idx).astype(np.int32)
                want = oracle.topk_prepare_indexed(v, a, inside, np.float32(topk))
                assert dev.topk_threshold_indexed(gv, ga, _gpu(idx), np.float32(topk)) == want
            # strided: ThresholdTopK(topK, m, 1.0) takes m sub-samples
            assert dev.topk_threshold(gv, ga, np.float32(topk), m, 1.0) == oracle.topk_prepare_with(v, a, np.float32(topk), m, 1.0)
            assert dev.topk_threshold(gv, None, np.float32(topk), m, 1.0) == oracle.topk_prepare(v, np.float32(topk), m, 1.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sampled_threshold_short_list_and_inputs_that_defeat_it(dev, oracle, dtype):
    """The two-launch select hands its second launch a short list of each block's top keys and
    falls back on the full key array when the list cannot hold the answer: large values
    clustered in a few blocks' share of the samples, all-equal keys (list overflows), sample sets
    too small or ranks too deep for the list.  The second launch takes its digits from the first bit in
    which the listed keys differ and ranks the last few keys by counting: inputs with few distinct
    magnitudes (ties) and with keys that differ in their first bit.  Same threshold as the checker
    with the list on and off."""
    rng = np.random.default_rng(31)
    n = 3_000_000
    if dtype == np.int32:
        spread = rng.integers(-1_000_000, 1_000_001, n).astype(np.int32)
        add = rng.integers(-10, 11, n).astype(np.int32)
    else:
        spread = (rng.laplace(size=n) * 2).astype(dtype)
        add = (rng.standard_normal(n) * 0.05).astype(dtype)
    clustered = (spread // 1000 if dtype == np.int32 else spread * 1e-3).astype(dtype)
    clustered[: n // 40] = spread[: n // 40]            # every large value sits at the front
    equal = np.full(n, 7, dtype)
    zero = np.zeros(n, dtype)
    # few distinct magnitudes: the keys left for the final count are full of ties
    quantized = (spread // 100_000 * 100_000 if dtype == np.int32 else np.round(spread * 2) / 2).astype(dtype)
    # the largest keys are the largest there are (-INT_MAX: the magnitude of INT_MIN is no int, and
    # the reference's abs() of it is undefined)
    extreme = spread.copy()
    extreme[:: 37] = -np.iinfo(np.int32).max if dtype == np.int32 else np.finfo(dtype).max
    extreme[5 :: 41] = np.iinfo(np.int32).max if dtype == np.int32 else np.finfo(dtype).tiny
    try:
        for name, v, a in [("spread", spread, add), ("clustered", clustered, zero), ("equal", equal, zero),
                           ("quantized", quantized, zero), ("extreme", extreme, zero)]:
            gv, ga = _gpu(v), _gpu(a)
            for m, topk in [(100_000, 0.01), (65_536, 0.0133), (8_192, 0.01), (200_000, 0.002), (100_000, 0.2),
                            (262_144, 0.01), (5_000, 0.01), (262_145, 0.01), (700_001, 0.003)]:
                idx = np.sort(rng.integers(0, n, m)).astype(np.int32)
                want = oracle.topk_prepare_indexed(v, a, idx, np.float32(topk))
                gi = _gpu(idx)
                for short in (1, 0):
                    say("sampled threshold", dtype.__name__, name, m, topk, "short list", short)
                    dev.set_option("select_short_list", short)
                    assert dev.topk_threshold_indexed(gv, ga, gi, np.float32(topk)) == want
                    # twice: the state the first run leaves must be clean
                    assert dev.topk_threshold_indexed(gv, ga, gi, np.float32(topk)) == want
    finally:
        dev.set_option("select_short_list", 1)


def test_topk_threshold_errors(dev):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    v = torch.zeros(10, device="cuda")
    with pytest.raises(ComprexError) as e:
        dev.topk_threshold(v, torch.zeros(11, device="cuda"), 0.1)
    assert e.value.code == _lib.CX_ERR_SIZE_MISMATCH
    for bad in (1.5, -0.1):
        with pytest.raises(ComprexError) as e:
            dev.topk_threshold(v, None, bad)
        assert e.value.code == _lib.CX_ERR_TOPK


# --------------------------------------------------------------------------- receive side
@pytest.mark.parametrize("dtype", DTYPES)
def test_decompress_add_match_oracle(dev, oracle, dtype):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rng = np.random.default_rng(16)
    for n in [1, 17, 1000, 33_333, 1_000_001]:
        d = _rand(rng, n, dtype)
        msg = oracle.ip_compress(d, None, dtype(np.quantile(np.abs(d), 0.9)))
        gmsg = _gpu(msg)
        for out_n in [n, n + 13]:
            say("decompress/add", dtype.__name__, n, out_n)
            base = _rand(rng, out_n, dtype)
            o = base.copy()
            want_bytes = oracle.ip_decompress(msg, o)
            g = _gpu(base)
            assert dev.decompress(g, gmsg) == want_bytes
            assert g.cpu().numpy().tobytes() == o.tobytes()
            o = base.copy()
            oracle.ip_add(msg, o)
            g = _gpu(base)
            dev.add(g, gmsg)
            assert g.cpu().numpy().tobytes() == o.tobytes()
        if n > 1:
            g = torch.ones(n - 1, dtype=NP2T[dtype], device="cuda")
            with pytest.raises(ComprexError) as e:
                dev.decompress(g, gmsg)
            assert e.value.code == _lib.CX_ERR_MSG_TOO_LARGE and (g == 0).all()
            g = torch.ones(n - 1, dtype=NP2T[dtype], device="cuda")
            with pytest.raises(ComprexError) as e:
                dev.add(g, gmsg)
            assert e.value.code == _lib.CX_ERR_MSG_TOO_LARGE and (g == 1).all()
    dev.synchronize()


def test_add_duplicate_indices_in_message_order(dev, oracle):
    rec = np.dtype([("i", np.int32), ("v", np.float32)])
    body = np.array([(2, 1e8), (2, 1.0), (2, -1e8), (5, 3.0), (7, 1.0), (7, 2.0)], dtype=rec)
    msg = np.concatenate([np.array([8, 6], np.int32).view(np.uint8), body.view(np.uint8)])
    want = np.zeros(8, np.float32)
    oracle.ip_add(msg, want)
    g = torch.zeros(8, device="cuda")
    dev.add(g, _gpu(msg))
    assert g.cpu().numpy().tobytes() == want.tobytes()
    want = np.ones(8, np.float32)
    oracle.ip_decompress(msg, want)
    g = torch.ones(8, device="cuda")
    dev.decompress(g, _gpu(msg))
    assert g.cpu().numpy().tobytes() == want.tobytes()


def test_index_out_of_range_is_reported_not_written(dev):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rec = np.dtype([("i", np.int32), ("v", np.float32)])
    body = np.array([(1, 1.0), (99, 5.0), (-4, 5.0)], dtype=rec)
    msg = np.concatenate([np.array([8, 3], np.int32).view(np.uint8), body.view(np.uint8)])
    g = torch.zeros(8, device="cuda")
    dev.add(g, _gpu(msg))
    with pytest.raises(ComprexError) as e:
        dev.synchronize()
    assert e.value.code == _lib.CX_ERR_INDEX
    assert g.tolist() == [0, 1, 0, 0, 0, 0, 0, 0]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reduce_rank_order_bit_exact_and_atomic_tolerance(dev, oracle, dtype):
    from comprex_amd import workloads as W
    n, ranks, k = 1 << 20, 8, 10_000
    msgs = W.c5_messages(seed=77, n=n, ranks=ranks, k=k, shared=k // 2, dtype=dtype)
    want = np.zeros(n, dtype)
    for m in msgs:
        oracle.ip_add(m, want)
    gm = [_gpu(m) for m in msgs]
    for accumulate in (False, True):
        say("reduce", dtype.__name__, "accumulate", accumulate)
        base = _rand(np.random.default_rng(5), n, dtype) if accumulate else np.zeros(n, dtype)
        w = base.copy()
        for m in msgs:
            oracle.ip_add(m, w)
        g = _gpu(base) if accumulate else torch.full((n,), 7, dtype=NP2T[dtype], device="cuda")
        dev.reduce(g, gm, accumulate=accumulate, mode=0)
        assert g.cpu().numpy().tobytes() == w.tobytes()
        # atomics add the same contributions in another order: the two sums differ by at most
        # 2 * gamma_m * sum|v| per element (m rounded additions, u = eps/2), and not at all where an
        # element has a single contribution
        g = _gpu(base) if accumulate else torch.full((n,), 7, dtype=NP2T[dtype], device="cuda")
        dev.reduce(g, gm, accumulate=accumulate, mode=1)
        got = g.cpu().numpy()
        bound = reorder_bound(msgs, dtype, n, base if accumulate else None)
        assert (np.abs(got.astype(np.float64) - w.astype(np.float64)) <= bound).all()
        alone = bound == 0.0
        assert alone.sum() > n // 2 and got[alone].tobytes() == w[alone].tobytes()
        # the bound is not slack: a relative tolerance of 1e-6 (fp32) would fail where contributions cancel
        if dtype == np.float32 and not accumulate:
            rel = np.abs(got - w) / np.maximum(np.abs(w), np.finfo(np.float32).tiny)
            say("largest relative difference of the atomic sum", float(rel.max()),
                "largest ratio to the bound", float((np.abs(got.astype(np.float64) - w) / np.maximum(bound, 1e-300)).max()))
    dev.synchronize()


def test_reduce_many_messages_duplicates_and_variants(dev, oracle):
    """More messages than one tiled launch takes (16), repeated indices inside a message, empty
    messages, a vector that ends inside a tile; both rank-ordered variants give the checker's bits."""
    rng = np.random.default_rng(23)
    n = 70_001
    rec = np.dtype([("i", np.int32), ("v", np.float32)])
    msgs = []
    for r in range(20):
        k = int(rng.integers(0, 900)) if r != 7 else 0
        idx = np.sort(rng.integers(0, n, k)).astype(np.int32)  # sorted, repeats allowed
        body = np.empty(k, rec)
        body["i"], body["v"] = idx, rng.standard_normal(k).astype(np.float32) * np.float32(10.0 ** float(rng.integers(-3, 4)))
        msgs.append(np.concatenate([np.array([n, k], np.int32).view(np.uint8), body.view(np.uint8)]))
    base = rng.standard_normal(n).astype(np.float32)
    gm = [_gpu(m) for m in msgs]
    try:
        for variant in (0, 1, 2, 3):
            dev.set_option("reduce_variant", variant)
            for accumulate in (False, True):
                want = base.copy() if accumulate else np.zeros(n, np.float32)
                for m in msgs:
                    oracle.ip_add(m, want)
                g = _gpu(base)
                dev.reduce(g, gm, accumulate=accumulate, mode=0)
                assert g.cpu().numpy().tobytes() == want.tobytes(), (variant, accumulate)
            want = np.ones(n, np.float32)
            oracle.ip_decompress(msgs[3], want)
            g = torch.ones(n, device="cuda")
            dev.decompress(g, gm[3])
            assert g.cpu().numpy().tobytes() == want.tobytes()
        dev.synchronize()
    finally:
        dev.set_option("reduce_variant", 0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_pipelined_reduce_many_tiles_per_block_clusters_and_ragged_ends(dev, oracle, dtype):
    """The pipelined rank-ordered reduce on vectors long enough that every block walks many tiles:
    2..9 messages (more than one launch carries), pairs clustered so that far more than one chunk
    of a message falls into one tile, long empty stretches, repeated indices, -0.0 values in the
    first message (added to zeros), a vector that ends inside a tile, an output pointer
    that is not 16-byte aligned, accumulate and overwrite: the checker's bits every time."""
    rng = np.random.default_rng(99)
    np_dt = np.dtype(dtype)
    rec = np.dtype([("i", np.int32), ("v", np_dt)], align=False)
    n = 6_000_011
    try:
        dev.set_option("reduce_variant", 3)
        for n_msgs, unique in ((2, True), (5, False), (8, True), (9, False)):
            msgs = []
            for r in range(n_msgs):
                parts = [rng.integers(0, n, 30_000)]
                c0 = int(rng.integers(0, n - 5000))
                parts.append(rng.integers(c0, c0 + 3000, 2500))          # a dense cluster: whole chunks in one tile
                parts.append(np.arange(n - 700, n, 3))                    # the ragged end
                if r == 1:
                    parts = [rng.integers(n // 2, n // 2 + 100, 40)]      # a nearly empty message
                idx = np.sort(np.concatenate(parts))
                if unique:
                    idx = np.unique(idx)
                idx = idx.astype(np.int32)
                body = np.empty(idx.size, rec)
                body["i"] = idx
                if np_dt.kind == "f":
                    body["v"] = (rng.standard_normal(idx.size) * 10.0 ** rng.integers(-3, 4, idx.size)).astype(np_dt)
                    if r == 0:
                        body["v"][::7] = np_dt.type(-0.0)
                else:
                    body["v"] = rng.integers(-10**6, 10**6, idx.size).astype(np_dt)
                msgs.append(np.concatenate([np.array([n, idx.size], np.int32).view(np.uint8), body.view(np.uint8)]))
            gm = [_gpu(m) for m in msgs]
            base = _rand(rng, n + 1, dtype)
            for accumulate in (False, True):
                for shift in (0, 1):  # shift 1: the output starts one element into an allocation
                    say("pipelined reduce", np_dt.name, n_msgs, "messages, accumulate", accumulate, "shift", shift)
                    want = base[shift:shift + n].copy() if accumulate else np.zeros(n, np_dt)
                    for m in msgs:
                        oracle.ip_add(m, want)
                    g_all = _gpu(base)
                    g = g_all[shift:shift + n]
                    dev.reduce(g, gm, accumulate=accumulate, mode=0)
                    dev.synchronize()
                    assert g.cpu().numpy().tobytes() == want.tobytes()
                    if shift == 0:
                        assert g_all[n:].cpu().numpy().tobytes() == base[n:].tobytes(), "wrote past the vector"
    finally:
        dev.set_option("reduce_variant", 0)


def test_pipelined_reduce_reports_unsorted_and_out_of_range(dev):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rec = np.dtype([("i", np.int32), ("v", np.float32)])
    n = 3_000_000
    rng = np.random.default_rng(3)
    good = np.unique(rng.integers(0, n, 20_000)).astype(np.int32)

    def message(idx):
        body = np.empty(idx.size, rec)
        body["i"], body["v"] = idx, 1.0
        return _gpu(np.concatenate([np.array([n, idx.size], np.int32).view(np.uint8), body.view(np.uint8)]))

    swapped = good.copy()
    swapped[[7000, 12000]] = swapped[[12000, 7000]]       # two pairs far apart trade places
    beyond = np.concatenate([good, np.array([n + 5], np.int32)])
    negative = np.concatenate([np.array([-3], np.int32), good])
    try:
        dev.set_option("reduce_variant", 3)
        for bad in (swapped, beyond, negative):
            g = torch.zeros(n, device="cuda")
            dev.reduce(g, [message(good), message(bad)], accumulate=False, mode=0)
            with pytest.raises(ComprexError) as e:
                dev.synchronize()
            assert e.value.code == _lib.CX_ERR_INDEX
        g = torch.zeros(n, device="cuda")
        dev.reduce(g, [message(good), message(good)], accumulate=False, mode=0)
        dev.synchronize()
        assert float(g.sum().item()) == 2.0 * good.size
    finally:
        dev.set_option("reduce_variant", 0)


def test_tiled_reduce_reports_unsorted_message(dev):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rec = np.dtype([("i", np.int32), ("v", np.float32)])
    body = np.array([(5000, 1.0), (3, 2.0), (9000, 3.0)], dtype=rec)
    msg = np.concatenate([np.array([10000, 3], np.int32).view(np.uint8), body.view(np.uint8)])
    g = torch.zeros(10000, device="cuda")
    dev.reduce(g, [_gpu(msg)], accumulate=False, mode=0)
    with pytest.raises(ComprexError) as e:
        dev.synchronize()
    assert e.value.code == _lib.CX_ERR_INDEX


def test_any_order_accumulate_takes_scatters_or_one_pass_by_pair_count(dev, oracle):
    """Adding index-sorted messages with CX_REDUCE_ANY_ORDER: the order check also reads the pair
    counts, and few sparse messages are applied as one scatter each (only their elements are touched)
    instead of one pass over the whole vector.  Both choices give the checker's sums, additions in
    message order (half of each message's indices are shared with the others)."""
    from comprex_amd import workloads as W
    n = 6_000_000
    for k, count in ((n // 2000, 3), (n // 20, 3), (n // 2000, 12)):
        say("any-order accumulate", n, k, count)
        msgs_h = W.c5_messages(seed=7 + k, n=n, ranks=count, k=k, shared=k // 2)
        base = np.random.default_rng(k).standard_normal(n).astype(np.float32)
        want = base.copy()
        for m in msgs_h:
            oracle.ip_add(m, want)
        out = _gpu(base)
        dev.reduce(out, [_gpu(m) for m in msgs_h], accumulate=True, mode=0, any_order=True)
        dev.synchronize()
        assert out.cpu().numpy().tobytes() == want.tobytes()


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_and_reduce_take_any_index_order_when_asked(dev, oracle, dtype):
    """The reference's add walks the pairs as stored (src/compressor.hxx:640-658): any index order, an
    index repeated anywhere, the additions in message order.  The fast paths want ascending indices.
    With CX_ADD_ANY_ORDER / CX_REDUCE_ANY_ORDER (what Compressor::add / add_many pass) the call looks
    at the indices first and applies such messages pair after pair: expected values from the
    checker, which is that loop.  Without the flag the disorder is reported (CX_ERR_INDEX), never
    turned into a different sum silently."""
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rng = np.random.default_rng(43)
    n, k = 40_000, 7_003
    rec = np.dtype([("i", np.int32), ("v", dtype)])

    def message(sorted_idx):
        idx = rng.integers(0, n // 8, k).astype(np.int32)            # many repeats, far apart
        idx[200:210] = idx[3000]                                       # and a run of repeats inside one chunk
        if sorted_idx:
            idx = np.sort(idx)
        body = np.empty(k, rec)
        body["i"], body["v"] = idx, _rand(rng, k, dtype)
        return np.concatenate([np.array([n, k], np.int32).view(np.uint8), body.view(np.uint8)])

    msgs = [message(False), message(True), message(False), message(False), message(True)]
    start = _rand(rng, n, dtype)
    # one message at a time
    want = start.copy()
    g = torch.from_numpy(start.copy()).cuda()
    for m in msgs:
        oracle.ip_add(m, want)
        dev.add(g, _gpu(m), any_order=True)
    dev.synchronize()
    assert g.cpu().numpy().tobytes() == want.tobytes()
    # all at once, added into the vector and from zeros
    gm = [_gpu(m) for m in msgs]
    g = torch.from_numpy(start.copy()).cuda()
    dev.reduce(g, gm, accumulate=True, any_order=True)
    dev.synchronize()
    assert g.cpu().numpy().tobytes() == want.tobytes()
    want0 = np.zeros(n, dtype)
    for m in msgs:
        oracle.ip_add(m, want0)
    g = torch.full((n,), 5, dtype=NP2T[dtype], device="cuda")
    dev.reduce(g, gm, accumulate=False, any_order=True)
    dev.synchronize()
    assert g.cpu().numpy().tobytes() == want0.tobytes()
    # sorted messages keep the fast path and its result
    sorted_only = [gm[1], gm[4]]
    wants = start.copy()
    oracle.ip_add(msgs[1], wants)
    oracle.ip_add(msgs[4], wants)
    g = torch.from_numpy(start.copy()).cuda()
    dev.reduce(g, sorted_only, accumulate=True, any_order=True)
    dev.synchronize()
    assert g.cpu().numpy().tobytes() == wants.tobytes()
    # without the flag: reported
    g = torch.zeros(n, dtype=NP2T[dtype], device="cuda")
    dev.add(g, gm[0], check_header=False)
    with pytest.raises(ComprexError) as e:
        dev.synchronize()
    assert e.value.code == _lib.CX_ERR_INDEX
    for acc in (False, True):
        dev.reduce(g, gm, accumulate=acc)
        with pytest.raises(ComprexError) as e:
            dev.synchronize()
        assert e.value.code == _lib.CX_ERR_INDEX


@pytest.mark.parametrize("dtype", DTYPES)
def test_decompress_takes_any_index_order_when_it_reports_back(dev, oracle, dtype):
    """The reference's decoder walks the pairs as stored (src/compressor.hxx:613-633): any index order,
    an index repeated anywhere, the last value wins.  The fast path wants ascending indices; a
    decompress that reports its byte count to the host repeats such a message pair after pair.
    Expected values: the checker, which is that loop.  Out-of-range indices stay errors, and an
    empty output vector still refuses a message made for a longer one."""
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rng = np.random.default_rng(41)
    n, k = 50_000, 9_001
    idx = rng.integers(0, n, k).astype(np.int32)                  # unsorted, with repeats far apart
    idx[100:110] = idx[5000]                                        # and a run of repeats inside one chunk
    val = _rand(rng, k, dtype)
    rec = np.dtype([("i", np.int32), ("v", dtype)])
    body = np.empty(k, rec)
    body["i"], body["v"] = idx, val
    msg = np.concatenate([np.array([n, k], np.int32).view(np.uint8), body.view(np.uint8)])
    want = np.full(n, 9, dtype)
    oracle.ip_decompress(msg, want)
    by_hand = np.zeros(n, dtype)
    for i, v in zip(idx, val):
        by_hand[i] = v
    assert want.tobytes() == by_hand.tobytes()
    g = torch.full((n,), 7, dtype=NP2T[dtype], device="cuda")
    assert dev.decompress(g, _gpu(msg)) == msg.size
    assert g.cpu().numpy().tobytes() == want.tobytes()
    # without the report the message is refused, not half applied silently
    dev.decompress(g, _gpu(msg), sync=False)
    with pytest.raises(ComprexError) as e:
        dev.synchronize()
    assert e.value.code == _lib.CX_ERR_INDEX
    # an index outside the vector is an error on both paths
    body["i"][17] = n + 3
    bad = np.concatenate([np.array([n, k], np.int32).view(np.uint8), body.view(np.uint8)])
    with pytest.raises(ComprexError) as e:
        dev.decompress(g, _gpu(bad))
    assert e.value.code == _lib.CX_ERR_INDEX
    # empty output vector
    empty = torch.zeros(0, dtype=NP2T[dtype], device="cuda")
    for variant in (0, 3):
        dev.set_option("reduce_variant", variant)
        try:
            dev.reduce(empty, [_gpu(msg)], accumulate=False, mode=0)
            with pytest.raises(ComprexError) as e:
                dev.synchronize()
            assert e.value.code == _lib.CX_ERR_MSG_TOO_LARGE
            none = np.array([0, 0], np.int32).view(np.uint8)
            dev.reduce(empty, [_gpu(none)], accumulate=False, mode=0)
            dev.synchronize()
        finally:
            dev.set_option("reduce_variant", 0)


# --------------------------------------------------------------------------- residual maintenance
@pytest.mark.parametrize("dtype", DTYPES)
def test_zero_addvec_apply(dev, oracle, dtype):
    rng = np.random.default_rng(17)
    for n in [1, 1000, 100_003]:
        a, b = _rand(rng, n + 1, dtype), _rand(rng, n + 1, dtype)
        for off in (0, 1):
            ga, gb = _gpu(a), _gpu(b)
            dev.add_vec(ga[off:off + n], gb[off:off + n])
            w = a.copy()
            oracle.add_rests(w[off:off + n], np.ascontiguousarray(b[off:off + n]))
            assert ga.cpu().numpy().tobytes() == w.tobytes()
            dev.zero(ga[off:off + n])
            w[off:off + n] = 0
            assert ga.cpu().numpy().tobytes() == w.tobytes()
        v = np.ascontiguousarray(a[:n])
        thr = dtype(np.quantile(np.abs(v), 0.7))
        hi, lo = dev.threshold_apply(_gpu(v), thr, split=True)
        whi, wlo = oracle.threshold_apply_split(v, thr)
        assert hi.cpu().numpy().tobytes() == whi.tobytes() and lo.cpu().numpy().tobytes() == wlo.tobytes()
        assert dev.threshold_apply(_gpu(v), thr).cpu().numpy().tobytes() == oracle.threshold_apply(v, thr).tobytes()


# --------------------------------------------------------------------------- golden fixtures
def test_small_golden_fixtures(dev):
    """Outputs of the compiled reference headers, committed under tests/golden/."""
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "small_cases.npz"))
    tags = {"f32": np.float32, "f64": np.float64, "i32": np.int32}
    keys = sorted({k.rsplit("_grads", 1)[0] for k in z.files if k.endswith("_grads")})
    assert len(keys) == int(z["n_cases"][0])
    for key in keys:
        dtype = tags[key.split("_")[1]]
        grads = z[key + "_grads"]
        n, ds = [int(x) for x in z[key + "_params"]]
        topk = np.float32(z[key + "_topk"][0])
        say("golden", key, n, topk, ds)
        rests = torch.zeros(n, dtype=NP2T[dtype], device="cuda")
        buf = _msgbuf(n, dtype)
        for it in range(grads.shape[0]):
            g = _gpu(grads[it])
            thr = dev.topk_threshold(rests, g, topk, ds, 10.0)
            assert thr == z[key + "_thr"][it]
            nbytes = dev.compress(buf, g, rests)  # threshold taken from the handle's device slot
            want = z["%s_msg%d" % (key, it)]
            assert nbytes == want.size and buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
            assert rests.cpu().numpy().tobytes() == z["%s_rests%d" % (key, it)].tobytes()
        g = _gpu(grads[-1])
        thr = dev.topk_threshold(g, None, topk, ds, 10.0)
        assert thr == z[key + "_thr_noresidual"][0]
        want = z[key + "_msg_dataonly"]
        nbytes = dev.compress(buf, g, None, thr=thr)
        assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
        u = _gpu(grads[-1])
        want = z[key + "_msg_updateonly"]
        nbytes = dev.compress(buf, None, u, thr=thr)
        assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
        assert u.cpu().numpy().tobytes() == z[key + "_upd_after"].tobytes()
        want = z[key + "_msg_flush"]
        nbytes = dev.compress(buf, rests, None, thr=0)
        assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes()
        m0 = _gpu(z[key + "_msg0"])
        o = _gpu(grads[0])
        dev.decompress(o, m0)
        assert o.cpu().numpy().tobytes() == z[key + "_dec0"].tobytes()
        o = _gpu(grads[0])
        dev.add(o, m0)
        assert o.cpu().numpy().tobytes() == z[key + "_add0"].tobytes()


# --------------------------------------------------------------------------- run-length codec
def _rle_buf(n, dtype, extra=0):
    return torch.zeros(16 + n * np.dtype(dtype).itemsize + 4 * (n + 1) + extra, dtype=torch.uint8, device="cuda")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", ["fused", "update", "data"])
def test_rle_compress_matches_oracle(dev, oracle, dtype, mode):
    """CompressorRLE: values + run lengths, |x| >= threshold, byte for byte as the checker, whose
    encoder is pinned through the reference's own decoder."""
    rng = np.random.default_rng(51)
    for n in [0, 1, 2, 63, 64, 65, 1000, 4097, 100_003, 1_000_001]:
        for q in [0.0, 0.5, 0.99, 0.9999, 1.5]:
            say("rle compress", dtype.__name__, mode, n, q)
            d = _rand(rng, n, dtype)
            u = _rand(rng, n, dtype, 0.5)
            ref = d if mode == "data" else (u if mode == "update" else (u + d).astype(dtype))
            thr = dtype(0) if n == 0 or q == 0 else dtype(np.quantile(np.abs(ref), min(q, 1.0)) * (2 if q > 1 else 1))
            dd = d.copy() if mode != "update" else None
            uu = u.copy() if mode != "data" else None
            if n == 0:
                want = oracle.rle_compress(np.zeros(0, dtype), None, thr)
            else:
                want = oracle.rle_compress(dd, uu, thr)
            gd = _gpu(d) if mode != "update" else None
            gu = _gpu(u) if mode != "data" else None
            if n == 0:
                gd, gu = torch.zeros(0, dtype=NP2T[dtype], device="cuda"), None
            buf = _rle_buf(n, dtype)
            prefix = torch.zeros(1, dtype=torch.int32, device="cuda")
            nbytes = dev.rle_compress(buf, gd, gu, thr=thr, size_prefix=prefix)
            assert nbytes == want.size == int(prefix.item()), (n, q, nbytes, want.size)
            assert buf[:nbytes].cpu().numpy().tobytes() == want.tobytes(), (n, q)
            if gu is not None and n > 0:
                assert gu.cpu().numpy().tobytes() == uu.tobytes()
            if gd is not None and n > 0:
                assert gd.cpu().numpy().tobytes() == d.tobytes()


def test_rle_runs_of_every_shape_and_threshold_on_the_device(dev, oracle):
    rng = np.random.default_rng(52)
    n = 300_000
    shapes = {
        "alternating": np.where(np.arange(n) % 2 == 0, 5.0, 0.0),
        "starts_unsent": np.where(np.arange(n) % 2 == 1, 5.0, 0.0),
        "long_runs": np.where((np.arange(n) // 10_000) % 2 == 0, 3.0, 0.25),
        "one_sent_at_the_end": np.where(np.arange(n) == n - 1, 9.0, 0.0),
        "one_unsent_in_the_middle": np.where(np.arange(n) == n // 2, 0.0, 9.0),
        "random_blocks": np.repeat(rng.random(n // 100) < 0.3, 100) * 4.0,
        "equal_to_threshold": np.where(rng.random(n) < 0.1, 1.0, 0.5),  # |x| == thr is sent
    }
    d_thr = torch.tensor([1.0], device="cuda")
    for name, v in shapes.items():
        v = (v * np.where(rng.random(n) < 0.5, -1, 1)).astype(np.float32)
        say("rle shape", name)
        want = oracle.rle_compress(v, None, np.float32(1.0))
        buf = _rle_buf(n, np.float32)
        nbytes = dev.rle_compress(buf, _gpu(v), None, d_thr=d_thr)  # threshold read on the device
        assert nbytes == want.size and buf[:nbytes].cpu().numpy().tobytes() == want.tobytes(), name
        out = torch.full((n + 7,), 3.0, device="cuda")
        assert dev.rle_decompress(out, buf) == n
        assert out[:n].cpu().numpy().tobytes() == np.where(np.abs(v) >= 1, v, 0).astype(np.float32).tobytes(), name
        assert bool((out[n:] == 3.0).all())


@pytest.mark.parametrize("dtype", DTYPES)
def test_rle_decompress_add_match_oracle_and_errors(dev, oracle, dtype):
    from comprex_amd.device import ComprexError
    from comprex_amd import _lib
    rng = np.random.default_rng(53)
    for n in [1, 5, 1000, 70_001, 1_000_003]:
        for q in [0.0, 0.9, 0.999]:
            say("rle decode", dtype.__name__, n, q)
            v = _rand(rng, n, dtype)
            thr = dtype(0) if q == 0 else dtype(np.quantile(np.abs(v), q))
            msg = oracle.rle_compress(v, None, thr)
            gmsg = _gpu(msg)
            base = _rand(rng, n + 9, dtype)
            o = base.copy()
            assert oracle.rle_decompress(msg, o) == n
            g = _gpu(base)
            assert dev.rle_decompress(g, gmsg) == n
            assert g.cpu().numpy().tobytes() == o.tobytes()
            o = base.copy()
            oracle.rle_add(msg, o)
            g = _gpu(base)
            dev.rle_add(g, gmsg)
            dev.synchronize()
            assert g.cpu().numpy().tobytes() == o.tobytes()
    with pytest.raises(ComprexError) as e:
        dev.rle_decompress(torch.zeros(n - 1, dtype=NP2T[dtype], device="cuda"), gmsg)
    assert e.value.code == _lib.CX_ERR_MSG_TOO_LARGE
    with pytest.raises(ComprexError) as e:
        dev.rle_add(torch.zeros(n - 1, dtype=NP2T[dtype], device="cuda"), gmsg)
    assert e.value.code == _lib.CX_ERR_MSG_TOO_LARGE
    # message buffer too small: reported, nothing written past the buffer
    small = torch.zeros(64, dtype=torch.uint8, device="cuda")
    guard = small.clone()
    with pytest.raises(ComprexError) as e:
        dev.rle_compress(small[:40], _gpu(v), None, thr=dtype(0))
    assert e.value.code == _lib.CX_ERR_CAPACITY
    assert torch.equal(small[40:], guard[40:])
