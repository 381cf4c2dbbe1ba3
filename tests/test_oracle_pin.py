"""Pins the CPU restatement (oracle/) before anything is compared against it.

Sources of truth, in order: the known answers of the reference's own tests
(test/threshold.cpp, test/compressor.cpp, test/comprex.cpp), the reference's
headers compiled as-is (oracle/_ref), and what the mathematics fixes (brute-force
sort, counting, round trips).  No test here retypes the oracle's own formula.
"""
import numpy as np
import pytest

from oracle.pyoracle import parse_message

DTYPES = [np.float32, np.float64, np.int32]


def _rand(rng, n, dtype, scale=1.0):
    if dtype == np.int32:
        return rng.integers(-1000, 1001, n).astype(np.int32)
    return (rng.standard_normal(n) * scale).astype(dtype)


# ---------------------------------------------------------------- known answers
def test_kat_threshold_const_and_topk(oracle):
    """test/threshold.cpp:29-85: v[i] = i*(1-2*(i%2)), n=100, int data."""
    i = np.arange(100)
    v = (i * (1 - 2 * (i % 2))).astype(np.int32)
    out = oracle.threshold_apply(v, 20)
    assert ((out != 0) == (np.abs(v) >= 20)).all()
    # ThresholdTopK(0.10): reference prints threshold 90 and 10 surviving elements
    thr = oracle.topk_prepare(v, np.float32(0.10))
    assert thr == 90
    out = oracle.threshold_apply(v, thr)
    assert np.count_nonzero(out) == 10
    assert ((out != 0) == (np.abs(v) >= thr)).all()
    # the same data through IndexPairs uses strict '>' (compressor.hxx:571): 9 survivors
    msg = oracle.ip_compress(v, None, thr)
    assert parse_message(msg, np.int32)[1] == 9


def test_kat_compressor_roundtrip(oracle):
    """test/compressor.cpp:29-38,74-94: 25 non-zeros, compress(thr 0) -> decompress == input."""
    i = np.arange(100)
    v = (i * ((i % 4) // 3) * (1 - 2 * ((i % 6) // 5))).astype(np.int32)
    assert np.count_nonzero(v) == 25
    msg = oracle.ip_compress(v, None, 0)
    n, k, idx, val = parse_message(msg, np.int32)
    assert (n, k) == (100, 25) and msg.size == 8 + 8 * 25
    out = np.full(100, 7, dtype=np.int32)
    assert oracle.ip_decompress(msg, out) == msg.size
    assert (out == v).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_kat_comprex_conservation(oracle, dtype):
    """test/comprex.cpp:38-118: n=50, TopK(0.1), 3 x writeRemote + flushRests,
    receiver readRemote_add; gold = (num_runs-1)*values, with the sizeBytes prefix on."""
    i = np.arange(50)
    values = (i * (1 - 2 * (i % 2))).astype(dtype)
    rests = np.zeros(50, dtype=dtype)
    result = np.zeros(50, dtype=dtype)
    for run in range(4):
        if run < 3:
            buf, _ = oracle.write_remote(rests, values, np.float32(0.1), send_size_bytes=True)
        else:
            buf = oracle.flush_rests(rests, send_size_bytes=True)
        assert int(buf[:4].view(np.int32)[0]) == buf.size - 4
        oracle.ip_add(buf[4:], result)
    assert (result == 3 * values).all()
    assert (rests == 0).all()


# ---------------------------------------------------------------- host arithmetic
def test_topk_pos_closed_forms(oracle):
    """Positions at the benchmark shapes, measured on the compiled reference."""
    table = [(1 << 20, 0.01, 10485), (61706, 0.1, 6170), (25557032, 0.001, 25557),
             (100_000_000, 0.01, 999_999), (100_000, 0.01, 999), (1000, 0.01, 9), (100, 0.10, 9),
             (50, 0.1, 4), (10, 0.01, 0), (0, 0.5, -1)]
    for m, topk, want in table:
        assert oracle.topk_pos(m, np.float32(topk)) == want, (m, topk)


def test_calc_subsamples_table_and_ref(oracle, refimpl):
    # defaults give 1000 for 0.1/0.01 and 10000 for 0.001 (threshold.hxx:182-186)
    assert oracle.calc_subsamples(np.float32(0.1)) == 1000
    assert oracle.calc_subsamples(np.float32(0.01)) == 1000
    assert oracle.calc_subsamples(np.float32(0.001)) == 10000
    # float/int ternary: default_subsamples goes through fp32
    assert oracle.calc_subsamples(np.float32(0.01), 100_000_001) == 100_000_000
    rng = np.random.default_rng(0)
    for _ in range(300):
        topk = np.float32(rng.uniform(1e-4, 1.0))
        ds = int(rng.integers(1, 1 << 28))
        sf = np.float32(rng.uniform(0.5, 50))
        assert oracle.calc_subsamples(topk, ds, sf) == refimpl.calc_subsamples(topk, ds, sf)


def test_strided_positions_match_ref_sampling(oracle, refimpl):
    """The strided positions are observable through the reference: on v[i] = i+1 the
    threshold is one of the sampled values, and the sample set decides which."""
    for n, topk in [(5000, 0.01), (123457, 0.003), (1 << 20, 0.001), (30_000_000, 0.0005)]:
        v = np.arange(1, n + 1, dtype=np.float64)  # exact in fp64 up to 2^53
        a = oracle.topk_prepare(v, np.float32(topk))
        b = refimpl.topk_prepare(v, np.float32(topk))
        assert a == b, (n, topk)
        m = oracle.calc_subsamples(np.float32(topk))
        pos = np.array([oracle.strided_pos(i, n, m) for i in range(m)])
        want = np.sort(v[pos])[::-1][oracle.topk_pos(m, np.float32(topk))]
        assert a == want


# ---------------------------------------------------------------- order statistic
@pytest.mark.parametrize("dtype", DTYPES)
def test_threshold_is_order_statistic_bruteforce(oracle, dtype):
    rng = np.random.default_rng(1)
    for n in [1, 2, 3, 7, 64, 1000, 4097]:
        for topk in [0.001, 0.01, 0.1, 0.5, 0.999, 1.0]:
            v = _rand(rng, n, dtype)
            if n > 8:  # plant ties around typical thresholds
                v[rng.integers(0, n, n // 4)] = v[0]
            thr = oracle.calc_threshold(v, np.float32(topk))
            pos = oracle.topk_pos(n, np.float32(topk))
            mags = np.sort(np.abs(v))[::-1]
            want = mags[0] + dtype(1) if pos <= 0 else mags[pos]
            assert thr == want, (n, topk)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prepare_matches_ref(oracle, refimpl, dtype):
    rng = np.random.default_rng(2)
    for n in [1, 5, 999, 1000, 1001, 4096, 50_000, 300_001]:
        for topk, ds, sf in [(0.01, 1000, 10.0), (0.1, 1000, 10.0), (0.001, 1000, 10.0),
                             (0.01, 125, 4.0), (0.02, 1 << 20, 10.0), (1.0, 10, 1.0)]:
            v = _rand(rng, n, dtype)
            a = _rand(rng, n, dtype, 0.3)
            t = np.float32(topk)
            assert oracle.topk_prepare(v, t, ds, sf) == refimpl.topk_prepare(v, t, ds, sf)
            assert oracle.topk_prepare_with(v, a, t, ds, sf) == refimpl.topk_prepare_with(v, a, t, ds, sf)
            assert oracle.calc_threshold(v, t) == refimpl.calc_threshold(v, t)


def test_prepare_with_size_mismatch_raises(oracle, refimpl):
    v, a = np.zeros(10, np.float32), np.zeros(11, np.float32)
    for impl in (oracle, refimpl):
        with pytest.raises(RuntimeError):
            impl.topk_prepare_with(v, a, np.float32(0.1))


def test_prepare_indexed_is_calc_threshold_on_gather(oracle):
    rng = np.random.default_rng(3)
    v = _rand(rng, 10_000, np.float32)
    a = _rand(rng, 10_000, np.float32)
    idx = rng.integers(0, 10_000, 777).astype(np.int32)
    thr = oracle.topk_prepare_indexed(v, a, idx, np.float32(0.05))
    mags = np.sort(np.abs(v[idx] + a[idx]))[::-1]
    assert thr == mags[oracle.topk_pos(777, np.float32(0.05))]


# ---------------------------------------------------------------- codec
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", ["fused", "update", "data"])
def test_compress_matches_ref_and_invariants(oracle, refimpl, dtype, mode):
    rng = np.random.default_rng(4)
    for n in [0, 1, 2, 63, 64, 65, 1000, 40_000]:
        for q in [0.0, 0.5, 0.99, 1.0]:
            d = _rand(rng, n, dtype)
            u = _rand(rng, n, dtype, 0.5)
            if n:
                u[rng.integers(0, n, max(1, n // 10))] = 0
            s = u + d if mode == "fused" else (u if mode == "update" else d)
            thr = dtype(0) if (q == 0.0 or n == 0) else dtype(np.quantile(np.abs(s), q))
            res = []
            for impl in (oracle, refimpl):
                dd = d.copy() if mode != "update" else None
                uu = u.copy() if mode != "data" else None
                msg = impl.ip_compress(dd, uu, thr).copy()
                res.append((msg, uu))
            (m0, u0), (m1, u1) = res
            assert m0.tobytes() == m1.tobytes()
            if u0 is not None:
                assert u0.tobytes() == u1.tobytes()
            # invariants the sequential loop fixes
            nn, k, idx, val = parse_message(m0, dtype)
            sel = np.abs(s) > thr
            assert nn == n and k == np.count_nonzero(sel)
            assert m0.size == 8 + k * (4 + np.dtype(dtype).itemsize)
            assert (idx == np.nonzero(sel)[0]).all() and (val == s[sel]).all()
            if u0 is not None:
                assert (u0[sel] == 0).all() and (u0[~sel] == s[~sel]).all()
                assert not np.signbit(u0[sel].astype(np.float64)).any()  # zeroing stores +0


def test_compress_nan_never_selected(oracle, refimpl):
    d = np.array([1, np.nan, -3, np.inf, -np.inf, 0.5], dtype=np.float32)
    u = np.zeros(6, dtype=np.float32)
    for impl in (oracle, refimpl):
        uu = u.copy()
        n, k, idx, val = parse_message(impl.ip_compress(d.copy(), uu, np.float32(0.75)), np.float32)
        assert list(idx) == [0, 2, 3, 4] and np.isnan(uu[1]) and uu[5] == 0.5


def test_compress_add_update_size_mismatch(oracle, refimpl):
    for impl in (oracle, refimpl):
        with pytest.raises(RuntimeError):
            impl.ip_compress_add_update(np.zeros(4, np.float32), np.zeros(5, np.float32), 0.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decompress_and_add_match_ref(oracle, refimpl, dtype):
    rng = np.random.default_rng(5)
    for n in [1, 17, 1000, 33_333]:
        d = _rand(rng, n, dtype)
        msg = oracle.ip_compress(d, None, dtype(np.quantile(np.abs(d), 0.9)))
        for out_n in [n, n + 13]:
            base = _rand(rng, out_n, dtype)
            o0, o1 = base.copy(), base.copy()
            assert oracle.ip_decompress(msg, o0) == refimpl.ip_decompress(msg, o1) == msg.size
            assert o0.tobytes() == o1.tobytes()
            nn, k, idx, val = parse_message(msg, dtype)
            dense = np.zeros(out_n, dtype)
            dense[idx] = val
            assert (o0 == dense).all()
            o0, o1 = base.copy(), base.copy()
            oracle.ip_add(msg, o0)
            refimpl.ip_add(msg, o1)
            assert o0.tobytes() == o1.tobytes()
            assert (o0 == base + dense).all()
        if n > 1:  # message larger than the output: reference throws (compressor.hxx:620-624,645-647)
            small = np.ones(n - 1, dtype)
            for impl in (oracle, refimpl):
                s = small.copy()
                with pytest.raises(RuntimeError):
                    impl.ip_decompress(msg, s)
                assert (s == 0).all()  # memset ran before the check
                s = small.copy()
                with pytest.raises(RuntimeError):
                    impl.ip_add(msg, s)
                assert (s == 1).all()


def test_add_duplicate_indices_sum_in_message_order(oracle, refimpl):
    """Hand-built message with a repeated index: contributions add sequentially."""
    rec = np.dtype([("i", np.int32), ("v", np.float32)])
    body = np.array([(2, 1e8), (2, 1.0), (2, -1e8), (5, 3.0)], dtype=rec)
    msg = np.concatenate([np.array([8, 4], np.int32).view(np.uint8), body.view(np.uint8)])
    for impl in (oracle, refimpl):
        out = np.zeros(8, np.float32)
        impl.ip_add(msg, out)
        assert out[2] == np.float32(np.float32(np.float32(1e8) + np.float32(1.0)) - np.float32(1e8))
        assert out[5] == 3.0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_threshold_apply_matches_ref(oracle, refimpl, dtype):
    rng = np.random.default_rng(6)
    v = _rand(rng, 5000, dtype)
    thr = dtype(0.8)
    assert oracle.threshold_apply(v, thr).tobytes() == refimpl.threshold_apply(v, thr).tobytes()
    h0, l0 = oracle.threshold_apply_split(v, thr)
    h1, l1 = refimpl.threshold_apply_split(v, thr)
    assert h0.tobytes() == h1.tobytes() and l0.tobytes() == l1.tobytes()
    assert (h0 + l0 == v).all()
    # ThresholdTopK::apply = prepare + >= mask
    out, t = refimpl.topk_apply(v, np.float32(0.05))
    assert t == oracle.topk_prepare(v, np.float32(0.05))
    assert out.tobytes() == oracle.threshold_apply(v, t).tobytes()


# ---------------------------------------------------------------- channel level
@pytest.mark.parametrize("send_size_bytes", [False, True])
def test_write_remote_is_prepare_plus_compress(oracle, refimpl, send_size_bytes):
    """comprEx.tpp:176-191 composed from the compiled reference's two calls."""
    rng = np.random.default_rng(7)
    n = 20_000
    r0, r1 = np.zeros(n, np.float32), np.zeros(n, np.float32)
    for it in range(5):
        g = _rand(rng, n, np.float32)
        buf, thr = oracle.write_remote(r0, g, np.float32(0.01), send_size_bytes=send_size_bytes)
        thr_ref = refimpl.topk_prepare_with(r1, g, np.float32(0.01))
        msg_ref = refimpl.ip_compress(g, r1, thr_ref)
        off = 4 if send_size_bytes else 0
        assert thr == thr_ref and buf[off:].tobytes() == msg_ref.tobytes()
        if send_size_bytes:
            assert int(buf[:4].view(np.int32)[0]) == msg_ref.size
        assert r0.tobytes() == r1.tobytes()
    # writeRemote_NoResidual (comprEx.tpp:208-222)
    g = _rand(rng, n, np.float32)
    buf, thr = oracle.write_remote_noresidual(g, np.float32(0.01))
    thr_ref = refimpl.topk_prepare(g, np.float32(0.01))
    assert thr == thr_ref and buf.tobytes() == refimpl.ip_compress(g, None, thr_ref).tobytes()
    # flushRests (comprEx.tpp:128-142)
    r_before = r0.copy()
    buf = oracle.flush_rests(r0)
    assert buf.tobytes() == refimpl.ip_compress(r_before, None, np.float32(0)).tobytes()
    assert (r0 == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_rests_is_elementwise_sum_in_the_same_type(oracle, dtype):
    """comprEx.tpp:159-169 addRests: data[i] += rests[i], one addition per element in T.  Pinned by
    what the arithmetic fixes: numpy's same-dtype sum (IEEE round-to-nearest for the float types,
    wrap-free int sums), hand-picked fp32 cases where the sum rounds, and the mistakes a restatement
    could make (swapped operands' sign, rests modified, one element too few, a wider accumulator)."""
    rng = np.random.default_rng(11)
    for n in (0, 1, 2, 7, 1000, 4099):
        data = _rand(rng, n, dtype, 100.0)
        rests = _rand(rng, n, dtype, 3.0)
        want = (data + rests).astype(dtype)
        d, r = data.copy(), rests.copy()
        oracle.add_rests(d, r)
        assert d.tobytes() == want.tobytes()
        assert r.tobytes() == rests.tobytes(), "the residual itself is read-only here"
        if n:
            assert not np.array_equal(d, data - rests) or not rests.any()
    if dtype == np.float32:
        # sums that are not representable: 2^24 + 1 is a tie and rounds to even, 0.1f + 0.2f rounds in
        # fp32, 1 + (2^-24 + 2^-47) lies just above the halfway point and rounds up
        data = np.array([16777216.0, 0.1, 1.0, -0.0, 1e38, 1.0], np.float32)
        rests = np.array([1.0, 0.2, 2.0 ** -24 + 2.0 ** -47, 0.0, 3e38, -1.0], np.float32)
        d = data.copy()
        oracle.add_rests(d, rests)
        assert d[0] == np.float32(16777216.0) and d[1] == np.float32(0.1) + np.float32(0.2)
        assert d[2] == np.nextafter(np.float32(1.0), np.float32(2.0))
        assert d[3] == 0 and not np.signbit(d[3]) and np.isinf(d[4]) and d[5] == 0
    if dtype == np.int32:
        d = np.array([2147483000, -5, 7], np.int32)
        oracle.add_rests(d, np.array([647, 5, -9], np.int32))
        assert d.tolist() == [2147483647, 0, -2]


def test_exact_mode_survivor_count(oracle):
    """Exact top-k sends ceil_f32(n*topK)-1 pairs when magnitudes are distinct:
    the threshold is the (pos+1)-th largest magnitude and selection is strict '>'."""
    n = 1 << 16
    rng = np.random.default_rng(8)
    g = rng.permutation(n).astype(np.float32) - np.float32(0.25)  # distinct magnitudes
    g *= rng.choice(np.array([-1, 1], np.float32), n)
    r = np.zeros(n, np.float32)
    buf, thr = oracle.write_remote(r, g, np.float32(0.01), default_subsamples=1 << 17)
    k = parse_message(buf, np.float32)[1]
    assert k == oracle.topk_pos(n, np.float32(0.01)) == 655


# --------------------------------------------------------------------------- run-length codec
def _rle_parts(msg, dtype):
    n, c = msg[:8].view(np.int32)
    item = np.dtype(dtype).itemsize
    vals = msg[8:8 + c * item].view(dtype)
    runs, signum = msg[8 + c * item:16 + c * item].view(np.int32)
    lens = msg[16 + c * item:16 + c * item + 4 * runs].view(np.int32)
    assert msg.size == 16 + c * item + 4 * runs
    return int(n), vals, int(signum), lens


def test_rle_known_answers_by_hand(oracle):
    """Small messages written out by hand from the layout the reference's decoder reads
    (src/compressor.hxx:415-470): n, c, values, runs, signum, alternating run lengths."""
    v = np.array([5, 0, 0, -7, 8, 0], np.int32)
    n, vals, signum, lens = _rle_parts(oracle.rle_compress(v, None, np.int32(1)), np.int32)
    assert (n, vals.tolist(), signum, lens.tolist()) == (6, [5, -7, 8], 1, [1, 2, 2, 1])
    v = np.array([0, 0, 3, 0, 4, 4], np.int32)
    n, vals, signum, lens = _rle_parts(oracle.rle_compress(v, None, np.int32(3)), np.int32)
    assert (vals.tolist(), signum, lens.tolist()) == ([3, 4, 4], 0, [2, 1, 1, 2])
    # |x| >= threshold: an element equal to the threshold is sent (IndexPairs would keep it)
    n, vals, signum, lens = _rle_parts(oracle.rle_compress(v, None, np.int32(4)), np.int32)
    assert (vals.tolist(), signum, lens.tolist()) == ([4, 4], 0, [4, 2])
    # nothing sent: one "not sent" run over the whole vector
    n, vals, signum, lens = _rle_parts(oracle.rle_compress(v, None, np.int32(9)), np.int32)
    assert (vals.size, signum, lens.tolist()) == (0, 0, [6])
    # fused mode: update += data, sent entries cleared
    u, d = np.array([1, 1, 1, 1], np.float32), np.array([0, 2, -3, 0], np.float32)
    n, vals, signum, lens = _rle_parts(oracle.rle_compress(d, u, np.float32(2.5)), np.float32)
    assert (vals.tolist(), signum, lens.tolist()) == ([3.0], 0, [1, 1, 2]) and u.tolist() == [1, 0, -2, 1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_rle_encoder_equals_reference_where_the_reference_is_sound(oracle, refimpl, dtype):
    """The reference's encoder indexes the sent values by vector position; with every element
    sent (threshold 0: its own round-trip test, test/compressor.cpp:74-82) position and count
    coincide and its output is well formed: same bytes in all three modes."""
    rng = np.random.default_rng(5)
    for n in [1, 2, 17, 1000]:
        v = (rng.standard_normal(n) * 9).astype(dtype)
        a = (rng.standard_normal(n) * 3).astype(dtype)
        for mode in ("data", "update", "fused"):
            outs = []
            for impl in (oracle, refimpl):
                d = v.copy() if mode != "update" else None
                u = a.copy() if mode != "data" else None
                outs.append((impl.rle_compress(d, u, dtype(0)).tobytes(), None if u is None else u.tobytes()))
            assert outs[0] == outs[1], (n, mode)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rle_messages_decode_with_the_reference_decoder(oracle, refimpl, dtype):
    """Messages of the corrected encoder through the reference's own decoder and adder give the
    thresholded vector; the restated decoder and adder agree with the reference's byte for byte."""
    rng = np.random.default_rng(6)
    for n in [1, 2, 3, 64, 1000, 4097]:
        for q in [0.0, 0.3, 0.9, 0.99, 1.1]:
            v = (rng.standard_normal(n) * 50).astype(dtype)
            thr = dtype(np.quantile(np.abs(v), min(q, 1.0)) + (1 if q > 1 else 0))
            msg = oracle.rle_compress(v, None, thr)
            want = np.where(np.abs(v) >= thr, v, 0).astype(dtype)
            nn, vals, signum, lens = _rle_parts(msg, dtype)
            assert nn == n and lens.sum() == n and (lens > 0).all()
            assert vals.tobytes() == v[np.abs(v) >= thr].tobytes()
            assert signum == int(np.abs(v[0]) >= thr)
            for impl in (oracle, refimpl):
                out = np.full(n + 5, 77, dtype)
                assert impl.rle_decompress(msg, out) == n
                assert out[:n].tobytes() == want.tobytes() and (out[n:] == 77).all()  # nothing beyond n is touched
                acc = np.arange(n + 5).astype(dtype)
                impl.rle_add(msg, acc)
                assert acc[:n].tobytes() == (np.arange(n).astype(dtype) + want).astype(dtype).tobytes()
                with pytest.raises(RuntimeError):
                    impl.rle_decompress(msg, np.zeros(n - 1, dtype))


# ---------------------------------------------------------------- dense codec, FastComprEx
@pytest.mark.parametrize("dtype", DTYPES)
def test_none_codec_matches_ref(oracle, refimpl, dtype):
    """CompressorNone (compressor.hxx:83-151) against the compiled reference in its three modes;
    its adder only on full-length messages (the reference's reads past a shorter one)."""
    rng = np.random.default_rng(31)
    for n in (1, 5, 1000):
        d, u = _rand(rng, n, dtype), _rand(rng, n, dtype)
        for data, update in ((d, u), (None, u), (d, None)):
            u0 = None if update is None else update.copy()
            u1 = None if update is None else update.copy()
            m0 = oracle.none_compress(data, u0)
            m1 = refimpl.none_compress(data, u1)
            assert m0.tobytes() == m1.tobytes() and m0.size == 4 + n * np.dtype(dtype).itemsize
            if update is not None:
                assert u0.tobytes() == u1.tobytes() and not u0.any()
            o0, o1 = _rand(rng, n + 3, dtype), None
            o1 = o0.copy()
            assert oracle.none_decompress(m0, o0) == refimpl.none_decompress(m0, o1) == m0.size
            assert o0.tobytes() == o1.tobytes()
            a0 = _rand(rng, n, dtype)
            a1 = a0.copy()
            oracle.none_add(m0, a0)
            refimpl.none_add(m0, a1)
            assert a0.tobytes() == a1.tobytes()
    for impl in (oracle, refimpl):  # a message longer than the output is refused by both
        with pytest.raises(RuntimeError):
            impl.none_decompress(m0, np.zeros(n - 1, dtype))
        with pytest.raises(RuntimeError):
            impl.none_add(m0, np.zeros(n - 1, dtype))


def test_fast_comprex_is_the_reference_calls_one_step_late(oracle, refimpl):
    """comprEx.tpp:404-448 composed from the compiled reference's own threshold and compressor calls,
    line by line, against the restated state machine: what leaves at call i is what call i-1
    compressed (an empty message at the first call), a flush returns the unsent message to the
    residual before it sends everything."""
    rng = np.random.default_rng(41)
    n, topk = 5000, np.float32(0.02)
    fast = oracle.fast_comprex(n, np.float32, "ip", topK=topk)
    rests = np.zeros(n, np.float32)       # the reference side
    halves = [np.zeros(0, np.uint8), np.zeros(0, np.uint8)]
    phase, is_first, thr = 0, True, np.float32(0)
    script = "WWWFWFFWW"
    for step, op in enumerate(script):
        if op == "W":
            g = _rand(rng, n, np.float32)
            got = fast.write_remote(g)
            write, send = phase, (phase + 1) % 2
            if is_first:                                                  # :436-440
                halves[send] = refimpl.ip_compress(None, rests, thr)
                is_first = False
            want = halves[send]                                           # :442
            thr = refimpl.topk_prepare_with(rests, g, topk)               # :444
            halves[write] = refimpl.ip_compress(g, rests, thr)            # :446
            phase = (phase + 1) % 2                                       # :447
            if step == 0:
                assert want.size == 8 and want[4:8].view(np.int32)[0] == 0, "the first message is empty"
        else:
            got = fast.flush_rests()
            send = (phase + 1) % 2
            if not is_first:
                refimpl.ip_add(halves[send], rests)                       # :413
            halves[send] = refimpl.ip_compress(rests, None, np.float32(0))  # :415
            want = halves[send]                                           # :417
            rests[:] = 0                                                  # :418
            is_first = True                                               # :419
        assert got.tobytes() == want.tobytes(), (step, op)
        assert fast.rests.tobytes() == rests.tobytes(), (step, op)
        assert float(fast.thr.value) == float(thr)


@pytest.mark.parametrize("codec", ["ip", "rle", "none"])
@pytest.mark.parametrize("dtype", [np.float32, np.int32])
def test_fast_comprex_conserves_what_it_is_given(oracle, codec, dtype):
    """Whatever the codec: the messages that leave (each one call late) plus the flush add up to the
    inputs, exactly for integer-valued data (gold of test/comprex.cpp:73-75 applied to FastComprEx),
    and writeRemote_sameAs hands on the other channel's waiting message unchanged."""
    rng = np.random.default_rng(43)
    n = 3000
    add = {"ip": oracle.ip_add, "rle": oracle.rle_add, "none": oracle.none_add}[codec]
    a = oracle.fast_comprex(n, dtype, codec, topK=np.float32(0.05))
    b = oracle.fast_comprex(n, dtype, codec, topK=np.float32(0.05))
    total, got_a, got_b = np.zeros(n, dtype), np.zeros(n, dtype), np.zeros(n, dtype)
    for it in range(6):
        g = rng.integers(-50, 50, n).astype(dtype)
        total += g
        waiting_before = None if a.st[2] else a.halves[a.half_bytes * ((a.st[1] + 1) % 2):][:a.st[0]].copy()
        add(a.write_remote(g), got_a)
        msg_b = b.write_remote_same_as(a)
        add(msg_b, got_b)
        if it >= 1:  # b sends, one call late, what was waiting in a when b last copied
            assert msg_b.tobytes() == copied.tobytes()
        copied = a.halves[a.half_bytes * ((a.st[1] + 1) % 2):][:a.st[0]].copy()
    add(a.flush_rests(), got_a)
    assert np.array_equal(got_a, total) and not a.rests.any()


def test_reorder_bound_holds_for_other_orders_and_vanishes_for_single_contributions():
    """The bound the atomic reduce is held to, tried on the CPU: the same contributions summed in
    fp32 in rank order, in reverse order and in two shuffled orders stay within it of each other,
    ill-conditioned (cancelling) elements included; where one message contributes it is zero."""
    from oracle.pyoracle import reorder_bound
    rng = np.random.default_rng(3)
    n, ranks, k = 5000, 8, 1500
    msgs, pairs = [], []
    for r in range(ranks):
        idx = np.sort(rng.choice(n, k, replace=False)).astype(np.int32)
        val = (rng.standard_normal(k) * 10.0 ** rng.integers(-3, 4, k)).astype(np.float32)
        if r % 2:  # cancellation against the previous message wherever both hit
            prev_i, prev_v = pairs[-1]
            both = np.isin(idx, prev_i)
            val[both] = -prev_v[np.searchsorted(prev_i, idx[both])] * np.float32(1.0 + 2.0 ** -12)
        rec = np.zeros(k, np.dtype([("i", np.int32), ("v", np.float32)]))
        rec["i"], rec["v"] = idx, val
        msgs.append(np.concatenate([np.array([n, k], np.int32).view(np.uint8), rec.view(np.uint8)]))
        pairs.append((idx, val))
    bound = reorder_bound(msgs, np.float32, n)

    def summed(order, base=None):
        out = np.zeros(n, np.float32) if base is None else base.copy()
        for r in order:
            out[pairs[r][0]] += pairs[r][1]
        return out
    ref = summed(range(ranks))
    worst = 0.0
    for order in (range(ranks - 1, -1, -1), rng.permutation(ranks), rng.permutation(ranks)):
        diff = np.abs(summed(order).astype(np.float64) - ref.astype(np.float64))
        assert (diff <= bound).all()
        worst = max(worst, float((diff / np.maximum(bound, 1e-300)).max()))
    assert worst > 0.05          # not a vacuous bound: some element comes within a factor 20 of it
    count = np.zeros(n, np.int64)
    for i, _ in pairs:
        count[i] += 1
    assert ((bound == 0.0) == (count <= 1)).all()
    base = rng.standard_normal(n).astype(np.float32)
    bound_b = reorder_bound(msgs, np.float32, n, base)
    assert (np.abs(summed(range(ranks - 1, -1, -1), base).astype(np.float64) - summed(range(ranks), base)) <= bound_b).all()
    assert ((bound_b == 0.0) == (count == 0)).all()
