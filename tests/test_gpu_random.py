"""Seeded random sweeps of the GPU path against the checker: many small cases with mixed element
types, sizes around the tile and wavefront boundaries, unaligned sub-vectors, densities from
nothing to everything, clustered survivors, both codecs, every sampling rule."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DTYPES = [np.float32, np.float64, np.int32]


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def dev():
    from comprex_amd.device import Handle
    h = Handle()
    yield h
    h.synchronize()
    h.close()


def test_random_compress_both_codecs(dev, oracle):
    rng = np.random.default_rng(99)
    for case in range(150):
        dtype = DTYPES[case % 3]
        n = int(rng.choice([1, 7, 63, 64, 65, 1023, 1024, 1025, 4097, 100_003, 1_000_000]))
        off = int(rng.choice([0, 0, 1, 2, 3, 5]))  # element offset: sub-vectors that are not 16-byte aligned
        mode = ["fused", "update", "data"][(case // 3) % 3]
        dens = float(rng.choice([0.0, 1e-4, 0.003, 0.01, 0.1, 0.125, 0.2, 0.5, 0.9, 1.0]))
        codec = "rle" if case % 5 == 4 else "ip"
        scale = 1000 if dtype == np.int32 else 1
        d = (rng.standard_normal(n + off) * scale).astype(dtype)
        u = (rng.standard_normal(n + off) * scale * 0.5).astype(dtype)
        if rng.random() < 0.3:  # clustered survivors
            d[: max(1, n // 10)] *= 50
        ref = (d if mode == "data" else u if mode == "update" else (u + d).astype(dtype))[off:]
        mags = np.abs(ref.astype(np.float64))
        thr = dtype(0) if dens >= 1.0 else dtype(np.quantile(mags, 1 - dens)) if dens > 0 else dtype(mags.max() + 1)
        say("random compress", case, dtype.__name__, n, off, mode, dens, codec)
        dd = d[off:].copy() if mode != "update" else None
        uu = u[off:].copy() if mode != "data" else None
        want = (oracle.rle_compress if codec == "rle" else oracle.ip_compress)(dd, uu, thr)
        gd_full, gu_full = torch.from_numpy(d).cuda(), torch.from_numpy(u).cuda()
        gd = gd_full[off:] if mode != "update" else None
        gu = gu_full[off:] if mode != "data" else None
        item = np.dtype(dtype).itemsize
        cap = 16 + n * item + 4 * (n + 1) if codec == "rle" else 8 + n * (4 + item)
        buf = torch.zeros(cap + 4, dtype=torch.uint8, device="cuda")
        nb = (dev.rle_compress if codec == "rle" else dev.compress)(buf, gd, gu, thr=thr)
        assert nb == want.size and buf[:nb].cpu().numpy().tobytes() == want.tobytes()
        if gu is not None:  # the residual, and nothing in front of the sub-vector
            assert gu_full.cpu().numpy()[off:].tobytes() == uu.tobytes()
            assert gu_full.cpu().numpy()[:off].tobytes() == u[:off].tobytes()
        if gd is not None:
            assert gd_full.cpu().numpy().tobytes() == d.tobytes()


def test_random_thresholds_every_sampling_rule(dev, oracle):
    rng = np.random.default_rng(77)
    for case in range(60):
        n = int(rng.choice([50_000, 1_000_000, 3_000_003]))
        dtype = DTYPES[case % 3]
        kind = (case // 3) % 5
        if kind == 0:
            v = rng.standard_normal(n)
        elif kind == 1:  # per-block scales, as layers of a network have
            v = rng.standard_normal(n) * np.repeat(10.0 ** rng.uniform(-4, 0, n // 4096 + 1), 4096)[:n]
        elif kind == 2:  # many ties
            v = np.round(rng.standard_normal(n) * 3)
        elif kind == 3:  # mostly zeros
            v = rng.standard_normal(n) * (rng.random(n) < 0.02)
        else:  # the large values all at the front
            v = np.where(np.arange(n) < n // 30, rng.standard_normal(n) * 100, rng.standard_normal(n) * 0.01)
        if dtype == np.int32:
            v = v * 1000
        v = v.astype(dtype)
        a = (rng.standard_normal(n) * (1000 if dtype == np.int32 else 1) * 0.01).astype(dtype)
        m = min(int(rng.choice([8192, 9000, 65536, 100_000, 150_000, 262_144])), n)
        topk = np.float32(rng.choice([0.001, 0.005, 0.01, 0.03, 0.1]))
        idx = rng.integers(0, n, m).astype(np.int32)
        if case % 2:
            idx = np.sort(idx)
        ds = int(rng.choice([1000, 20000, 100000, 1 << 18, 1 << 22]))
        say("random threshold", case, dtype.__name__, n, kind, m, float(topk), ds)
        gv, ga = torch.from_numpy(v).cuda(), torch.from_numpy(a).cuda()
        assert dev.topk_threshold_indexed(gv, ga, torch.from_numpy(idx).cuda(), topk) == \
            oracle.topk_prepare_indexed(v, a, idx, topk)
        assert dev.topk_threshold(gv, ga, topk, ds, 10.0) == oracle.topk_prepare_with(v, a, topk, ds, 10.0)
        assert dev.topk_threshold(gv, None, topk, ds, 10.0) == oracle.topk_prepare(v, topk, ds, 10.0)


def test_random_thresholds_from_at_most_one_block_of_keys(dev, oracle):
    """Up to 1024 keys (ThresholdTopK's default is 1000 strided samples, src/threshold.hxx:130) are
    selected by one launch of one block: every sampling rule, lengths from 1 on, ties, all-zero and
    constant-magnitude vectors, top-k fractions from one key to all of them."""
    rng = np.random.default_rng(5)
    for case in range(240):
        dtype = DTYPES[case % 3]
        n = int(rng.choice([1, 2, 5, 63, 64, 65, 255, 256, 257, 1000, 1023, 1024, 1025, 5000, 61706, 1_000_003]))
        kind = int(rng.integers(0, 5))
        if kind == 0:
            v = rng.standard_normal(n)
        elif kind == 1:
            v = np.round(rng.standard_normal(n) * 2)
        elif kind == 2:
            v = rng.standard_normal(n) * (rng.random(n) < 0.05)
        elif kind == 3:
            v = np.zeros(n)
        else:
            v = np.full(n, 3.0) * rng.choice([-1, 1], n)
        if dtype == np.int32:
            v = v * 1000
        v = v.astype(dtype)
        a = (rng.standard_normal(n) * (10 if dtype == np.int32 else 0.01)).astype(dtype)
        topk = np.float32(rng.choice([0.0001, 0.001, 0.01, 0.1, 0.5, 0.999, 1.0]))
        ds = int(rng.choice([1, 7, 100, 1000, 1024]))
        m = int(rng.integers(1, 1025))
        idx = rng.integers(0, n, m).astype(np.int32)
        say("random one-block threshold", case, dtype.__name__, n, kind, float(topk), ds, m)
        gv, ga = torch.from_numpy(v).cuda(), torch.from_numpy(a).cuda()
        assert dev.topk_threshold(gv, ga, topk, ds, 10.0) == oracle.topk_prepare_with(v, a, topk, ds, 10.0)
        assert dev.topk_threshold(gv, None, topk, ds, 10.0) == oracle.topk_prepare(v, topk, ds, 10.0)
        assert dev.topk_threshold_indexed(gv, ga, torch.from_numpy(idx).cuda(), topk) == \
            oracle.topk_prepare_indexed(v, a, idx, topk)


def test_random_one_call_exact_topk(dev, oracle):
    from comprex_amd.device import message_capacity
    rng = np.random.default_rng(2024)
    thr_out = torch.zeros(1, device="cuda")
    routes = set()
    for case in range(12):
        n = int(rng.choice([1 << 23, (1 << 23) + 1, 9_999_999, 12_345_678]))
        topk = np.float32(rng.choice([0.0005, 0.001, 0.005, 0.01, 0.02, 0.05]))
        kind = case % 6
        if kind == 0:
            u = rng.standard_normal(n)
        elif kind == 1:
            u = rng.laplace(size=n)
            u[rng.integers(0, n, n // 10000)] = 1e3
        elif kind == 2:
            u = np.round(rng.standard_normal(n) * 4) / 4
        elif kind == 3:
            u = rng.standard_normal(n) * (rng.random(n) < 0.1)
        elif kind == 4:
            u = rng.standard_normal(n) * np.repeat(10.0 ** rng.uniform(-4, 0, n // 4096 + 1), 4096)[:n]
        else:
            u = rng.standard_normal(n) ** 3
        u = u.astype(np.float32)
        d = (rng.standard_normal(n) * rng.choice([0.0, 0.01, 1.0])).astype(np.float32)
        say("random one-call exact top-k", case, n, float(topk), kind)
        want_thr = oracle.topk_prepare_with(u, d, topk, 1 << 25, 10.0)
        uu = u.copy()
        want = oracle.ip_compress(d.copy(), uu, want_thr)
        gu, gd = torch.from_numpy(u).cuda(), torch.from_numpy(d).cuda()
        buf = torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")
        dev.set_option("fused_topk", 2 if case % 3 else 1)  # the single pass at these lengths, or what is faster
        try:
            nb = dev.compress_topk(buf, gd, gu, topk, d_thr=thr_out)
        finally:
            dev.set_option("fused_topk", 1)
        routes.add(dev.get_option("fused_topk_taken"))
        assert thr_out.item() == want_thr and nb == want.size
        assert buf[:nb].cpu().numpy().tobytes() == want.tobytes()
        assert gu.cpu().numpy().tobytes() == uu.tobytes()
    assert 1 in routes


def test_random_write_step_across_the_selection_paths(dev, oracle):
    """cx_ip_write_step on vector lengths on both sides of every limit between the selection paths (two
    launches / chained passes / one candidate pass / single pass over both vectors), strided sample or
    whole vector, three element types, inputs of several kinds, two residual-carrying steps each:
    threshold, message and residual are the checker's."""
    from comprex_amd.device import message_capacity
    rng = np.random.default_rng(99)
    np2t = {np.float32: torch.float32, np.float64: torch.float64, np.int32: torch.int32}
    sizes = [1, 63, 4097, 40_960, 40_961, 100_000, 262_144, 262_145, 1 << 20, (1 << 22) + 1, (10 << 20) - 1, 10 << 20,
             12_000_001, (20 << 20) - 4, (20 << 20) + 4]
    routes = set()
    for case, n in enumerate(sizes + sizes):
        dtype = [np.float32, np.float64, np.int32][case % 3]
        if dtype == np.float64 and n > 12_000_000:
            dtype = np.float32
        topk = np.float32(rng.choice([0.0005, 0.01, 0.04, 0.1, 0.3]))
        ds = 1000 if case % 4 == 3 else 1 << 30  # strided sample now and then, else the whole vector
        kind = int(rng.integers(0, 4))
        scale = 1000 if dtype == np.int32 else 1

        def grad():
            if kind == 0:
                v = rng.standard_normal(n)
            elif kind == 1:  # stretches of different scale
                v = rng.standard_normal(n) * np.repeat(10.0 ** rng.uniform(-4, 0, n // 4096 + 1), 4096)[:n]
            elif kind == 2:  # ties
                v = np.round(rng.standard_normal(n) * 3)
            else:            # mostly zeros
                v = rng.standard_normal(n) * (rng.random(n) < 0.05)
            return (v * scale).astype(dtype)

        say("random write_step", case, dtype.__name__, n, float(topk), ds, kind)
        r_h = np.zeros(n, dtype)
        r = torch.zeros(n, dtype=np2t[dtype], device="cuda")
        buf = torch.zeros(message_capacity(n, np2t[dtype]), dtype=torch.uint8, device="cuda")
        thr_out = torch.zeros(1, dtype=np2t[dtype], device="cuda")
        for _ in range(2):
            g_h = grad()
            g = torch.from_numpy(g_h).cuda()
            nb = dev.write_step(buf, g, r, topk, ds, 10.0, d_thr=thr_out)
            want_thr = oracle.topk_prepare_with(r_h, g_h, topk, ds, 10.0)
            want = oracle.ip_compress(g_h, r_h, dtype(want_thr))
            assert thr_out.cpu().numpy()[0] == dtype(want_thr), (case, n)
            assert nb == want.size and buf[:nb].cpu().numpy().tobytes() == want.tobytes(), (case, n)
            assert r.cpu().numpy().tobytes() == r_h.tobytes(), (case, n)
        routes.add(dev.get_option("fused_topk_taken"))
    assert 1 in routes or 2 in routes  # the single pass was among them


def test_write_step_on_sub_vectors_that_are_not_16_byte_aligned(dev, oracle):
    """cx_ip_write_step on vectors that start 1 or 3 elements into an allocation (scalar loads in every
    kernel of the step, the last pick of a chained selection made by the compress pass): threshold, message
    and residual are the checker's, and nothing in front of the sub-vector is touched."""
    from comprex_amd.device import message_capacity
    rng = np.random.default_rng(3)
    np2t = {np.float32: torch.float32, np.float64: torch.float64, np.int32: torch.int32}
    for dtype in (np.float32, np.float64, np.int32):
        for n in (4097, 100_003, 1_000_001):
            for off in (1, 3):
                for ds in (1 << 30, 1000):
                    topk = np.float32(rng.choice([0.001, 0.02, 0.2]))
                    scale = 1000 if dtype == np.int32 else 1
                    g_full = (rng.standard_normal(n + off) * scale).astype(dtype)
                    r_full = (0.3 * rng.standard_normal(n + off) * scale).astype(dtype)
                    g_h, r_h = g_full[off:].copy(), r_full[off:].copy()
                    gg, rr = torch.from_numpy(g_full).cuda(), torch.from_numpy(r_full).cuda()
                    say("unaligned write_step", dtype.__name__, n, off, ds, float(topk))
                    buf = torch.zeros(message_capacity(n, np2t[dtype]), dtype=torch.uint8, device="cuda")
                    thr_out = torch.zeros(1, dtype=np2t[dtype], device="cuda")
                    nb = dev.write_step(buf, gg[off:], rr[off:], topk, ds, 10.0, d_thr=thr_out)
                    want_thr = oracle.topk_prepare_with(r_h, g_h, topk, ds, 10.0)
                    want = oracle.ip_compress(g_h, r_h, dtype(want_thr))
                    assert thr_out.cpu().numpy()[0] == dtype(want_thr)
                    assert nb == want.size and buf[:nb].cpu().numpy().tobytes() == want.tobytes()
                    back = rr.cpu().numpy()
                    assert back[off:].tobytes() == r_h.tobytes() and back[:off].tobytes() == r_full[:off].tobytes()
                    assert gg.cpu().numpy().tobytes() == g_full.tobytes()
