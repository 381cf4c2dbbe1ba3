"""The drop-in layers above the kernels, on the GPU: the C++ classes (driven by C++ tests that
mirror the reference's own) and the reference's float C ABI behind its Python wrappers."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle.pyoracle import parse_message

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin")


@pytest.mark.parametrize("name", ["threshold_test", "compressor_test", "comprex_test", "fast_comprex_test", "allreduce_test",
                                  "tf_ops_test", "capi_test", "streams_test"])
def test_cpp_mirror_of_reference_tests(name):
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "build tests/cpp first (make -C tests/cpp, or __graft_entry__.build())"
    print("running", exe, file=sys.stderr, flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    sys.stderr.write(r.stdout[-3000:] + r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-2000:]
    assert "+++ PASSED +++" in r.stdout and "--- FAILED ---" not in r.stdout


@pytest.mark.parametrize("name,passes", [("refsrc_threshold", 2), ("refsrc_compressor", 2)])
def test_reference_own_test_sources_against_these_headers(name, passes):
    """test/threshold.cpp and test/compressor.cpp of the reference, compiled UNCHANGED with this
    repository's include/ in front of the reference's src/ (tests/cpp/Makefile, target refsrc) and
    linked to the HIP library: the drop-in claim at the C++ source level.  The binaries exist where
    the reference tree was present at build time."""
    exe = os.path.join(BIN, name)
    if not os.path.exists(exe):
        pytest.skip("built only where the reference tree is present")
    print("running", exe, file=sys.stderr, flush=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    sys.stderr.write(r.stdout[-2000:] + r.stderr[-2000:])
    assert r.returncode == 0
    assert r.stdout.count("+++ PASSED +++") == passes and "--- FAILED ---" not in r.stdout


def _pair(env, n, size_factor=3.0, topk=0.01, tag=1, compressor="CompressorIndexPairs"):
    from comprex_amd import pygpi
    objs = []
    for rank in range(2):
        env.set_rank(rank, 2)
        c = pygpi.Comprex(env, n, size_factor)
        c.setThreshold(pygpi.ThresholdTopK(topk))
        c.setCompressor(getattr(pygpi, compressor)())
        c.connectTo((rank + 1) % 2, (rank + 1) % 2, tag)
        objs.append(c)
    return objs


@pytest.mark.parametrize("on_device", [False, True])
def test_reference_abi_matches_oracle(oracle, on_device):
    """Comprex.writeRemote / readRemote / flushRests through the reference's symbol set, against
    the checker's writeRemote (default ThresholdTopK: 1000 strided samples), bit for bit."""
    from comprex_amd import pygpi
    n, topk = 200_003, np.float32(0.01)
    env = pygpi.GaspiEnvironment()
    tx, rx = _pair(env, n, topk=float(topk))
    rng = np.random.default_rng(31)
    rests = np.zeros(n, np.float32)
    for it in range(6):
        g = rng.standard_normal(n).astype(np.float32)
        want_msg, want_thr = oracle.write_remote(rests, g, topk)
        tx.writeRemote(torch.from_numpy(g).cuda() if on_device else g)
        want_dense = np.zeros(n, np.float32)
        oracle.ip_decompress(want_msg, want_dense)
        if on_device:
            got = torch.empty(n, device="cuda")
            rx.readRemote(got)
            got = got.cpu().numpy()
        else:
            got = rx.readRemote()
        assert got.tobytes() == want_dense.tobytes()
        assert tx.getRests().tobytes() == rests.tobytes()
    want_flush = oracle.flush_rests(rests)
    tx.flushRests()
    acc = np.ones(n, np.float32)
    want_acc = acc.copy()
    oracle.ip_add(want_flush, want_acc)
    rx.readRemote_add(acc)
    assert acc.tobytes() == want_acc.tobytes()
    assert not tx.getRests().any()


@pytest.mark.parametrize("compressor", ["CompressorIndexPairs", "CompressorRLE", "CompressorNone"])
def test_reference_abi_conservation_and_errors(compressor):
    """test/comprex.cpp's gold through the Python wrappers with each codec, plus the errors the
    reference throws."""
    from comprex_amd import pygpi
    n = 50
    env = pygpi.GaspiEnvironment()
    tx, rx = _pair(env, n, topk=0.1, compressor=compressor)
    i = np.arange(n)
    values = (i * (1 - 2 * (i % 2))).astype(np.float32)
    result = np.zeros(n, np.float32)
    for run in range(4):
        if run < 3:
            tx.writeRemote(values)
        else:
            tx.flushRests()
        rx.readRemote_add(result)
    assert (result == 3 * values).all()
    with pytest.raises(RuntimeError, match="no message pending"):
        rx.readRemote()
    with pytest.raises(RuntimeError):
        tx.writeRemote(values[:-1].copy())
    lone = pygpi.Comprex(env, n)
    with pytest.raises(RuntimeError, match="without connecting"):
        lone.writeRemote(values)
    with pytest.raises(RuntimeError, match="between 0.0 and 1.0"):
        pygpi.ThresholdTopK(1.5)
    with pytest.raises(RuntimeError):
        pygpi.ThresholdConst(-1.0)
    t = pygpi.ThresholdConst(2.5)
    assert t.getThreshold() == 2.5


def test_simulated_all_to_one_reduce_matches_oracle(oracle):
    """Config-5 shaped flow at a small size: R workers' messages reduced by the chief in rank
    order (src/allreduce.tpp:183-189), then the chief's broadcast-leg writeRemote applies the
    reduced vector to its residual (:205).  Checked against the checker's sequential loop."""
    from comprex_amd import pygpi
    R, n, topk = 5, 300_007, np.float32(0.01)
    env = pygpi.GaspiEnvironment()
    workers, chief_rx = [], []
    for r in range(1, R):
        env.set_rank(r, R)
        w = pygpi.Comprex(env, n, 3.0)
        w.setThreshold(pygpi.ThresholdTopK(float(topk)))
        w.setCompressor(pygpi.CompressorIndexPairs())
        w.connectTx(0, 100 + r)
        workers.append(w)
    env.set_rank(0, R)
    for r in range(1, R):
        c = pygpi.Comprex(env, n, 3.0)
        c.setCompressor(pygpi.CompressorIndexPairs())
        c.connectRx(r, 100 + r)
        chief_rx.append(c)
    bc = pygpi.Comprex(env, n, 3.0)
    bc.setThreshold(pygpi.ThresholdTopK(float(topk)))
    bc.setCompressor(pygpi.CompressorIndexPairs())
    bc.connectTx(1, 200)
    rng = np.random.default_rng(41)
    o_rests = [np.zeros(n, np.float32) for _ in range(R)]
    o_bc = np.zeros(n, np.float32)
    for it in range(3):
        grads = [rng.standard_normal(n).astype(np.float32) for _ in range(R)]
        dense = torch.from_numpy(grads[0]).cuda()
        want = grads[0].copy()
        for r in range(1, R):
            workers[r - 1].writeRemote(torch.from_numpy(grads[r]).cuda())
            msg, _ = oracle.write_remote(o_rests[r], grads[r], topk)
            oracle.ip_add(msg, want)
        for r in range(1, R):
            chief_rx[r - 1].readRemote_add(dense)
        assert dense.cpu().numpy().tobytes() == want.tobytes()
        bc.writeRemote(dense)
        oracle.write_remote(o_bc, want, topk)
        assert bc.getRests().tobytes() == o_bc.tobytes()


@pytest.mark.parametrize("family", ["Comprex_AllToOneAllreduce", "Comprex_RingAllreduce", "Comprex_BigRingAllreduce"])
def test_allreduce_schedules_from_python_threads(family):
    """The reference's Python allreduce tests (test/AllToOneAllreduce.py etc.): one thread per rank,
    device tensors handed to apply/flush in place, gold (num_runs*(numRanks-1)+1)*values."""
    import threading
    from comprex_amd import pygpi
    R, n, runs = 3, 30_000, 4
    env = pygpi.GaspiEnvironment()
    env.set_rank(0, R)
    env.set_blocking(True, 60.0)
    i = np.arange(n)
    values = ((i % 251) * (1 - 2 * (i % 2))).astype(np.float32)
    gold = (runs * (R - 1) + 1) * values
    results, errors = {}, []

    def rank_program(rank):
        try:
            env.set_rank(rank, R)
            ar = getattr(pygpi, family)(env)
            if family == "Comprex_AllToOneAllreduce":
                ar.setup_connections(n, 0, 0, 1e-2, 3.0)
            else:
                ar.setup_connections(n, 0, 1e-2, 3.0)
            env.barrier()
            result = torch.from_numpy(values).cuda()
            for run in range(runs):
                env.barrier()
                if family == "Comprex_RingAllreduce":
                    seg = n // R
                    lo = ((rank + 1) % R) * seg
                    keep = result[lo:lo + seg].clone()
                    result.copy_(torch.from_numpy(values))
                    result[lo:lo + seg] = keep
                elif rank != 0:
                    result.copy_(torch.from_numpy(values))
                ar.apply(result)
            ar.flush(result)
            results[rank] = result.cpu().numpy()
            env.barrier()
        except Exception as e:  # noqa: BLE001
            errors.append((rank, repr(e)))

    threads = [threading.Thread(target=rank_program, args=(r,)) for r in range(R)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
    checked = range(R) if family == "Comprex_RingAllreduce" else [0]
    for r in checked:
        assert (results[r] == gold).all(), (family, r)


def test_optimizer_single_rank_matches_reference_formula():
    """keras/comprex_optimizer.py:134-141,155-163: m = momentum*m + g; w = (1-wd)*w - m."""
    from comprex_amd import pygpi
    from comprex_amd.optimizer import ComprexOptimizer
    env = pygpi.GaspiEnvironment()
    w = torch.nn.Parameter(torch.arange(6, dtype=torch.float32, device="cuda"))
    opt = ComprexOptimizer([w], env, learning_rate=0.5, momentum=0.9, weight_decay=0.1)
    want_w, m = w.detach().clone(), torch.zeros(6, device="cuda")
    for step in range(3):
        w.grad = torch.full((6,), float(step + 1), device="cuda")
        opt.step()
        m = 0.9 * m + w.grad
        want_w = (1 - 0.1) * want_w - m
        assert torch.equal(w.detach(), want_w)
    with pytest.raises(ValueError):
        ComprexOptimizer([w], env, allreduce_type="nope")


@pytest.mark.parametrize("schedule", ["comprex_alltoone", "comprex_ring", "comprex_bigring"])
def test_optimizer_trains_over_simulated_ranks(schedule):
    """Three ranks (threads), each with its own data shard, fit a shared linear model through the
    compressed allreduce; the loss of every rank's replica on the full data drops."""
    import threading
    from comprex_amd import pygpi
    from comprex_amd.optimizer import ComprexOptimizer
    R, dim, steps = 3, 4096, 40
    env = pygpi.GaspiEnvironment()
    env.set_rank(0, R)
    env.set_blocking(True, 60.0)
    gen = torch.Generator().manual_seed(5)
    target = torch.randn(dim, generator=gen)
    xs = torch.randn(R, 64, dim, generator=gen)
    ys = xs @ target
    losses, errors = {}, []

    def full_loss(w):
        return float(((xs.reshape(-1, dim).cuda() @ w - ys.reshape(-1).cuda()) ** 2).mean())

    def rank_program(rank):
        try:
            env.set_rank(rank, R)
            w = torch.nn.Parameter(torch.zeros(dim, device="cuda"))
            opt = ComprexOptimizer([w], env, learning_rate=2e-4, momentum=0.5, compression_ratio=0.05,
                                   allreduce_type=schedule, size_factor=3.0, pre_clipnorm=1e9)
            x, y = xs[rank].cuda(), ys[rank].cuda()
            first = full_loss(w.detach())
            for _ in range(steps):
                env.barrier()
                loss = ((x @ w - y) ** 2).mean()
                w.grad = torch.autograd.grad(loss, w)[0]
                opt.step()
            losses[rank] = (first, full_loss(w.detach()))
            env.barrier()
        except Exception as e:  # noqa: BLE001
            errors.append((rank, repr(e)))

    threads = [threading.Thread(target=rank_program, args=(r,)) for r in range(R)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(180)
    assert not errors, errors
    for rank, (first, last) in losses.items():
        assert np.isfinite(last) and last < 0.7 * first, (schedule, rank, first, last)


@pytest.mark.parametrize("schedule", ["comprex_alltoone", "comprex_ring", "comprex_bigring"])
def test_optimizer_over_ranks_adds_up_to_the_closed_form(schedule):
    """Four ranks, five steps, integer gradients, momentum 1/2, learning rate 1, no clipping, no weight
    decay: every momentum term is a dyadic rational, so every sum below is exact in fp32 whatever
    the compressor holds back and in whatever order it is added.  What the compressed allreduce
    delays it delivers with the flush, so after the steps plus one flush (applied like a step)

        w = w0 - (1/R) * sum over ranks q and steps s of m[q][s],   m[q][s] = m[q][s-1] / 2 + g[q][s]

    wherever the schedule delivers everything: on every rank for the big ring, on the chief for
    all-to-one (its broadcast is compressed without a flush, src/allreduce.tpp:196-239), and for
    the ring on the segment a rank finishes itself (the others arrive thresholded, without a
    residual, src/allreduce.tpp:441-457).  The expectation is computed here in float64 from the
    gradients alone; nothing of the library or the checker takes part in it."""
    import threading
    from comprex_amd import pygpi
    from comprex_amd.optimizer import ComprexOptimizer
    R, dim, steps = 4, 6002, 5
    rng = np.random.default_rng(77)
    grads = rng.integers(-8, 9, (R, steps, dim)).astype(np.float64)
    grads[:, :, ::7] *= 16                       # a heavy tail, so that the top-k has something to prefer
    w0 = rng.integers(-100, 101, dim).astype(np.float64)
    m = np.zeros((R, dim))
    total = np.zeros(dim)
    for s in range(steps):
        m = 0.5 * m + grads[:, s]
        total += m.sum(axis=0)
    want = (w0 - total / R).astype(np.float32)
    assert (want.astype(np.float64) == w0 - total / R).all()   # the expectation itself is exact in fp32
    env = pygpi.GaspiEnvironment()
    env.set_rank(0, R)
    env.set_blocking(True, 60.0)
    got, held_back, errors = {}, {}, []

    def rank_program(rank):
        try:
            env.set_rank(rank, R)
            w = torch.nn.Parameter(torch.from_numpy(w0.astype(np.float32)).cuda())
            opt = ComprexOptimizer([w], env, learning_rate=1.0, momentum=0.5, compression_ratio=0.05,
                                   allreduce_type=schedule, size_factor=3.0, pre_clipnorm=1e30)
            for s in range(steps):
                env.barrier()
                w.grad = torch.from_numpy(grads[rank, s].astype(np.float32)).cuda()
                opt.step()
            env.barrier()
            # what is still held back arrives with the flush; it is applied like a step
            opt.blob.zero_()
            opt.allreduce.flush(opt.blob)
            held_back[rank] = int(torch.count_nonzero(opt.blob))
            with torch.no_grad():
                w.sub_(opt.blob / R)
            got[rank] = w.detach().cpu().numpy()
            env.barrier()
        except Exception as e:  # noqa: BLE001
            errors.append((rank, repr(e)))

    threads = [threading.Thread(target=rank_program, args=(r,)) for r in range(R)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(180)
    assert not errors, errors
    if schedule == "comprex_bigring":
        for r in range(R):
            assert (got[r] == want).all(), (schedule, r)
        assert all(held_back[r] > 0 for r in range(R))       # the compressor did hold something back
    elif schedule == "comprex_alltoone":
        assert (got[0] == want).all()
        assert held_back[0] > 0
    else:
        sizes = [dim // R + (1 if c < dim % R else 0) for c in range(R)]
        starts = np.concatenate([[0], np.cumsum(sizes)])
        for r in range(R):
            c = (r + 1) % R
            assert (got[r][starts[c]:starts[c + 1]] == want[starts[c]:starts[c + 1]]).all(), (schedule, r)
        assert all(held_back[r] > 0 for r in range(R))


def test_exact_whole_vector_step_can_be_captured_in_a_hip_graph(oracle):
    """The exact whole-vector threshold on a long vector (sampled bound, candidate pass, radix passes
    that read the candidate count on the device) and the compress behind it wait for nothing, so they
    can be captured: two steps replayed three times, with eager work and synchronisations between the
    replays, give the eager result every time, and the eager result is the checker's."""
    from comprex_amd.device import Handle, message_capacity
    rng = np.random.default_rng(43)
    n = 11_000_001
    g_h = rng.laplace(size=n).astype(np.float32)
    g = torch.from_numpy(g_h).cuda()
    rests = torch.zeros(n, device="cuda")
    msg = torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        h = Handle()
        h.reserve(n, torch.float32, Handle.RESERVE_ALL)

        def step():
            h.topk_threshold(rests, g, np.float32(0.002), 1 << 30, to_host=False)
            h.compress(msg, g, rests, sync=False)

        for _ in range(2):
            step()
        side.synchronize()
        rests.zero_()
        step(), step()
        side.synchronize()
        want_rests = rests.clone()
        want_msg = msg[: 8 + 8 * int(msg[4:8].view(torch.int32).item())].clone()
        # the checker on the same two steps
        r_h = np.zeros(n, np.float32)
        for _ in range(2):
            thr = oracle.topk_prepare_with(r_h, g_h, np.float32(0.002), 1 << 30, 10.0)
            ref_msg = oracle.ip_compress(g_h, r_h, np.float32(thr))
        assert want_msg.cpu().numpy().tobytes() == ref_msg.tobytes()
        assert want_rests.cpu().numpy().tobytes() == r_h.tobytes()
        rests.zero_()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(), step()
        side.synchronize()
        for _ in range(3):
            rests.zero_()
            msg.zero_()
            side.synchronize()
            graph.replay()
            side.synchronize()
            k = int(msg[4:8].view(torch.int32).item())
            assert torch.equal(rests, want_rests)
            assert torch.equal(msg[: 8 + 8 * k], want_msg)
        h.synchronize()
        h.close()


def test_sampled_step_can_be_captured_in_a_hip_graph():
    """threshold (left on the device) + compress enqueue kernels only, so a caller may capture them.
    Two steps (one in each walking direction) are captured and replayed three times, with eager
    work and synchronisations in between; every replay gives the eager result."""
    from comprex_amd.device import Handle, message_capacity
    rng = np.random.default_rng(41)
    n, m = 3_000_000, 20_000
    g = torch.from_numpy(rng.laplace(size=n).astype(np.float32)).cuda()
    idx = torch.from_numpy(rng.integers(0, n, m).astype(np.int32)).cuda()
    rests = torch.zeros(n, device="cuda")
    msg = torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        h = Handle()

        def step():
            h.topk_threshold_indexed(rests, g, idx, np.float32(0.01), to_host=False)
            h.compress(msg, g, rests, sync=False)

        for _ in range(2):  # scratch is allocated by now
            step()
        side.synchronize()
        start = rests.clone()
        step(), step()
        side.synchronize()
        want_rests = rests.clone()
        want_msg = msg[: 8 + 8 * int(msg[4:8].view(torch.int32).item())].clone()
        rests.copy_(start)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(), step()
        side.synchronize()
        for _ in range(3):
            rests.copy_(start)
            msg.zero_()
            side.synchronize()
            graph.replay()
            side.synchronize()
            k = int(msg[4:8].view(torch.int32).item())
            assert torch.equal(rests, want_rests)
            assert torch.equal(msg[: 8 + 8 * k], want_msg)
        h.synchronize()


def test_handle_on_a_stream_of_its_own_starts_from_clean_state(oracle):
    """A handle created on a non-blocking stream clears its status words, select state and flags on
    THAT stream before cx_create returns (the null stream, where a plain memset runs, is not ordered
    with such a stream): device memory that held other bytes just before must not show through as a
    device-side error or a wrong threshold."""
    import ctypes as C
    from comprex_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(3)
    n = 20_000
    v_h = rng.standard_normal(n).astype(np.float32)
    v = torch.from_numpy(v_h).cuda()
    want = oracle.topk_prepare(v_h, np.float32(0.05), 1 << 20, 10.0)
    junk_h = np.full(1 << 16, 0x5a5a5a5a, np.uint32)
    torch.cuda.synchronize()
    for _ in range(25):
        # bytes other than zero in memory of the sizes a handle allocates, then free it again
        held = []
        for size in (256, 256, 256, 1 << 16, 1 << 17):
            p = C.c_void_p()
            _lib.check(L.cx_device_alloc(C.byref(p), size))
            held.append((p, size))
        tmp = C.c_void_p()
        _lib.check(L.cx_create(C.byref(tmp), None))
        for p, size in held:
            _lib.check(L.cx_copy(tmp, p, C.c_void_p(junk_h.ctypes.data), size))
        _lib.check(L.cx_synchronize(tmp))
        for p, _size in held:
            _lib.check(L.cx_device_free(p))
        L.cx_destroy(tmp)
        stream, h = C.c_void_p(), C.c_void_p()
        _lib.check(L.cx_stream_create(C.byref(stream)))
        _lib.check(L.cx_create(C.byref(h), stream))
        try:
            _lib.check(L.cx_synchronize(h))  # a status word that is not zero would be reported here
            thr = C.c_float(0)
            _lib.check(L.cx_topk_threshold(h, _lib.CX_F32, C.c_void_p(v.data_ptr()), None, n, 0, C.c_float(0.05),
                                           1 << 20, C.c_float(10.0), None, C.byref(thr)))
            assert thr.value == want
        finally:
            L.cx_destroy(h)
            L.cx_stream_destroy(stream)
