"""The five benchmark configurations at their full sizes, on the GPU.

Three kinds of evidence per configuration:
  * the outputs of the COMPILED REFERENCE recorded in tests/golden/full_size.json (threshold
    bits, pair count, checksums of message and residual), compared when the inputs regenerate
    to the recorded checksum;
  * the CPU checker run live on the same buffers where that takes seconds;
  * size-independent properties (ascending indices, k == #{|r+g| > t}, conservation).
"""
import json
import os
import sys

import numpy as np
import pytest
import torch

from comprex_amd import workloads as W
from oracle.pyoracle import reorder_bound

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "full_size.json")))


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def dev():
    from comprex_amd.device import Handle
    h = Handle()
    yield h
    h.synchronize()
    h.close()


def _msgbuf(n):
    from comprex_amd.device import message_capacity
    return torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")


def _hex(x):
    return np.float32(x).tobytes().hex()


def _error_feedback(dev, oracle, cfg, grad_fn, iters, gold_rows, oracle_live=True, fused_route=None):
    """fused_route: None = threshold call then compress call; else the single call
    (cx_ip_compress_topk) is used and must report that route."""
    n, topk, ds = cfg["n"], np.float32(cfg["topK"]), cfg["default_subsamples"]
    rests = torch.zeros(n, device="cuda")
    rests_h = np.zeros(n, np.float32)
    buf = _msgbuf(n)
    thr_out = torch.zeros(1, device="cuda")
    compared = 0
    for it in range(iters):
        g_h = grad_fn(it)
        g = torch.from_numpy(g_h).cuda()
        if fused_route == "step":
            # threshold and compress enqueued by ONE call (what ComprEx::writeRemote uses)
            nbytes = dev.write_step(buf, g, rests, topk, ds, d_thr=thr_out)
            thr = float(thr_out.item())
        elif fused_route is None:
            thr = dev.topk_threshold(rests, g, topk, ds)
            nbytes = dev.compress(buf, g, rests)  # threshold from the handle's device slot
        else:
            assert ds > n, "the single call is the whole-vector mode"
            nbytes = dev.compress_topk(buf, g, rests, topk, d_thr=thr_out)
            thr = float(thr_out.item())
            assert dev.get_option("fused_topk_taken") == fused_route
        msg = buf[:nbytes].cpu().numpy()
        k = int(msg[4:8].view(np.int32)[0])
        say(cfg["name"], "iter", it, "thr", thr, "k", k)
        idx = msg[8:].view(np.dtype([("i", np.int32), ("v", np.float32)]))["i"]
        assert (np.diff(idx) > 0).all() and nbytes == 8 + 8 * k
        if oracle_live:
            want_msg, want_thr = oracle.write_remote(rests_h, g_h, topk, ds)
            assert thr == want_thr and msg.tobytes() == want_msg.tobytes()
            assert rests.cpu().numpy().tobytes() == rests_h.tobytes()
        if it < len(gold_rows) and gold_rows[it]["input"] == W.checksum(g_h):
            row = gold_rows[it]
            assert _hex(thr) == row["thr_hex"] and k == row["k"]
            assert W.checksum(msg) == row["msg"]
            assert W.checksum(rests.cpu().numpy()) == row["rests"]
            compared += 1
    return compared


def test_c1_one_million_top1pct_ten_iterations(dev, oracle):
    compared = _error_feedback(dev, oracle, W.C1, W.c1_gradient, W.C1["iters"], GOLD["C1"])
    assert compared == W.C1["iters"], "inputs did not regenerate to the recorded bits"


def test_c2_lenet5_top10pct_fifty_iterations(dev, oracle):
    compared = _error_feedback(dev, oracle, W.C2, W.c2_gradient, W.C2["iters"], GOLD["C2"])
    assert compared == W.C2["iters"]


def test_c1_and_c3_threshold_and_compress_as_one_call(dev, oracle):
    # C1 is too small for the single pass (route 0), C3 takes it (route 1); same recorded outputs
    assert _error_feedback(dev, oracle, W.C1, W.c1_gradient, 3, GOLD["C1"], fused_route=0) == 3
    assert _error_feedback(dev, oracle, W.C3, W.c3_gradient, 3, GOLD["C3"], fused_route=1) == 3


def test_c1_c2_c3_write_step_one_call(dev, oracle):
    """cx_ip_write_step on the reference's configurations: chained radix passes (C1), the two-launch
    select (C2), the single pass over both vectors (C3); the recorded reference outputs and the
    live checker."""
    assert _error_feedback(dev, oracle, W.C1, W.c1_gradient, W.C1["iters"], GOLD["C1"], fused_route="step") == W.C1["iters"]
    assert _error_feedback(dev, oracle, W.C2, W.c2_gradient, W.C2["iters"], GOLD["C2"], fused_route="step") == W.C2["iters"]
    assert _error_feedback(dev, oracle, W.C3, W.c3_gradient, 4, GOLD["C3"], fused_route="step") == 4


def test_c3_resnet50_top0p1pct(dev, oracle):
    # all 20 residual-carrying iterations: recorded reference outputs and a live checker run
    compared = _error_feedback(dev, oracle, W.C3, W.c3_gradient, W.C3["iters"], GOLD["C3"])
    assert compared == W.C3["iters"] == 20


def test_c4_hundred_million_laplace(dev, oracle):
    g_h = W.c4_gradient()
    n = g_h.size
    assert W.checksum(g_h) == GOLD["C4"]["input"], "inputs did not regenerate to the recorded bits"
    g = torch.from_numpy(g_h).cuda()
    buf = _msgbuf(n)
    topk = np.float32(W.C4["topK"])

    def run(kind, thr_fn):
        rests = torch.zeros(n, device="cuda")
        thr = thr_fn(rests)
        nbytes = dev.compress(buf, g, rests)
        msg = buf[:nbytes].cpu().numpy()
        k = int(msg[4:8].view(np.int32)[0])
        row = GOLD["C4"][kind]
        say("C4", kind, "thr", thr, "k", k)
        assert _hex(thr) == row["thr_hex"] and k == row["k"]
        assert W.checksum(msg) == row["msg"]
        r = rests.cpu().numpy()
        assert W.checksum(r) == row["rests"]
        # properties: k == #{|g| > thr}; sent entries are +0 in the residual, the rest equals g
        sel = np.abs(g_h) > np.float32(thr)
        assert k == int(np.count_nonzero(sel))
        idx = msg[8:].view(np.dtype([("i", np.int32), ("v", np.float32)]))["i"]
        assert (idx == np.nonzero(sel)[0]).all()
        assert not r[sel].any() and (r[~sel] == g_h[~sel]).all()
        return rests

    # reference-faithful strided sampling (1000 samples), exact top-k, and host-supplied positions
    run("strided", lambda r: dev.topk_threshold(r, g, topk, 1000, 10.0))
    run("exact", lambda r: dev.topk_threshold(r, g, topk, W.C4["default_subsamples_exact"], 10.0))
    # the same as one call (single pass over the vectors): same recorded outputs
    thr_out = torch.zeros(1, device="cuda")
    r1 = torch.zeros(n, device="cuda")
    nbytes = dev.compress_topk(buf, g, r1, topk, d_thr=thr_out)
    assert dev.get_option("fused_topk_taken") == 1
    row = GOLD["C4"]["exact"]
    assert _hex(thr_out.item()) == row["thr_hex"] and nbytes == 8 + 8 * row["k"]
    assert W.checksum(buf[:nbytes].cpu().numpy()) == row["msg"]
    assert W.checksum(r1.cpu().numpy()) == row["rests"]
    del r1
    idx_h = W.c4_sample_indices()
    assert W.checksum(idx_h) == GOLD["C4"]["indexed"]["idx"]
    idx = torch.from_numpy(idx_h).cuda()
    rests = run("indexed", lambda r: dev.topk_threshold_indexed(r, g, idx, topk))
    # exact mode sends ceil_f32(n*topK)-1 pairs when no magnitude ties with the threshold
    assert GOLD["C4"]["exact"]["k"] == 999_999

    # conservation over error-feedback steps at full size: sum of decompressed messages + flush
    # == steps * gradient, exact because every value here is a small multiple of 2^-10
    q_h = np.round(g_h * 64).astype(np.float32) / np.float32(64)
    q = torch.from_numpy(q_h).cuda()
    rests.zero_()
    total = torch.zeros(n, device="cuda")
    for step in range(3):
        dev.topk_threshold_indexed(rests, q, idx, topk, to_host=False)
        dev.compress(buf, q, rests, sync=False)
        dev.add(total, buf, check_header=False)
    dev.compress(buf, rests, None, thr=0.0, sync=False)  # flushRests: data-only at threshold 0
    dev.add(total, buf, check_header=False)
    dev.synchronize()
    assert torch.equal(total, q * 3)


def test_c5_sparse_reduce_eight_ranks(dev, oracle):
    msgs_h = W.c5_messages()
    assert [W.checksum(m) for m in msgs_h] == GOLD["C5"]["msgs"], "inputs did not regenerate to the recorded bits"
    n = W.C5["n"]
    msgs = [torch.from_numpy(m).cuda() for m in msgs_h]
    dense = torch.full((n,), 3.0, device="cuda")
    dev.reduce(dense, msgs, accumulate=False, mode=0)
    got = dense.cpu().numpy()
    assert W.checksum(got) == GOLD["C5"]["dense"]  # rank-ordered: bit-exact with the reference
    # atomics reorder the 8 contributions of the shared indices: per element at most
    # 2 * gamma_7 * sum|v| apart (7 rounded additions, u = 2^-24), identical where one message contributes
    dev.reduce(dense, msgs, accumulate=False, mode=1)
    got_atomic = dense.cpu().numpy()
    bound = reorder_bound(msgs_h, np.float32, n)
    assert (np.abs(got_atomic.astype(np.float64) - got.astype(np.float64)) <= bound).all()
    assert got_atomic[bound == 0.0].tobytes() == got[bound == 0.0].tobytes()
    # apply the reduced vector to a residual (addRests' loop) and compress it at 1 %
    rests = torch.from_numpy(np.random.default_rng(9).standard_normal(n).astype(np.float32)).cuda()
    want = rests.cpu().numpy() + got
    dev.add_vec(rests, torch.from_numpy(got).cuda())
    assert rests.cpu().numpy().tobytes() == want.tobytes()
    # ... and the chief's broadcast leg as the reference runs it (src/allreduce.tpp:205): writeRemote
    # of the reduced vector into a residual, exact top-k 1 %, against the checker
    topk, ds = np.float32(0.01), 1 << 27
    rests_h = np.random.default_rng(10).standard_normal(n).astype(np.float32)
    rests = torch.from_numpy(rests_h.copy()).cuda()
    want_msg, want_thr = oracle.write_remote(rests_h, got, topk, ds)
    dense = torch.from_numpy(got).cuda()
    buf = torch.zeros(8 + 8 * (n // 50), dtype=torch.uint8, device="cuda")
    thr = dev.topk_threshold(rests, dense, topk, ds)
    nbytes = dev.compress(buf, dense, rests)
    assert thr == want_thr and nbytes == want_msg.size
    assert buf[:nbytes].cpu().numpy().tobytes() == want_msg.tobytes()
    assert rests.cpu().numpy().tobytes() == rests_h.tobytes()
    dev.synchronize()


def test_largest_vector_an_int32_length_allows(dev):
    """n = 2^31 - 1 elements (the reference's sizes are `int`): sampled threshold + fused compress,
    the one-call exact top-k, and decompress, checked on the GPU against the definition
    (k = #{|r+g| > t}, ascending indices = the positions of those elements, values = their sums,
    residual = the sums with the sent ones cleared), chunk by chunk."""
    n = 2**31 - 1
    gen = torch.Generator(device="cuda").manual_seed(7)
    g = torch.empty(n, device="cuda").normal_(generator=gen)
    r0 = torch.empty(n, device="cuda").normal_(std=0.25, generator=gen)
    idx = torch.randint(0, n, (100_000,), device="cuda", dtype=torch.int32, generator=gen)
    buf = torch.zeros(8 + 8 * (n // 50), dtype=torch.uint8, device="cuda")  # room for 2 %
    chunks = [(a, min(a + (1 << 29), n)) for a in range(0, n, 1 << 29)]

    def check(rests, thr, nbytes):
        k = int(buf[4:8].view(torch.int32).item())
        assert int(buf[0:4].view(torch.int32).item()) == n and nbytes == 8 + 8 * k
        pairs = buf[8:nbytes].view(torch.int32).view(-1, 2)
        got_idx, got_val = pairs[:, 0].long(), pairs[:, 1].contiguous().view(torch.float32)
        at = 0
        for a, b in chunks:
            s = r0[a:b] + g[a:b]
            sel = s.abs() > thr
            pos = sel.nonzero().flatten()
            c = pos.numel()
            assert torch.equal(got_idx[at:at + c], pos + a)
            assert torch.equal(got_val[at:at + c], s[pos])
            assert torch.equal(rests[a:b], torch.where(sel, torch.zeros_like(s), s))
            at += c
            del s, sel, pos
        assert at == k
        return k

    say("largest vector: sampled threshold + compress")
    rests = r0.clone()
    thr = dev.topk_threshold_indexed(rests, g, idx, np.float32(0.01))
    nbytes = dev.compress(buf, g, rests)
    k = check(rests, thr, nbytes)
    assert abs(k / n - 0.01) < 0.002

    say("largest vector: decompress")
    dense = torch.empty(n, device="cuda")
    assert dev.decompress(dense, buf) == nbytes
    for a, b in chunks:
        s = r0[a:b] + g[a:b]
        assert torch.equal(dense[a:b], torch.where(s.abs() > thr, s, torch.zeros_like(s)))
        del s
    del dense

    say("largest vector: threshold and compress as one call")
    rests.copy_(r0)
    thr_out = torch.zeros(1, device="cuda")
    nbytes = dev.compress_topk(buf, g, rests, np.float32(0.01), d_thr=thr_out)
    assert dev.get_option("fused_topk_taken") == 1
    k = check(rests, float(thr_out.item()), nbytes)
    # whole-vector top-k: the (pos+1)-th largest magnitude is the threshold, pos = ceil_f32(n*topK) - 1
    pos = int(np.ceil(np.float32(n) * np.float32(0.01)) - np.float32(1.0))
    assert pos - 8 <= k <= pos  # ties with the threshold stay behind


def test_largest_vector_receive_side_and_rank_ordered_reduce(dev):
    """n = 2^31 - 1, the largest `int size` of the reference's interface (8.6 GB per fp32 vector):
    every index, tile number and byte offset near 2^31 has to be computed in 64 bits somewhere.
    Checked on the GPU with torch as the independent side: pair count, ascending indices including
    the very last element, values, residual, then decompress / add / two-message reduce of the
    message over the same length, and the sampled threshold at positions up to the last one."""
    n = 2**31 - 1
    free, _ = torch.cuda.mem_get_info()
    if free < 80 * 2**30:
        pytest.skip("needs about 80 GB of free device memory")
    say("largest vector: generating", n, "elements")
    gen = torch.Generator(device="cuda").manual_seed(99)
    g = torch.randn(n, device="cuda", generator=gen)
    r = torch.randn(n, device="cuda", generator=gen) * 0.25
    g[-1], r[-1] = 50.0, 0.5          # the last element is sent
    g[0], r[0] = -40.0, 0.25          # and the first
    s = r + g
    thr = np.float32(2.75)            # about 0.76 % of |N(0, 1.03)|
    want_k = int((s.abs() > float(thr)).sum().item())
    assert 10_000_000 < want_k < 30_000_000
    cap = 8 + 8 * (want_k + 1000)
    msg = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    say("largest vector: compress")
    nbytes = dev.compress(msg, g, r, thr=thr)
    assert nbytes == 8 + 8 * want_k
    hdr = msg[:8].view(torch.int32)
    assert int(hdr[0]) == n and int(hdr[1]) == want_k
    pairs = msg[8:nbytes].view(torch.int32).view(-1, 2)
    idx = pairs[:, 0].to(torch.int64)
    val = pairs[:, 1].contiguous().view(torch.float32)
    assert int(idx[0]) == 0 and int(idx[-1]) == n - 1
    assert bool((idx[1:] > idx[:-1]).all())
    assert torch.equal(val, s[idx])
    keep = s.abs() <= float(thr)
    assert torch.equal(r, torch.where(keep, s, torch.zeros((), device="cuda")))
    del keep, g
    say("largest vector: decompress, add, reduce")
    dense = torch.full((n,), 3.0, device="cuda")
    assert dev.decompress(dense, msg) == nbytes
    assert int(torch.count_nonzero(dense).item()) == int(torch.count_nonzero(val).item())
    assert torch.equal(dense[idx], val) and float(dense[-1]) == 50.5
    dev.add(dense, msg)
    assert torch.equal(dense[idx], val + val)
    dev.reduce(dense, [msg, msg, msg], accumulate=False, mode=0)
    dev.synchronize()
    assert torch.equal(dense[idx], (val + val) + val)
    assert int(torch.count_nonzero(dense).item()) == int(torch.count_nonzero(val).item())
    dev.reduce(dense, [msg, msg, msg], accumulate=True, mode=0)
    dev.synchronize()
    assert torch.equal(dense[idx], ((((val + val) + val) + val) + val) + val)
    del dense
    say("largest vector: sampled threshold")
    pos = torch.cat([torch.randint(0, n, (49_998,), device="cuda", generator=gen),
                     torch.tensor([0, n - 1], device="cuda")]).to(torch.int32)
    got = dev.topk_threshold_indexed(r, s, pos, np.float32(0.01))
    sample = (r[pos.to(torch.int64)] + s[pos.to(torch.int64)]).abs()
    want = float(torch.sort(sample, descending=True).values[int(np.ceil(np.float32(50_000) * np.float32(0.01))) - 1])
    assert got == want
