#!/usr/bin/env python3
"""Benchmark of the compression hot path on one MI355X.

A step = one writeRemote of the 100 M-element workload (config C4): the sampled
ThresholdTopK threshold from 100 000 host-supplied sample positions (1 % density), then the
fused accumulate + select + ordered compaction + residual zeroing kernel.  Inputs are
resident in HBM before the timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published


def measured_traffic(workload, n):
    """Bytes per launch of the streaming kernel from the committed counter runs (FETCH_SIZE and
    WRITE_SIZE, scaled by a plain copy of known size); None when they cover another workload."""
    path = os.path.join(ROOT, "profiles", "stage_kernel_C4_100M_traffic.json")
    try:
        rec = json.load(open(path))
    except (OSError, ValueError):
        return None
    return rec["traffic_bytes_per_launch"] if rec.get("workload") == workload and rec.get("n") == n else None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def event_ms(torch, fn, reps, between=None):
    """Mean milliseconds of fn() from HIP events on torch's current stream (the stream the library
    launches on here); `between` runs untimed before every repetition."""
    e0 = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    e1 = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        if between is not None:
            between()
        e0[i].record()
        fn()
        e1[i].record()
    torch.cuda.synchronize()
    return float(np.mean([a.elapsed_time(b) for a, b in zip(e0, e1)]))


def host_description():
    """Core count and CPU model of the box the CPU legs run on."""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"nproc": os.cpu_count(), "cpu_model": model}


def cpu_baseline(g, idx, topk, seconds):
    """The same step on one host core: the compiled reference headers when their library
    travelled with the tree, else the plain-C restatement.  Threshold (prepare) and compress are
    timed separately, as the reference runs them as two calls."""
    from oracle.pyoracle import Oracle, ref_available
    impl = Oracle(ref=True) if ref_available() else Oracle()
    n = g.size
    rests = np.zeros(n, np.float32)
    times, k = [], 0
    t_end = time.perf_counter() + seconds
    it = 0
    while it < 2 or (time.perf_counter() < t_end and it < 200):
        t0 = time.perf_counter()
        sums = rests[idx] + g[idx]                       # prep_add_vec's gather on the chosen positions
        thr = impl.calc_threshold(sums, topk)            # calc_threshold (nth_element)
        t1 = time.perf_counter()
        msg = impl.ip_compress(g, rests, thr)            # compress_add_update
        t2 = time.perf_counter()
        k = int(msg[4:8].view(np.int32)[0])
        if it > 0:  # first pass is the warm-up
            times.append((t2 - t0, 12 * n + 8 * k + 8 + 8 * idx.size, t1 - t0, t2 - t1))
        it += 1
    med = sorted(times)[len(times) // 2]
    out = dict(value=med[1] / med[0] / 1e9, unit="GB/s", cores=1, kind=impl.kind,
               sample="%d full steps (n=%d, %d sample positions) after 1 warm-up, median; %.1f ms/step"
                      % (len(times), n, idx.size, med[0] * 1e3),
               ms_per_step=med[0] * 1e3, prepare_ms=float(np.median([t[2] for t in times])) * 1e3,
               compress_ms=float(np.median([t[3] for t in times])) * 1e3)
    out.update(host_description())
    return out


def cpu_reduce_baseline(msgs_h, n, seconds):
    """Config C5 on one host core: zero the dense vector, add the messages in rank order
    (add_strategy), then residual += dense (the accumulate half of the broadcast-leg writeRemote)."""
    from oracle.pyoracle import Oracle, ref_available
    impl = Oracle(ref=True) if ref_available() else Oracle()
    plain = Oracle()
    dense = np.zeros(n, np.float32)
    rests = np.zeros(n, np.float32)
    red, app = [], []
    t_end = time.perf_counter() + seconds
    it = 0
    while it < 2 or (time.perf_counter() < t_end and it < 50):
        t0 = time.perf_counter()
        dense[:] = 0
        for m in msgs_h:
            impl.ip_add(m, dense)
        t1 = time.perf_counter()
        plain.add_rests(rests, dense)
        t2 = time.perf_counter()
        if it > 0:
            red.append(t1 - t0)
            app.append(t2 - t1)
        it += 1
    return float(np.median(red)) * 1e3, float(np.median(app)) * 1e3, impl.kind, len(red)


def golden_rows(name):
    """Recorded outputs of the compiled reference for a configuration (tests/golden/full_size.json,
    written by tests/golden/make_golden.py), or [] when the file is not there."""
    try:
        return json.load(open(os.path.join(ROOT, "tests", "golden", "full_size.json"))).get(name, [])
    except (OSError, ValueError):
        return []


def config_leg(torch, W, cfg, grad_fn, cpu_seconds, with_cpu, cpu_iters_cap):
    """One of the smaller configurations (C1, C2, C3): exact top-k threshold + fused compress per
    iteration, residual carried, as ONE call per iteration (cx_ip_write_step: what
    ComprEx::writeRemote enqueues).  Timed eagerly (events around every call) and, where the call
    never waits, as a replayed HIP graph of `ring` iterations (short vectors are launch latency:
    the graph removes the host's share of it).  The first iterations are compared bit for bit with
    the compiled reference's recorded outputs."""
    from comprex_amd.device import Handle, message_capacity
    n, topk, ds = cfg["n"], np.float32(cfg["topK"]), cfg["default_subsamples"]
    ring = 4
    grads_h = [grad_fn(it) for it in range(ring)]
    side = torch.cuda.Stream()
    out = {"workload": cfg["name"], "n": n, "topK": float(topk)}
    with torch.cuda.stream(side):
        h = Handle()
        grads = [torch.from_numpy(g).cuda() for g in grads_h]
        rests = torch.zeros(n, device="cuda")
        msg = torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")
        hdr = msg[:8].view(torch.int32)

        # parity: the recorded reference outputs of the first iterations
        rows = golden_rows(cfg["name"].split("-")[0])
        checked = 0
        for it in range(ring):
            nbytes = h.write_step(msg, grads[it], rests, topk, ds)
            if it < len(rows) and rows[it].get("input") == W.checksum(grads_h[it]):
                m_h = msg[:nbytes].cpu().numpy()
                assert int(hdr[1].item()) == rows[it]["k"] and W.checksum(m_h) == rows[it]["msg"], \
                    "%s iteration %d differs from the reference's recorded message" % (cfg["name"], it)
                assert W.checksum(rests.cpu().numpy()) == rows[it]["rests"]
                checked += 1
        out["iterations_checked_against_reference"] = checked
        fused_route = h.get_option("fused_topk_taken")  # 1: single pass over the vectors (waits once per call)

        def step(it):
            h.write_step(msg, grads[it % ring], rests, topk, ds, sync=False)

        reps = 10 * ring
        for it in range(2 * ring):
            step(it)
        side.synchronize()
        e0 = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
        e1 = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
        ks = []
        for it in range(reps):
            e0[it].record(side)
            step(it)
            e1[it].record(side)
        side.synchronize()
        eager_us = float(np.median([a.elapsed_time(b) for a, b in zip(e0, e1)])) * 1e3
        k = int(hdr[1].item())
        step_bytes = 20 * n + 8 * k + 8
        out.update(k_last=k, algorithmic_bytes=step_bytes, eager_us=eager_us,
                   eager_GBps=step_bytes / (eager_us * 1e-6) / 1e9,
                   eager_frac=step_bytes / (eager_us * 1e-6) / 1e9 / HBM_PEAK_GBPS)
        if fused_route == 0:
            # the call only enqueues: capture `ring` iterations, replay them back to back
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for it in range(ring):
                    step(it)
            side.synchronize()
            for _ in range(3):
                graph.replay()
            side.synchronize()
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            replays = 20
            g0.record(side)
            for _ in range(replays):
                graph.replay()
            g1.record(side)
            side.synchronize()
            graph_us = g0.elapsed_time(g1) * 1e3 / (replays * ring)
            out.update(graph_us=graph_us, graph_GBps=step_bytes / (graph_us * 1e-6) / 1e9,
                       graph_frac=step_bytes / (graph_us * 1e-6) / 1e9 / HBM_PEAK_GBPS)
            del graph
        else:
            out["graph_us"] = None  # the single-pass route reads one word back per call: not capturable
        h.synchronize()
        h.close()
    log("%s: step %.1f us eager%s (%.0f GB/s of 20n+8k+8, %.1f%% of peak), k=%d, %d iterations checked"
        % (cfg["name"], eager_us, "" if out.get("graph_us") is None else ", %.1f us as a replayed graph" % out["graph_us"],
           out["eager_GBps"], 100 * out["eager_frac"], k, checked))
    if with_cpu:
        from oracle.pyoracle import Oracle, ref_available
        impl = Oracle(ref=True) if ref_available() else Oracle()
        rests_h = np.zeros(n, np.float32)
        times = []
        t_end = time.perf_counter() + cpu_seconds
        it = 0
        while it < 2 or (time.perf_counter() < t_end and it < cpu_iters_cap):
            g = grads_h[it % ring]
            t0 = time.perf_counter()
            thr = impl.calc_threshold(rests_h + g, topk)   # prep_add_vec (whole vector) + nth_element
            impl.ip_compress(g, rests_h, thr)               # compress_add_update
            if it > 0:
                times.append(time.perf_counter() - t0)
            it += 1
        med = float(np.median(times))
        out["cpu_baseline"] = {"cores": 1, "kind": impl.kind, "us": med * 1e6, "GBps": step_bytes / med / 1e9,
                               "sample": "%d iterations after 1 warm-up, median" % len(times)}
        log("%s cpu baseline (%s, 1 core): %.0f us/iteration" % (cfg["name"], impl.kind, med * 1e6))
    return out


def api_leg(torch, n, reps=200):
    """writeRemote / readRemote_add through the reference's own C symbols (Comprex_*; comprex_amd/pygpi.py binds
    them as the reference's ComprEx.py does) on device vectors, with the reference's default threshold: a
    ThresholdTopK of 1 % over 1000 strided samples.  Host time per call, the device kept busy back to back."""
    from comprex_amd import pygpi as P
    env = P.GaspiEnvironment(1 << 20)
    thr, comp = P.ThresholdTopK(0.01), P.CompressorIndexPairs()
    cs = []
    for rank in range(2):
        env.set_rank(rank, 2)
        c = P.Comprex(env, n, 0.2)
        c.setThreshold(thr)
        c.setCompressor(comp)
        c.connectTo((rank + 1) % 2, (rank + 1) % 2, 5)
        cs.append(c)
    g = torch.randn(n, device="cuda")
    out = torch.zeros(n, device="cuda")
    env.set_user_stream(torch.cuda.current_stream())

    def pair():
        cs[0].writeRemote(g)
        cs[1].readRemote_add(out)

    for _ in range(10):
        pair()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        pair()
    torch.cuda.synchronize()
    pair_us = (time.perf_counter() - t0) / reps * 1e6
    tw = tr = 0.0
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cs[0].writeRemote(g)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        cs[1].readRemote_add(out)
        torch.cuda.synchronize()
        tw += t1 - t0
        tr += time.perf_counter() - t1
    del cs, env
    return {"n": n, "threshold": "ThresholdTopK(0.01): 1000 strided samples", "pair_us": pair_us,
            "writeRemote_alone_us": tw / reps * 1e6, "readRemote_add_alone_us": tr / reps * 1e6,
            "what": "pair = writeRemote + readRemote_add back to back; alone = one call and a device wait after it"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--n", type=int, default=None, help="override the vector length (debugging)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the exact-top-k and reduce legs")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--items", type=int, default=None, help="compaction tile option (2/4/8)")
    ap.add_argument("--alternate", type=int, default=None, help="stage_alternate option (0/1)")
    ap.add_argument("--cached-tail-mb", type=int, default=None, help="stage_cached_tail_mb option (-1 = all cacheable)")
    ap.add_argument("--configs-only", action="store_true",
                    help="run only the legs of the smaller configurations C1, C2, C3 (for a kernel trace of them)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device copy of the gradient (4n bytes read, 4n written) so that "
                         "a counter run has a kernel of known traffic to scale FETCH_SIZE/WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU; the path has no inter-GPU part (--gpus %d refused)" % args.gpus)
        sys.exit(2)

    import torch
    from comprex_amd import workloads as W
    from comprex_amd.device import Handle, message_capacity

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.configs_only:
        legs = {}
        for key, cfg, fn, cap in (("C1", W.C1, W.c1_gradient, 100), ("C2", W.C2, W.c2_gradient, 200),
                                  ("C3", W.C3, W.c3_gradient, 3)):
            legs[key] = config_leg(torch, W, cfg, fn, min(args.cpu_seconds, 5.0), not args.no_cpu, cap)
        print(json.dumps({"configs": legs}), flush=True)
        return
    n = args.n or W.C4["n"]
    topk = np.float32(W.C4["topK"])
    m = W.C4["n_samples"] if n >= W.C4["n_samples"] * 10 else max(1000, n // 100)

    t0 = time.time()
    g_h = W.c4_gradient(n=n)
    idx_h = W.c4_sample_indices(n=n, m=m)
    log("generated %s: n=%d in %.1fs (input checksum %s)" % (W.C4["name"], n, time.time() - t0, W.checksum(g_h)))

    h = Handle()
    if args.items is not None:
        h.set_option("compact_items", args.items)
    if args.alternate is not None:
        h.set_option("stage_alternate", args.alternate)
    if args.cached_tail_mb is not None:
        h.set_option("stage_cached_tail_mb", args.cached_tail_mb)
    g = torch.from_numpy(g_h).cuda()
    idx = torch.from_numpy(idx_h).cuda()
    rests = torch.zeros(n, device="cuda")
    msg = torch.zeros(message_capacity(n, torch.float32), dtype=torch.uint8, device="cuda")
    hdr = msg[:8].view(torch.int32)

    def step():
        h.topk_threshold_indexed(rests, g, idx, topk, to_host=False)  # threshold stays on the device
        h.compress(msg, g, rests, sync=False)                         # reads it from the handle's slot

    for _ in range(args.warmup):
        step()
    h.synchronize()
    if args.calibrate_copy:
        scratch = torch.empty_like(g)
        scratch.copy_(g)
        torch.cuda.synchronize()
        del scratch
    # the library records a HIP event before and after its streaming kernel, on the stream it
    # launches on, for every fifth step of the timed region
    every = 5  # the two events cost the step a few microseconds: one launch in five carries them
    h.set_option("profile_stage", every)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stage_ms = h.profile_read()
    h.set_option("profile_stage", 0)
    h.synchronize()  # raises if any launch recorded a device-side error
    k = int(hdr[1].item())
    assert int(hdr[0].item()) == n and len(stage_ms) == min((args.steps + every - 1) // every, 1024)
    ms_per_step = elapsed / args.steps * 1e3
    step_bytes = 12 * n + 8 * k + 8 + 8 * m
    kern_ms = float(np.mean(stage_ms))
    kern_bytes = 12 * n + 8 * k + 8
    achieved = kern_bytes / (kern_ms * 1e-3) / 1e9
    log("step %.3f ms, streaming kernel %.3f ms (%.0f GB/s, %.1f%% of peak), k=%d (%.3f%%)"
        % (ms_per_step, kern_ms, achieved, 100 * achieved / HBM_PEAK_GBPS, k, 100.0 * k / n))

    extra = {"k_last_step": k, "density": k / n, "elements_per_s": n / (ms_per_step * 1e-3),
             "stage_kernel_ms": kern_ms, "rest_of_step_ms": ms_per_step - kern_ms,
             "hbm_peak_fraction_step": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
             "cache_state": "warm: consecutive steps, the residual's tail is still in the 256 MB memory-side cache"}

    # the same step with a COLD residual: between two steps another kernel streams through 1 GiB
    # (a training step's backward pass runs there), which evicts the 256 MB memory-side cache; the
    # eviction itself is outside the events.  Two kinds: a kernel that only READS (the cache is left
    # full of clean lines) and one that WRITES (left full of dirty lines, whose write-back then
    # competes with the step).
    evict = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)
    cold_reps = max(5, min(args.steps, 20))
    for key, what, fn in (("cold", "1 GiB read by another kernel between steps (memory-side cache evicted, clean)",
                           lambda: evict.sum()),
                          ("cold_after_writes", "1 GiB rewritten by another kernel between steps (cache evicted, dirty)",
                           lambda: evict.add_(1.0)),
                          ("gradient_rewritten", "the gradient itself rewritten in place by another kernel between steps "
                           "(what a backward pass leaves: its tail in the cache, dirty)", lambda: g.mul_(1.0))):
        # two passes: the step is timed without the library's events around its streaming kernel
        # (each event costs the step some 3 us between two kernels), the kernel in a pass of its own
        cold_step_ms = event_ms(torch, step, cold_reps, between=fn)
        h.set_option("profile_stage", 1)
        event_ms(torch, step, cold_reps, between=fn)
        cold_stage = h.profile_read()
        h.set_option("profile_stage", 0)
        cold_kern_ms = float(np.mean(cold_stage))
        extra[key] = {"what": what, "steps": cold_reps, "step_ms": cold_step_ms, "stage_kernel_ms": cold_kern_ms,
                      "stage_kernel_GBps": kern_bytes / (cold_kern_ms * 1e-3) / 1e9,
                      "stage_kernel_frac": kern_bytes / (cold_kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                      "step_GBps": step_bytes / (cold_step_ms * 1e-3) / 1e9,
                      "hbm_peak_fraction_step": step_bytes / (cold_step_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        log("%s: step %.3f ms (%.1f%% of peak), streaming kernel %.3f ms (%.1f%% of peak)"
            % (key, cold_step_ms, 100 * extra[key]["hbm_peak_fraction_step"], cold_kern_ms,
               100 * extra[key]["stage_kernel_frac"]))
    del evict

    if not args.no_extra:
        # what plain streaming reaches on this GPU, for scale: a device copy (8n bytes) and an
        # in-place add (12n bytes, the streaming kernel's own access pattern) through torch
        probe = torch.empty_like(g)
        for name, fn, nbytes in (("device_copy", lambda: probe.copy_(g), 8 * n),
                                 ("inplace_add", lambda: probe.add_(g), 12 * n)):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            extra[name + "_GBps"] = nbytes / ((time.perf_counter() - t0) / 20) / 1e9
        del probe
        log("plain streaming on this GPU: copy %.0f GB/s, in-place add %.0f GB/s"
            % (extra["device_copy_GBps"], extra["inplace_add_GBps"]))

        # The same step with the vector cut into S contiguous segments, each with a handle and a stream
        # of its own (what Comprex_RingAllreduce's per-segment ComprEx objects amount to on one GPU,
        # src/allreduce.tpp:372-416): the segments' latency-bound small kernels run beside the other
        # segments' streaming kernels.  The cached tail of the residual is shared out among the segments.
        seg_out = {}
        for S in (2, 4):
            seg = (n // S) & ~3
            streams = [torch.cuda.Stream() for _ in range(S)]
            hs, seg_msgs, seg_idx = [], [], []
            for q in range(S):
                with torch.cuda.stream(streams[q]):
                    hs.append(Handle())
                hs[q].set_option("stage_cached_tail_mb", 192 // S)
                seg_msgs.append(torch.zeros(message_capacity(seg, torch.float32) // 8, dtype=torch.uint8, device="cuda"))
                pos = idx_h[(idx_h >= q * seg) & (idx_h < (q + 1) * seg)] - q * seg
                seg_idx.append(torch.from_numpy(pos.astype(np.int32)).cuda())

            def seg_steps():
                for q in range(S):
                    with torch.cuda.stream(streams[q]):
                        gq, rq = g[q * seg:(q + 1) * seg], rests[q * seg:(q + 1) * seg]
                        hs[q].topk_threshold_indexed(rq, gq, seg_idx[q], topk, to_host=False)
                        hs[q].compress(seg_msgs[q], gq, rq, sync=False)

            torch.cuda.synchronize()
            for _ in range(5):
                seg_steps()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(30):
                seg_steps()
            torch.cuda.synchronize()
            seg_ms = (time.perf_counter() - t0) / 30 * 1e3
            ks = sum(int(mq[4:8].view(torch.int32).item()) for mq in seg_msgs)
            seg_bytes = 12 * S * seg + 8 * ks + 8 * S + 8 * sum(int(t.numel()) for t in seg_idx)
            seg_out[str(S)] = {"ms": seg_ms, "GBps": seg_bytes / (seg_ms * 1e-3) / 1e9,
                               "frac": seg_bytes / (seg_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "k": ks,
                               "cached_tail_mb_each": 192 // S}
            for hq in hs:
                hq.synchronize()
                hq.close()
            del seg_msgs, seg_idx
        extra["segments_on_own_streams"] = seg_out
        log("the step as 2 / 4 segments on streams of their own: %.3f / %.3f ms (one stream: %.3f ms)"
            % (seg_out["2"]["ms"], seg_out["4"]["ms"], ms_per_step))

        # exact top-k (radix select over all n) + compress, same vector
        rests.zero_()
        ds = W.C4["default_subsamples_exact"] if n == W.C4["n"] else 1 << 30
        for _ in range(2):
            h.topk_threshold(rests, g, topk, ds, to_host=False)
            h.compress(msg, g, rests, sync=False)
        torch.cuda.synchronize()
        reps = 10
        t0 = time.perf_counter()
        for _ in range(reps):
            h.topk_threshold(rests, g, topk, ds, to_host=False)
            h.compress(msg, g, rests, sync=False)
        torch.cuda.synchronize()
        ex_ms = (time.perf_counter() - t0) / reps * 1e3
        kx = int(hdr[1].item())
        extra["exact_topk_step_ms"] = ex_ms
        extra["exact_topk_GBps"] = (20 * n + 8 * kx + 8) / (ex_ms * 1e-3) / 1e9
        extra["exact_topk_k"] = kx
        log("exact top-k step %.3f ms (%.0f GB/s of 20n+8k+8), k=%d" % (ex_ms, extra["exact_topk_GBps"], kx))
        # the exact threshold alone (one read of both vectors: 8n bytes), on the residual those steps left
        for _ in range(2):
            h.topk_threshold(rests, g, topk, ds, to_host=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            h.topk_threshold(rests, g, topk, ds, to_host=False)
        torch.cuda.synchronize()
        et_ms = (time.perf_counter() - t0) / reps * 1e3
        extra["exact_threshold_ms"] = et_ms
        extra["exact_threshold_GBps"] = 8 * n / (et_ms * 1e-3) / 1e9
        log("exact threshold alone %.3f ms (%.0f GB/s of 8n, %.1f%% of peak)"
            % (et_ms, extra["exact_threshold_GBps"], 100 * extra["exact_threshold_GBps"] / HBM_PEAK_GBPS))
        # the same as one call: exact threshold and compress in a single pass over the vectors
        rests.zero_()
        for _ in range(2):
            h.compress_topk(msg, g, rests, topk)
        t0 = time.perf_counter()
        routes = []
        for _ in range(reps):
            h.compress_topk(msg, g, rests, topk)  # waits for the stream itself
            routes.append(h.get_option("fused_topk_taken"))
        fx_ms = (time.perf_counter() - t0) / reps * 1e3
        kf = int(hdr[1].item())
        extra["exact_topk_fused_step_ms"] = fx_ms
        extra["exact_topk_fused_GBps"] = (20 * n + 8 * kf + 8) / (fx_ms * 1e-3) / 1e9
        extra["exact_topk_fused_k"] = kf
        extra["exact_topk_fused_routes"] = sorted(set(routes))
        log("exact top-k, single pass: %.3f ms (%.0f GB/s of 20n+8k+8), k=%d, routes %s"
            % (fx_ms, extra["exact_topk_fused_GBps"], kf, extra["exact_topk_fused_routes"]))
        del g, rests, msg
        torch.cuda.empty_cache()

        if n == W.C4["n"]:
            # the other compress configurations, each as its own leg
            extra["configs"] = {}
            for key, cfg, fn, cap in (("C1", W.C1, W.c1_gradient, 100), ("C2", W.C2, W.c2_gradient, 200),
                                      ("C3", W.C3, W.c3_gradient, 3)):
                extra["configs"][key] = config_leg(torch, W, cfg, fn, min(args.cpu_seconds, 5.0), not args.no_cpu, cap)
            extra["configs"]["launches_per_step"] = {
                "C1": 5, "C2": 5, "C3": 9,
                "source": "rocprofv3 kernel trace of these legs, profiles/configs_C1_C2_C3_kernel_trace.txt, not this run"}
            # the reference's calls with its default threshold, through its C symbols
            extra["reference_api_calls"] = [api_leg(torch, W.C2["n"]), api_leg(torch, W.C1["n"])]
            for leg in extra["reference_api_calls"]:
                log("Comprex_writeRemote + Comprex_readRemote_add, n=%d, default threshold: %.1f us per pair (alone: %.1f + %.1f us)"
                    % (leg["n"], leg["pair_us"], leg["writeRemote_alone_us"], leg["readRemote_add_alone_us"]))

        # reduce: 8 simulated ranks' 1 %-dense messages into a 64 Mi dense vector (config C5)
        c5n = W.C5["n"] if n == W.C4["n"] else 1 << 22
        c5k = W.C5["k"] if n == W.C4["n"] else c5n // 100
        t0 = time.time()
        msgs_h = W.c5_messages(n=c5n, k=c5k, shared=c5k // 2)
        log("generated %s in %.1fs" % (W.C5["name"], time.time() - t0))
        msgs = [torch.from_numpy(mm).cuda() for mm in msgs_h]
        dense = torch.empty(c5n, device="cuda")
        red_bytes = 4 * c5n + 16 * len(msgs) * c5k
        reduce = {"workload": W.C5["name"], "n": c5n, "ranks": len(msgs), "k_per_rank": c5k,
                  "algorithmic_bytes": red_bytes, "peak": HBM_PEAK_GBPS, "unit": "GB/s"}
        for mode, name in ((0, "ordered"), (1, "atomic")):
            for _ in range(2):
                h.reduce(dense, msgs, accumulate=False, mode=mode)
            r_ms = event_ms(torch, lambda: h.reduce(dense, msgs, accumulate=False, mode=mode), reps)
            reduce[name + "_ms"] = r_ms
            reduce[name + "_GBps"] = red_bytes / (r_ms * 1e-3) / 1e9
            reduce[name + "_frac"] = reduce[name + "_GBps"] / HBM_PEAK_GBPS
            extra["reduce_" + name + "_ms"] = r_ms
            extra["reduce_" + name + "_GBps"] = reduce[name + "_GBps"]
            log("reduce %s %.3f ms (%.0f GB/s of 4n+16Rk, %.1f%% of peak)"
                % (name, r_ms, reduce[name + "_GBps"], 100 * reduce[name + "_frac"]))
        reduce["pairs_per_s"] = len(msgs) * c5k / (reduce["ordered_ms"] * 1e-3)
        # the chief's own form of the loop: the messages are added INTO its vector (readRemote_add per
        # worker), so every element is read and written: 8n + 16Rk bytes
        acc_bytes = 8 * c5n + 16 * len(msgs) * c5k
        for _ in range(2):
            h.reduce(dense, msgs, accumulate=True, mode=0)
        acc_ms = event_ms(torch, lambda: h.reduce(dense, msgs, accumulate=True, mode=0), reps)
        reduce["accumulate"] = {"algorithmic_bytes": acc_bytes, "ms": acc_ms, "GBps": acc_bytes / (acc_ms * 1e-3) / 1e9,
                                "frac": acc_bytes / (acc_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        log("reduce ordered, added into the vector %.3f ms (%.0f GB/s of 8n+16Rk, %.1f%% of peak)"
            % (acc_ms, reduce["accumulate"]["GBps"], 100 * reduce["accumulate"]["frac"]))
        # the same shape in fp64: half as many elements (the same 256 MB vector), 1 %-dense messages of
        # 12-byte pairs; per pair 12 B of message + 8 B read + 8 B write, the vector read and written
        n64, k64 = c5n // 2, c5k // 2
        msgs64 = [torch.from_numpy(mm).cuda() for mm in W.c5_messages(n=n64, k=k64, shared=k64 // 2, dtype=np.float64)]
        dense64 = torch.zeros(n64, dtype=torch.float64, device="cuda")
        f64 = {}
        for acc, key, nbytes in ((False, "from_zeros", 8 * n64 + 28 * len(msgs64) * k64),
                                 (True, "accumulate", 16 * n64 + 28 * len(msgs64) * k64)):
            for _ in range(2):
                h.reduce(dense64, msgs64, accumulate=acc, mode=0)
            ms64 = event_ms(torch, lambda: h.reduce(dense64, msgs64, accumulate=acc, mode=0), reps)
            f64[key] = {"algorithmic_bytes": nbytes, "ms": ms64, "GBps": nbytes / (ms64 * 1e-3) / 1e9,
                        "frac": nbytes / (ms64 * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        reduce["f64"] = dict(f64, n=n64, k_per_rank=k64)
        log("reduce ordered, fp64 (%d elements): from zeros %.3f ms (%.1f%% of peak of 8n+28Rk), added into the vector "
            "%.3f ms (%.1f%% of peak of 16n+28Rk)" % (n64, f64["from_zeros"]["ms"], 100 * f64["from_zeros"]["frac"],
                                                       f64["accumulate"]["ms"], 100 * f64["accumulate"]["frac"]))
        del msgs64, dense64
        # The chief's apply as the reference runs it (src/allreduce.tpp:183-205): readRemote_add per
        # worker into its own vector (here ONE rank-ordered accumulate), then the broadcast leg's
        # writeRemote(data): residual += reduced vector, exact top-k 1 %, compact, zero
        c5_brests = torch.zeros(c5n, device="cuda")
        bmsg = torch.zeros(8 + 8 * (c5n // 25), dtype=torch.uint8, device="cuda")
        ds_exact = 1 << 27 if c5n >= 1 << 23 else 1 << 30

        def chief_apply():
            h.reduce(dense, msgs, accumulate=True, mode=0)
            h.write_step(bmsg, dense, c5_brests, np.float32(0.01), ds_exact)  # (the single pass waits once)

        for _ in range(2):
            chief_apply()
        ca_ms = event_ms(torch, chief_apply, reps)
        kb = int(bmsg[4:8].view(torch.int32).item())
        ca_bytes = acc_bytes + 12 * c5n + 8 * kb + 8
        for _ in range(2):
            h.write_step(bmsg, dense, c5_brests, np.float32(0.01), ds_exact)
        bw_ms = event_ms(torch, lambda: h.write_step(bmsg, dense, c5_brests, np.float32(0.01), ds_exact), reps)
        reduce["chief_apply"] = {"what": "accumulating rank-ordered reduce into the chief's vector, then writeRemote of it "
                                         "(exact top-k 1 %) on the broadcast channel",
                                 "algorithmic_bytes": ca_bytes, "ms": ca_ms, "GBps": ca_bytes / (ca_ms * 1e-3) / 1e9,
                                 "frac": ca_bytes / (ca_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                 "broadcast_leg_alone_ms": bw_ms, "reduce_alone_ms": acc_ms, "k_broadcast": kb}
        log("chief's apply (accumulate + broadcast-leg writeRemote): %.3f ms (%.0f GB/s of 8n+16Rk+12n+8k, %.1f%% of peak); "
            "parts alone %.3f + %.3f ms" % (ca_ms, reduce["chief_apply"]["GBps"], 100 * reduce["chief_apply"]["frac"],
                                            acc_ms, bw_ms))
        del c5_brests, bmsg
        # residual apply (K4): rests += dense, 12 bytes per element
        c5_rests = torch.zeros(c5n, device="cuda")
        for _ in range(2):
            h.add_vec(c5_rests, dense)
        a_ms = event_ms(torch, lambda: h.add_vec(c5_rests, dense), reps)
        apply_bytes = 12 * c5n
        reduce["apply"] = {"algorithmic_bytes": apply_bytes, "ms": a_ms, "GBps": apply_bytes / (a_ms * 1e-3) / 1e9,
                           "frac": apply_bytes / (a_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                           "elements_per_s": c5n / (a_ms * 1e-3)}
        log("residual apply %.3f ms (%.0f GB/s of 12n, %.1f%% of peak)"
            % (a_ms, reduce["apply"]["GBps"], 100 * reduce["apply"]["frac"]))
        h.synchronize()
        if not args.no_cpu:
            c_red, c_app, kind, cnt = cpu_reduce_baseline(msgs_h, c5n, min(args.cpu_seconds, 8.0))
            reduce["cpu_baseline"] = {"cores": 1, "kind": kind, "sample": "%d full passes, median" % cnt,
                                      "reduce_ms": c_red, "reduce_GBps": red_bytes / (c_red * 1e-3) / 1e9,
                                      "apply_ms": c_app, "apply_GBps": apply_bytes / (c_app * 1e-3) / 1e9}
            log("cpu baseline, reduce (%s, 1 core): %.1f ms (%.2f GB/s), apply %.1f ms (%.2f GB/s)"
                % (kind, c_red, reduce["cpu_baseline"]["reduce_GBps"], c_app, reduce["cpu_baseline"]["apply_GBps"]))
        extra["reduce"] = reduce

    cpu = None
    if not args.no_cpu:
        t0 = time.time()
        cpu = cpu_baseline(g_h, idx_h, topk, args.cpu_seconds)
        log("cpu baseline (%s, 1 core): %.2f GB/s, %.1f ms/step (%.1fs)"
            % (cpu["kind"], cpu["value"], cpu["ms_per_step"], time.time() - t0))

    out = {
        "metric": "compress GB/s (algorithmic bytes 12n+8k+8+8m per writeRemote step: sampled top-k threshold + "
                  "fused accumulate/select/compact/zero), 100M fp32, 1% top-k",
        "value": step_bytes / (ms_per_step * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": W.C4["name"], "n": n, "topK": float(topk), "sample_positions": m,
                   "threshold": "sampled ThresholdTopK over host-supplied positions", "input_checksum": W.checksum(g_h)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": measured_traffic(W.C4["name"], n),
                     "traffic_source": "committed counter run profiles/stage_kernel_C4_100M_pmc.txt, not this run",
                     "kernel": "stage_kernel<float,0,4,%d>" % (args.items or 4), "algorithmic_bytes": kern_bytes,
                     "avg_ms": kern_ms, "cache_state": "warm (see extra.cold for the cold-residual figures)"},
        "roofline_realistic": {"bound": "hbm", "achieved": extra["gradient_rewritten"]["stage_kernel_GBps"],
                               "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": extra["gradient_rewritten"]["stage_kernel_frac"],
                               "kernel": "stage_kernel<float,0,4,%d>" % (args.items or 4), "algorithmic_bytes": kern_bytes,
                               "avg_ms": extra["gradient_rewritten"]["stage_kernel_ms"],
                               "step_frac": extra["gradient_rewritten"]["hbm_peak_fraction_step"],
                               "cache_state": "the gradient is rewritten in place by another kernel between two steps, as a "
                                              "backward pass leaves it: the memory-side cache holds its dirty tail, not the "
                                              "residual's"},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
