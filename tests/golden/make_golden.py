"""Writes the committed fixtures of this folder from the COMPILED REFERENCE HEADERS.

Run where the reference tree is present:  python tests/golden/make_golden.py [--full]

It drives oracle/_ref/libref.so (src/threshold.hxx + src/compressor.hxx of the
reference, compiled unmodified behind oracle/ref_shim.cpp) on seeded inputs and
stores inputs + the reference's outputs:

  small_cases.npz   arrays for small shapes, all three element types and the three
                    compression modes, several error-feedback iterations
  full_size.json    (--full) checksums of the reference's outputs at the benchmark
                    shapes C1..C5, with a checksum of the inputs so a consumer only
                    compares when it regenerated the same bits

Fixtures are data only: inputs and expected outputs.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from comprex_amd import workloads as W  # noqa: E402
from oracle.pyoracle import Oracle  # noqa: E402


def small_cases(ref):
    out = {}
    rng = np.random.Generator(np.random.PCG64(20240607))
    case = 0
    for dtype, tag in [(np.float32, "f32"), (np.float64, "f64"), (np.int32, "i32")]:
        for n, topk, ds in [(257, 0.1, 1000), (4099, 0.01, 1000), (4099, 0.05, 1 << 13),
                            (9973, 0.001, 1000), (9973, 0.01, 1 << 14)]:
            iters = 3
            if dtype == np.int32:
                grads = rng.integers(-500, 501, (iters, n)).astype(np.int32)
            else:
                grads = (rng.standard_normal((iters, n)) * rng.uniform(0.01, 10)).astype(dtype)
            rests = np.zeros(n, dtype)
            key = "ef_%s_%d" % (tag, case)
            out[key + "_grads"] = grads
            out[key + "_params"] = np.array([n, ds], dtype=np.int64)
            out[key + "_topk"] = np.array([topk], dtype=np.float32)
            thrs = []
            for it in range(iters):
                thr = ref.topk_prepare_with(rests, grads[it], np.float32(topk), ds, 10.0)
                msg = ref.ip_compress(grads[it].copy(), rests, thr)
                thrs.append(thr)
                out["%s_msg%d" % (key, it)] = msg.copy()
                out["%s_rests%d" % (key, it)] = rests.copy()
            out[key + "_thr"] = np.array(thrs, dtype=dtype)
            # data-only and update-only modes on the last gradient, no-residual threshold
            thr = ref.topk_prepare(grads[-1], np.float32(topk), ds, 10.0)
            out[key + "_thr_noresidual"] = np.array([thr], dtype=dtype)
            out[key + "_msg_dataonly"] = ref.ip_compress(grads[-1].copy(), None, thr).copy()
            u = grads[-1].copy()
            out[key + "_msg_updateonly"] = ref.ip_compress(None, u, thr).copy()
            out[key + "_upd_after"] = u
            # flush of the final residual: threshold 0, data-only
            out[key + "_msg_flush"] = ref.ip_compress(rests.copy(), None, dtype(0)).copy()
            # receive side
            base = grads[0].copy()
            dec = base.copy()
            ref.ip_decompress(out[key + "_msg0"], dec)
            add = base.copy()
            ref.ip_add(out[key + "_msg0"], add)
            out[key + "_dec0"] = dec
            out[key + "_add0"] = add
            case += 1
    out["n_cases"] = np.array([case], dtype=np.int64)
    return out


def full_size(ref):
    res = {}
    t0 = time.time()

    def ef_run(name, cfg, grad_fn, iters):
        n, topk, ds = cfg["n"], np.float32(cfg["topK"]), cfg["default_subsamples"]
        rests = np.zeros(n, np.float32)
        rows = []
        for it in range(iters):
            g = grad_fn(it)
            thr = ref.topk_prepare_with(rests, g, topk, ds, 10.0)
            msg = ref.ip_compress(g.copy(), rests, thr)
            rows.append(dict(input=W.checksum(g), thr=float(thr), thr_hex=np.float32(thr).tobytes().hex(),
                             k=int(msg[4:8].view(np.int32)[0]),
                             msg=W.checksum(msg), rests=W.checksum(rests)))
            print(name, it, rows[-1], "%.0fs" % (time.time() - t0), flush=True)
        res[name] = rows

    ef_run("C1", W.C1, W.c1_gradient, W.C1["iters"])
    ef_run("C2", W.C2, W.c2_gradient, W.C2["iters"])
    ef_run("C3", W.C3, W.c3_gradient, W.C3["iters"])

    # C4: sampled (host-supplied indices are not a reference feature; the reference-faithful
    # strided default is) and exact
    g = W.c4_gradient()
    n = g.size
    rows = {"input": W.checksum(g)}
    rests = np.zeros(n, np.float32)
    thr = ref.topk_prepare_with(rests, g, np.float32(0.01), 1000, 10.0)
    msg = ref.ip_compress(g.copy(), rests, thr)
    rows["strided"] = dict(thr_hex=np.float32(thr).tobytes().hex(), k=int(msg[4:8].view(np.int32)[0]),
                           msg=W.checksum(msg), rests=W.checksum(rests))
    rests = np.zeros(n, np.float32)
    thr = ref.topk_prepare_with(rests, g, np.float32(0.01), W.C4["default_subsamples_exact"], 10.0)
    msg = ref.ip_compress(g.copy(), rests, thr)
    rows["exact"] = dict(thr_hex=np.float32(thr).tobytes().hex(), k=int(msg[4:8].view(np.int32)[0]),
                         msg=W.checksum(msg), rests=W.checksum(rests))
    # threshold from the seeded index list = calc_threshold on the gathered sums
    idx = W.c4_sample_indices()
    thr = ref.calc_threshold(g[idx], np.float32(0.01))
    rests = np.zeros(n, np.float32)
    msg = ref.ip_compress(g.copy(), rests, thr)
    rows["indexed"] = dict(idx=W.checksum(idx), thr_hex=np.float32(thr).tobytes().hex(),
                           k=int(msg[4:8].view(np.int32)[0]), msg=W.checksum(msg), rests=W.checksum(rests))
    res["C4"] = rows
    print("C4", rows, flush=True)
    del g, rests, msg

    # C5: rank-ordered add of 8 messages into a zero vector, then residual += dense
    msgs = W.c5_messages()
    dense = np.zeros(W.C5["n"], np.float32)
    for m in msgs:
        ref.ip_add(m, dense)
    res["C5"] = dict(msgs=[W.checksum(m) for m in msgs], dense=W.checksum(dense))
    print("C5", res["C5"], flush=True)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--full", action="store_true", help="also write full_size.json (minutes)")
    args = ap.parse_args()
    ref = Oracle(ref=True)
    np.savez_compressed(os.path.join(HERE, "small_cases.npz"), **small_cases(ref))
    print("wrote small_cases.npz")
    if args.full:
        with open(os.path.join(HERE, "full_size.json"), "w") as f:
            json.dump(full_size(ref), f, indent=1, sort_keys=True)
        print("wrote full_size.json")


if __name__ == "__main__":
    main()
