"""Seeded synthetic inputs for the five benchmark configurations.

Host-side numpy only.  Every buffer is generated once and handed, bit for bit, to
both the GPU path and the CPU checker, so no cross-machine libm agreement is
needed; ``checksum`` lets a stored fixture assert it is looking at the same bits.

Shapes follow the gradient vectors the reference feeds its compressor: one flat
fp32 blob of all layers (keras/comprex_optimizer.py:97-124).
"""
import hashlib

import numpy as np

# exact top-k mode is reached in the reference by choosing default_subsamples > n
# (src/threshold.hxx:226); a power of two survives calc_subsamples' fp32 rounding (:182-186).
C1 = dict(name="C1-1M-top1%", n=1 << 20, topK=0.01, default_subsamples=1 << 21, iters=10)
C2 = dict(name="C2-lenet5-top10%", n=61706, topK=0.1, default_subsamples=1 << 16, iters=50,
          segments=[150, 6, 2400, 16, 48000, 120, 10080, 84, 840, 10])
C3 = dict(name="C3-resnet50-top0.1%", n=25557032, topK=0.001, default_subsamples=1 << 25, iters=20,
          n_segments=161)
C4 = dict(name="C4-100M-laplace-top1%", n=100_000_000, topK=0.01, default_subsamples_exact=1 << 27,
          n_samples=100_000, spike_fraction=1e-4, spike_magnitude=1e3)
C5 = dict(name="C5-reduce-8x1%-64M", n=1 << 26, ranks=8, k=671088, shared=335544)


def checksum(a):
    return hashlib.sha256(np.ascontiguousarray(a).view(np.uint8)).hexdigest()[:16]


def normal(n, seed, dtype=np.float32):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal(n, dtype=np.float32).astype(dtype, copy=False) if dtype == np.float32 \
        else rng.standard_normal(n).astype(dtype)


def c1_gradient(it, seed=1234, n=C1["n"]):
    return normal(n, seed + it)


def c2_gradient(it, seed=2345):
    segs = C2["segments"]
    scales = np.logspace(-2, -4, num=len(segs)).astype(np.float32)
    g = normal(sum(segs), seed + it)
    off = 0
    for s, sc in zip(segs, scales):
        g[off:off + s] *= sc
        off += s
    return g


def c3_segments(seed=3456, n=C3["n"], n_segments=C3["n_segments"]):
    """161 segment sizes summing to n and their log-uniform scales in [1e-5, 1e-1]."""
    rng = np.random.Generator(np.random.PCG64(seed))
    w = rng.random(n_segments) ** 3 + 1e-4
    sizes = np.maximum(1, np.floor(w / w.sum() * n)).astype(np.int64)
    sizes[-1] += n - sizes.sum()
    assert sizes.sum() == n and (sizes > 0).all()
    scales = np.exp(rng.uniform(np.log(1e-5), np.log(1e-1), n_segments)).astype(np.float32)
    return sizes, scales


def c3_gradient(it, seed=3456, n=C3["n"], n_segments=C3["n_segments"]):
    sizes, scales = c3_segments(seed, n, n_segments)
    g = normal(n, seed + 1000 + it)
    off = 0
    for s, sc in zip(sizes, scales):
        g[off:off + s] *= sc
        off += s
    return g


def c4_gradient(seed=4567, n=C4["n"]):
    """Laplace(0,1) with a fraction of positions replaced by +-spike_magnitude."""
    rng = np.random.Generator(np.random.PCG64(seed))
    g = np.empty(n, dtype=np.float32)
    step = 1 << 24
    for off in range(0, n, step):
        m = min(step, n - off)
        g[off:off + m] = rng.laplace(0.0, 1.0, m).astype(np.float32)
    n_spikes = int(round(n * C4["spike_fraction"]))
    pos = rng.choice(n, size=n_spikes, replace=False)
    sign = rng.integers(0, 2, n_spikes).astype(np.float32) * 2 - 1
    g[pos] = sign * np.float32(C4["spike_magnitude"])
    return g


def c4_sample_indices(seed=4568, n=C4["n"], m=C4["n_samples"]):
    rng = np.random.Generator(np.random.PCG64(seed))
    return np.sort(rng.integers(0, n, m, dtype=np.int64)).astype(np.int32)


def c5_messages(seed=5678, n=C5["n"], ranks=C5["ranks"], k=C5["k"], shared=C5["shared"],
                dtype=np.float32):
    """Per-rank IndexPairs messages: `shared` indices common to all ranks plus
    k-shared indices drawn per rank (distinct from the hot set and each other),
    sorted ascending, values N(0,1).  Returns a list of uint8 message buffers."""
    rng = np.random.Generator(np.random.PCG64(seed))
    hot = rng.choice(n, size=shared, replace=False).astype(np.int64)
    msgs = []
    rec = np.dtype([("i", np.int32), ("v", np.dtype(dtype))], align=False)
    for r in range(ranks):
        need = k - shared
        own = np.empty(0, dtype=np.int64)
        while own.size < need:  # re-draw on collision
            cand = rng.integers(0, n, int((need - own.size) * 1.1) + 16, dtype=np.int64)
            cand = np.setdiff1d(np.unique(cand), hot, assume_unique=True)
            own = np.union1d(own, cand)
        if own.size > need:
            own = rng.permutation(own)[:need]
        idx = np.sort(np.concatenate([hot, own])).astype(np.int32)
        assert idx.size == k and (np.diff(idx) > 0).all()
        body = np.empty(k, dtype=rec)
        body["i"] = idx
        body["v"] = rng.standard_normal(k).astype(dtype)
        msg = np.empty(8 + k * rec.itemsize, dtype=np.uint8)
        msg[:8] = np.array([n, k], dtype=np.int32).view(np.uint8)
        msg[8:] = body.view(np.uint8)
        msgs.append(msg)
    return msgs
