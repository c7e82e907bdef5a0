"""Seed-stable synthetic inputs -- TEST INFRASTRUCTURE ONLY.

A counter-based generator (splitmix64 over the element index, Box-Muller for
normals) written in numpy integer arithmetic, so the same seed gives the same
bits in any container and under any torch version.  The five named workloads
are the benchmark's configurations; ``scale`` shrinks them for CPU-sized tests.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = x
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def _bits(seed, stream, count, chunk_start=0):
    idx = np.arange(chunk_start, chunk_start + count, dtype=np.uint64)
    with np.errstate(over="ignore"):
        key = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream))
        return _splitmix64(idx ^ key)


def uniform01(seed, stream, count):
    """float64 in (0, 1): 53 random bits, never exactly 0."""
    b = _bits(seed, stream, count)
    return ((b >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, stream, shape, mean=0.0, std=1.0, dtype=np.float32):
    count = int(np.prod(shape))
    out = np.empty(count, dtype=dtype)
    step = 1 << 22
    for s in range(0, count, step):
        n = min(step, count - s)
        b1 = _bits(seed, 2 * stream, n, s)
        b2 = _bits(seed, 2 * stream + 1, n, s)
        u1 = ((b1 >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)
        u2 = ((b2 >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
        out[s:s + n] = (mean + std * z).astype(dtype)
    return out.reshape(shape)


def randint(seed, stream, shape, low, high):
    count = int(np.prod(shape))
    b = _bits(seed, stream, count)
    return (low + (b >> np.uint64(16)) % np.uint64(high - low)).astype(np.int64).reshape(shape)


def bernoulli(seed, stream, shape, p):
    count = int(np.prod(shape))
    return (uniform01(seed, stream, count) < p).reshape(shape)


def categorical(seed, stream, shape, probs):
    count = int(np.prod(shape))
    cdf = np.cumsum(np.asarray(probs, dtype=np.float64))
    cdf /= cdf[-1]
    u = uniform01(seed, stream, count)
    return np.minimum(np.searchsorted(cdf, u, side="right"), len(probs) - 1).astype(np.int64).reshape(shape)


def seg_labels(seed, shape, n_classes, ignore_index=255, ignore_frac=0.05, probs=None):
    """Uniform (or ``probs``-distributed) class labels with an independent ignore mask."""
    if probs is None:
        lb = randint(seed, 11, shape, 0, n_classes)
    else:
        lb = categorical(seed, 11, shape, probs)
    if ignore_frac > 0:
        lb[bernoulli(seed, 12, shape, ignore_frac)] = ignore_index
    return lb


def zipf_probs(n_classes, s=1.1):
    p = (np.arange(n_classes, dtype=np.float64) + 1.0) ** (-s)
    return p / p.sum()


def _scaled(hw, scale):
    return tuple(max(1, int(round(d * scale))) for d in hw)


def workload(name, seed=15, scale=1.0, batch=None):
    """Inputs of one named benchmark configuration.

    -> dict(op=..., logits=..., labels=..., kwargs=constructor arguments)
    """
    if name == "cfg1":   # CPU plumbing case
        shape = (2, 19) + _scaled((64, 64), scale)
        return dict(op="lsr", logits=normal(seed, 1, shape, 0.0, 2.0),
                    labels=seg_labels(seed, shape[:1] + shape[2:], 19),
                    kwargs=dict(lb_smooth=0.1, reduction="mean", ignore_index=255))
    if name in ("cfg2", "cfg4"):
        shape = (batch or 8, 19) + _scaled((1024, 1024), scale)
        kw = (dict(lb_smooth=0.1, reduction="mean", ignore_index=255) if name == "cfg2"
              else dict(lam=0.3, reduction="mean", ignore_index=255))
        return dict(op="lsr" if name == "cfg2" else "lmargin",
                    logits=normal(seed, 1, shape, 0.0, 2.0),
                    labels=seg_labels(seed, shape[:1] + shape[2:], 19), kwargs=kw)
    if name == "cfg3":
        shape = (batch or 16, 80) + _scaled((128, 128), scale)
        return dict(op="focal", logits=normal(seed, 1, shape, -2.0, 1.5),
                    labels=bernoulli(seed, 11, shape, 0.02).astype(np.float32),
                    kwargs=dict(alpha=0.25, gamma=2, reduction="mean"))
    if name == "cfg5":
        shape = (batch or 4, 19) + _scaled((512, 1024), scale)
        return dict(op="lovasz", logits=normal(seed, 1, shape, 0.0, 2.0),
                    labels=seg_labels(seed, shape[:1] + shape[2:], 19, probs=zipf_probs(19, 1.1)),
                    kwargs=dict(reduction="mean", ignore_index=255))
    raise KeyError(name)
