"""Writes tests/golden/*.npz: expected outputs for the four losses on seed-fixed inputs.

The reference holds no golden vectors, known-answer tests or fixtures for this path, and every
function of the CPU oracle is pinned without it (tests/test_oracle_pinning.py: library
identities, brute force from the definition, fp64 autograd of independent formulations), so the
reference is NOT imported here.  The vectors below come from the fp64 instantiation of that
pinned oracle; they freeze its results so that a later change to the oracle, to the input
generator or to a kernel shows up against a fixed record.  Inputs are not stored: they are
regenerated from oracle/synth.py (bit-stable, checked in test_oracle_pinning.py).

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from oracle import synth  # noqa: E402

SEED = 15
SMALL = (2, 19, 16, 16)       # per-element outputs are stored for this shape
CFG1 = (2, 19, 64, 64)        # the CPU-runnable benchmark configuration: scalars only


def inputs(shape, kind):
    if kind == "focal":
        x = synth.normal(SEED, 1, shape, -2.0, 1.5)
        y = synth.bernoulli(SEED, 11, shape, 0.02).astype(np.float32)
        return x, y
    probs = synth.zipf_probs(shape[1], 1.1) if kind == "lovasz" else None
    x = synth.normal(SEED, 1, shape, 0.0, 2.0)
    y = synth.seg_labels(SEED, shape[:1] + shape[2:], shape[1], 255, 0.05, probs)
    return x, y


def record(kind, shape):
    x, y = inputs(shape, kind)
    x64 = x.astype(np.float64)
    if kind == "lsr":
        per = oracle.lsr_forward(x64, y, 255, 0.1)
        grad = oracle.lsr_backward(x64, y, 255, 0.1)
        mean, total = oracle.reduce_pixels(per, y, "mean", 255), per.sum()
    elif kind == "lmargin":
        per = oracle.lmargin_forward(x64, y, 0.3, 255)
        grad = oracle.lmargin_backward(x64, y, 0.3, 255)
        mean, total = oracle.reduce_pixels(per, y, "mean", 255), per.sum()
    elif kind == "focal":
        y64 = y.astype(np.float64)
        per = oracle.focal_forward(x64, y64, 0.25, 2.0)
        grad = oracle.focal_backward(x64, y64, 0.25, 2.0)
        mean, total = per.mean(), per.sum()
    else:
        per, jacc = oracle.lovasz_forward(x64, y, 255)
        grad = oracle.lovasz_backward(np.ones(shape[1]), x64, y, jacc, 255)
        mean, total = per.mean(), per.sum()
    return dict(per=per, grad=grad, mean=np.float64(mean), sum=np.float64(total),
                n_valid=np.int64((y != 255).sum()) if kind != "focal" else np.int64(y.size),
                input_checksum=np.float64(x64.sum()), label_checksum=np.float64(np.asarray(y, dtype=np.float64).sum()))


def main():
    for kind in ("lsr", "lmargin", "focal", "lovasz"):
        small = record(kind, SMALL)
        big = record(kind, CFG1)
        out = {"small_" + k: v for k, v in small.items()}
        out.update({"cfg1_" + k: v for k, v in big.items() if k not in ("per", "grad")})
        if kind == "lovasz":
            out["cfg1_per"] = big["per"]           # 19 per-class losses
        path = os.path.join(HERE, kind + ".npz")
        np.savez_compressed(path, **out)
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
