"""Build libpytorch_loss_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python pytorch-loss_amd/build.py            # rebuild everything
    python pytorch-loss_amd/build.py --if-stale # only what changed

Objects go to pytorch-loss_amd/build/, the shared library next to the Python
package (pytorch-loss_amd/pytorch_loss/libpytorch_loss_hip.so) so that it
travels with the source tree.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "pytorch_loss", "libpytorch_loss_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "--offload-compress", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def _includes(path, seen=None):
    """The csrc/ and include/ headers that `path` pulls in through #include "...", transitively."""
    seen = set() if seen is None else seen
    for line in open(path, errors="replace"):
        line = line.strip()
        if line.startswith('#include "'):
            name = line.split('"')[1]
            for base in (CSRC, os.path.join(os.path.dirname(HERE), "include")):
                cand = os.path.join(base, name)
                if os.path.exists(cand) and cand not in seen:
                    seen.add(cand)
                    _includes(cand, seen)
    return seen


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=True, verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    jobs = []
    objs = []
    for src in sources:
        obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if force or _stale(obj, [src] + sorted(_includes(src))):
            jobs.append([HIPCC] + FLAGS + ["-c", src, "-o", obj])

    def run(cmd):
        t0 = time.time()
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-8000:]))
        if verbose:
            print("%6.1f s  %s" % (time.time() - t0, os.path.basename(cmd[-1])), flush=True)
        return r.stderr

    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "8")), 16))
    # the units that take longest (the backward kernels hold two slices) start first
    def weight(cmd):
        name = os.path.basename(cmd[-3])
        return (-(4 * ("taylor" in name) + 2 * ("layernorm" in name) + ("bwd" in name or "both" in name)), name)
    jobs.sort(key=weight)
    t_all = time.time()
    if jobs:
        with concurrent.futures.ThreadPoolExecutor(workers) as pool:
            for _ in pool.map(run, jobs):
                pass
    if jobs or force or _stale(LIB, objs):
        run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB])
    if verbose:
        print("%d units on %d workers in %.0f s; %s: %.1f MiB" % (len(jobs), workers, time.time() - t_all, os.path.basename(LIB),
                                                                 os.path.getsize(LIB) / 2**20), flush=True)
    return LIB


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv, verbose=True))
