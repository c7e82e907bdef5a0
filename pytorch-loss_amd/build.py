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

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "pytorch_loss", "libpytorch_loss_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=True, verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    headers = sorted(glob.glob(os.path.join(CSRC, "*.hpp"))) + [
        os.path.join(os.path.dirname(HERE), "include", "pytorch_loss_hip.h")]
    jobs = []
    objs = []
    for src in sources:
        obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if force or _stale(obj, [src] + headers):
            jobs.append([HIPCC] + FLAGS + ["-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-8000:]))
        return r.stderr

    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "8")), 16))
    if jobs:
        with concurrent.futures.ThreadPoolExecutor(workers) as pool:
            for warn in pool.map(run, jobs):
                if verbose and warn.strip():
                    print(warn)
    if jobs or force or _stale(LIB, objs):
        run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv, verbose=True))
