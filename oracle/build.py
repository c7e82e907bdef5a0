"""Build the CPU oracle (test infrastructure) into oracle/liboracle.so with gcc."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")


def build(force=True):
    src = os.path.join(HERE, "plo_oracle.c")
    inc = os.path.join(HERE, "oracle_body.inc")
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= max(
            os.path.getmtime(src), os.path.getmtime(inc)):
        return LIB
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-fno-fast-math",
           "-ffp-contract=off", "-o", LIB, src, "-lm"]
    subprocess.run(cmd, check=True, cwd=HERE)
    return LIB


if __name__ == "__main__":
    print(build())
