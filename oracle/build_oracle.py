"""Build the plain-C oracle (attn_ref.c -> libattn_ref.so).  Test infrastructure only.

The reference's own implementation of this path cannot be built here: it needs nvcc for sm_90a and the
ThunderKittens headers of an empty git submodule, so no oracle/_ref library exists.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "attn_ref.c")
OUT = os.path.join(HERE, "libattn_ref.so")


def build_oracle():
    cmd = ["gcc", "-O3", "-march=x86-64-v2", "-fopenmp", "-shared", "-fPIC", SRC, "-o", OUT + ".tmp", "-lm"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + r.stdout + r.stderr)
    os.replace(OUT + ".tmp", OUT)
    return OUT


if __name__ == "__main__":
    print(build_oracle())
    sys.exit(0)
