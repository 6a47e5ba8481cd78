"""Build recipe for the gfx950 shared library (hipcc cross-compiles without a GPU).

    python -m flex_block_attn_amd.build            # compile csrc/*.hip -> csrc/libfba_gfx950.so
    python -m flex_block_attn_amd.build --verbose  # also print per-kernel register / LDS usage

The library is built in-tree so that it travels with the source tree to the machine that has the GPU.
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_NAME = "libfba_gfx950.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)
SOURCES = ["fba_api.hip", "fba_mask_compact.hip", "fba_ssta_mask.hip", "fba_fwd.hip", "fba_bwd_dq.hip", "fba_bwd_dq_ds.hip", "fba_bwd_dkdv.hip", "fba_bwd_dkdv64.hip", "fba_probe.hip", "fba_split.hip"]

# Per-file extras.  --amdgpu-mfma-vgpr-form keeps MFMA accumulators in ordinary VGPRs, so the softmax arithmetic on
# them needs no accumulator-register copies; it pays off where the whole working set fits 256 registers.
EXTRA_FLAGS = {
    "fba_fwd.hip": ["-mllvm", "--amdgpu-mfma-vgpr-form"],
    "fba_bwd_dq.hip": ["-mllvm", "--amdgpu-mfma-vgpr-form"],
    "fba_bwd_dq_ds.hip": ["-mllvm", "--amdgpu-mfma-vgpr-form"],
    "fba_bwd_dkdv64.hip": ["-mllvm", "--amdgpu-mfma-vgpr-form"],
}

# -packed-fp32-ops is switched off: hipcc otherwise fuses pairs of fp32 operations into packed instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffast-math",
    "-fno-finite-math-only",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 library cannot be built")
    return exe


def _compile_one(src, verbose):
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [_hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        cmd += ["-Rpass-analysis=kernel-resource-usage"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{log}")
    return obj, log


def build_library(verbose=False):
    """Compile every HIP source and link libfba_gfx950.so. Returns the library path."""
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as ex:
        results = list(ex.map(lambda s: _compile_one(s, verbose), SOURCES))
    if verbose:
        for _, log in results:
            if log:
                print(log)
    objs = [o for o, _ in results]
    tmp = LIB_PATH + ".tmp"
    r = subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}{r.stderr}")
    os.replace(tmp, LIB_PATH)
    for o in objs:
        os.remove(o)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--verbose", action="store_true")
    args = ap.parse_args()
    print(build_library(verbose=args.verbose))
    sys.exit(0)
