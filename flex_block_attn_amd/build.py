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


# Sources whose accumulating matrix instructions are inline asm (accumulation-register form).  The compiler gives a
# matrix instruction of its own the wait states it needs behind a vector instruction that writes one of its operands;
# an inline-asm one gets none and then reads what the register held before.  The sources keep such writes away from
# those instructions (opaque pins); this check reads the compiler's assembly of our own kernels and fails the build if a
# schedule ever brings one within `ASM_HAZARD_WINDOW` instructions again.
ASM_MFMA_SOURCES = ["fba_bwd_dkdv64.hip"]
ASM_HAZARD_WINDOW = 4


def find_asm_mfma_hazards(asm_text, window=ASM_HAZARD_WINDOW):
    """[(writer, matrix instruction, distance)] for every vector instruction that writes a register which an
    accumulation-register matrix instruction at most `window` instructions later reads as operand A or B."""
    import re

    def regs(tok):
        m = re.match(r"v\[(\d+):(\d+)\]$", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.match(r"v(\d+)$", tok)
        return {int(m.group(1))} if m else set()

    ins = []
    for line in asm_text.split("\n"):
        t = line.strip()
        if not t or t.startswith(";") or t.startswith("."):
            continue  # comments, directives and labels (a block may be fallen into, so labels do not end the search)
        ins.append(t)
    found = []
    for i, t in enumerate(ins):
        if not (t.startswith("v_mfma") and " a[" in t):
            continue
        ops = [o.strip() for o in t.split(None, 1)[1].split(",")]
        src = regs(ops[1]) | regs(ops[2])
        for back in range(1, window + 1):
            if i - back < 0:
                break
            w = ins[i - back]
            if w.startswith("v_") and not w.startswith("v_mfma") and not w.startswith("v_accvgpr_read") and " " in w:
                if regs(w.split(None, 1)[1].split(",")[0].strip()) & src:
                    found.append((w, t, back))
    return found


def check_asm_mfma_hazards():
    """Compiles the sources with inline-asm matrix instructions to assembly and raises if a hazard is found."""
    for src in ASM_MFMA_SOURCES:
        cmd = [_hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", "-"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc -S failed for {src}:\n{r.stderr[-2000:]}")
        found = find_asm_mfma_hazards(r.stdout)
        if found:
            lines = "\n".join(f"  {w}   ->   {m} (distance {d})" for w, m, d in found)
            raise RuntimeError(f"{src}: a vector instruction writes an operand of an inline-asm matrix instruction right in front of it:\n{lines}")


def build_library(verbose=False):
    """Compile every HIP source and link libfba_gfx950.so. Returns the library path."""
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as ex:
        check = ex.submit(check_asm_mfma_hazards)
        results = list(ex.map(lambda s: _compile_one(s, verbose), SOURCES))
        check.result()
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
