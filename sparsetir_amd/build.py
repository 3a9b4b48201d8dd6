"""Builds ``libsparsetir_amd.so`` (HIP kernels + C ABI) for gfx950 with hipcc.

Run as ``python -m sparsetir_amd.build``.  hipcc cross-compiles, so no GPU is needed.
The library is placed next to this file; it is what ``sparsetir_amd._lib`` loads.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libsparsetir_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "-I", os.path.join(HERE, "..", "include")]
# Packed fp32 VALU ops are kept off for every device translation unit.
DEVICE = [f"--offload-arch={ARCH}", "-munsafe-fp-atomics",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# Per-file additions.  The destination-tiled RGMS kernel chains MFMAs through ordinary vector
# registers (one accumulator feeds the next stage's operand); with the accumulator-register form
# the compiler copies both accumulators between the two register files on every step.
EXTRA = {"rgms_tiles.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [HIPCC] + COMMON
    if src.endswith(".hip"):
        cmd += DEVICE + EXTRA.get(os.path.basename(src), []) + ["-x", "hip"]
    cmd += ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, r.returncode, r.stdout + r.stderr


def build(verbose=True, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    objs = []
    for src, obj, rc, log in results:
        log = "\n".join(l for l in log.splitlines()
                        if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
        if rc != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{log}")
        if verbose and log.strip():
            print(log)
        objs.append(obj)
    cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
