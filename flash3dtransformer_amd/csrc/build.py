"""Builds flash3dtransformer_amd/lib/libf3d_hip.so from the HIP sources in this directory.

    python -m flash3dtransformer_amd.csrc.build        # or: python flash3dtransformer_amd/csrc/build.py

hipcc cross-compiles for gfx950 without a GPU.  Objects go to csrc/build/, the library next to the
Python binding so that it travels with the tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "lib", "libf3d_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]
# MFMA accumulators live in ordinary VGPRs (unified register file on gfx90a+): the softmax and the
# epilogues read them without v_accvgpr moves
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
NO_VGPR_FORM = set()
# bit-exact integer / quantiser kernels: no fused multiply-add contraction
EXACT = {"psh_bucket.hip", "subbuck_pool.hip", "unpool.hip", "pool_bwd.hip"}


def sources():
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    cmd = ["hipcc", "-c", os.path.join(HERE, src), "-o", obj] + COMMON
    cmd += ["-ffp-contract=off"] if src in EXACT else ["-ffp-contract=fast"]
    if src not in NO_VGPR_FORM:
        cmd += VGPR_FORM
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", LIB] + objs
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError(f"link failed:\n{p.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build()
