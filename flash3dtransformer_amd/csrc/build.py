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
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-inline-asm",
]
# MFMA accumulators live in ordinary VGPRs (unified register file on gfx90a+): the softmax and the
# epilogues read them without v_accvgpr moves
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
NO_VGPR_FORM = set()
# bit-exact integer / quantiser kernels: no fused multiply-add contraction
EXACT = {"psh_bucket.hip", "subbuck_pool.hip", "unpool.hip", "pool_bwd.hip"}


def sources():
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _newest_header():
    return max(os.path.getmtime(os.path.join(d, f)) for d in (HERE, os.path.join(os.path.dirname(PKG), "include"))
               for f in os.listdir(d) if f.endswith(".h"))


def _compile(src, incremental=False):
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(
            os.path.getmtime(os.path.join(HERE, src)), _newest_header(), os.path.getmtime(__file__)):
        return obj
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


def build(verbose=True, jobs=None, incremental=False):
    """incremental=True keeps objects that are newer than their source, every header and this file (a developer's
    shortcut: `python -m flash3dtransformer_amd.csrc.build -i`); the default compiles everything."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda f: _compile(f, incremental), srcs))
    cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", LIB] + objs
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError(f"link failed:\n{p.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


if __name__ == "__main__":
    build(incremental="-i" in sys.argv[1:])
