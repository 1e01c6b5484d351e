"""Builds libaether_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python aether-ml_amd/build.py [--force]

Objects land in aether-ml_amd/build/, the library in aether-ml_amd/aether/lib/.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "aether", "lib")
LIB = os.path.join(LIBDIR, "libaether_hip.so")
SOURCES = ["runtime.hip", "gather_f32.hip", "gather_bf16.hip", "gather_res9_bf16.hip", "wgrad_f32.hip", "wgrad_bf16.hip", "pair_f32.hip",
           "layers.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# MFMA results in the ordinary registers: what the kernels that hold a tile's accumulators next to their operands want.  Not
# for the kernel that fills all 512 registers of a lane and needs the accumulation registers for accumulators and filter.
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
AGPR_SOURCES = {"gather_res9_bf16.hip"}


def _headers():
    out = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    out.append(os.path.join(HERE, "..", "include", "aether_hip.h"))
    out.append(os.path.abspath(__file__))       # the flags live here
    return out


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + _headers()):
        cmd = [HIPCC] + FLAGS + ([] if src in AGPR_SOURCES else VGPR_FORM) + ["-c", path, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def build(force=False):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
