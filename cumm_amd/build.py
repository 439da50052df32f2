"""Ahead-of-time build of libcummhip.so for gfx950 (no JIT at run time).

``python -m cumm_amd.build`` compiles every HIP translation unit under
``cumm_amd/csrc`` with hipcc and links them into ``cumm_amd/libcummhip.so``.
This replaces the reference's NVRTC / pccm JIT builds
(cumm/nvrtc/__init__.py:179-283, cumm/gemm/main_real.py:59-70).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "libcummhip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-inline-asm",   # the direct-to-LDS loads set M0 themselves
         # MFMA accumulators in ordinary VGPRs: with AGPR accumulators the multi-exit step loops
         # copy every accumulator AGPR -> VGPR -> AGPR once per trip (a quarter of the loop's
         # vector instructions in the 64x128 kernels)
         "-mllvm", "-amdgpu-mfma-vgpr-form=1"]

ELEMS = [("F16", "f16"), ("BF16", "bf16"), ("S8", "s8")]


def _units():
    units = [("api", os.path.join(CSRC, "api.hip"), []),
             ("pairs", os.path.join(CSRC, "pairs_inst.hip"), []),
             ("gather", os.path.join(CSRC, "gather_inst.hip"), []),
             ("elementwise", os.path.join(CSRC, "elementwise_inst.hip"), []),
             ("sort", os.path.join(CSRC, "sort_inst.hip"), [])]
    for tag, name in ELEMS:
        defs = ["-DCUMM_ELEM=%s" % tag, "-DCUMM_NAME=%s" % name]
        units.append(("rowgemm_" + name, os.path.join(CSRC, "rowgemm_inst.hip"), defs))
        extra = ["-DCUMM_NO_WGRAD_ATOMIC"] if tag == "S8" else []   # no s8 backward pass
        units.append(("tilegemm_" + name, os.path.join(CSRC, "tilegemm_inst.hip"), defs + extra))
        # the same kernels with four-byte outputs (s8 -> s32, f16 / bf16 -> f32)
        units.append(("rowgemm_wide_" + name, os.path.join(CSRC, "rowgemm_inst.hip"), defs + ["-DCUMM_WIDE=1"]))
        units.append(("tilegemm_wide_" + name, os.path.join(CSRC, "tilegemm_inst.hip"), defs + ["-DCUMM_WIDE=1"]))
    return units


def _headers_mtime():
    newest = 0.0
    for root in (CSRC, os.path.join(HERE, "..", "include")):
        for f in os.listdir(root):
            if f.endswith(".h"):
                newest = max(newest, os.path.getmtime(os.path.join(root, f)))
    return newest


def _compile(unit, force, verbose):
    name, src, defs = unit
    obj = os.path.join(OBJ, name + ".o")
    stamp = max(os.path.getmtime(src), _headers_mtime())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= stamp:
        return obj
    cmd = [HIPCC] + FLAGS + defs + ["-c", src, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (name, out))
    if verbose and out.strip():
        print(out, flush=True)
    return obj


def build(force=False, verbose=False, jobs=None):
    """Compile (if stale or ``force``) and link; returns the path of the library."""
    os.makedirs(OBJ, exist_ok=True)
    units = _units()
    jobs = jobs or min(len(units), max(1, (os.cpu_count() or 2)), 8)
    with ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(lambda u: _compile(u, force, verbose), units))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
    print(LIB)
