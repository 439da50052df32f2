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


# ---- check of the generated code around the hand-written vector-memory instructions
#
# The kernels issue their direct-to-LDS loads (and a few register loads) from asm statements, which
# the compiler's hazard recognizer does not look into.  One hardware rule then has nobody to keep
# it: a vector-memory instruction that reads a scalar register needs five wait states after a
# VECTOR instruction that wrote that register (v_readlane_b32 restoring a spilled descriptor,
# v_readfirstlane_b32, a compare into a register pair); without them it reads the old value -
# a load with a stale descriptor returns zeros or touches memory it should not.  The register
# loads carry their own wait states (lds_dma.h); for the LDS loads of the step loops this pass
# over the device assembly of every translation unit proves there is no such neighbour.

_VALU_SGPR_WRITERS = ("v_readlane_b32", "v_readfirstlane_b32", "v_cmp", "v_add_co", "v_sub_co", "v_subrev_co",
                      "v_addc_co", "v_subb_co", "v_subbrev_co", "v_div_scale", "v_mad_u64_u32", "v_mad_i64_i32",
                      "v_cmpx")


def _sgprs(text):
    """Scalar registers named in an operand string: 's5' -> {5}, 's[4:7]' -> {4, 5, 6, 7}."""
    import re
    found = set()
    for lo, hi in re.findall(r"\bs\[(\d+):(\d+)\]", text):
        found.update(range(int(lo), int(hi) + 1))
    for one in re.findall(r"\bs(\d+)\b", text):
        found.add(int(one))
    if "vcc" in text:
        found.update((-1, -2))   # vcc_lo, vcc_hi
    return found


def find_asm_hazards(asm_text, window=5):
    """[(kernel, line number, the load, the writer)] for every vector-memory instruction inside an
    asm statement whose scalar operands were written by a vector instruction fewer than `window`
    wait states earlier (straight-line code: a label ends the look-back)."""
    import re
    findings = []
    kernel = "?"
    history = []          # (wait states this instruction is worth, written scalar registers, text)
    in_asm = False
    for number, raw in enumerate(asm_text.split("\n"), 1):
        line = raw.split(";")[0].strip() if not raw.strip().startswith(";;#") else raw.strip()
        if raw.strip().startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if raw.strip().startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not line or line.startswith("."):
            if re.match(r"^\.LBB\d+_\d+:", line or ""):
                history = []
            continue
        if line.endswith(":"):
            if not line.startswith(".L"):
                kernel = line[:-1]
            history = []
            continue
        op, _, rest = line.partition(" ")
        if in_asm and (op.startswith("buffer_load") or op.startswith("buffer_store") or op.startswith("global_") or
                       op.startswith("flat_")):
            reads = _sgprs(rest)
            states = 0
            for worth, written, text in reversed(history):
                if states >= window:
                    break
                if written & reads:
                    findings.append((kernel, number, line, text))
                    break
                states += worth
        worth = 1
        written = set()
        if op == "s_nop":
            worth = int(rest.strip() or 0) + 1
        elif op.startswith(_VALU_SGPR_WRITERS):
            first = rest.split(",")[0]
            written = _sgprs(first)
            if op.startswith(("v_add_co", "v_sub_co", "v_subrev_co", "v_addc_co", "v_subb_co", "v_subbrev_co",
                              "v_div_scale", "v_mad_u64_u32", "v_mad_i64_i32")):
                parts = rest.split(",")
                written = _sgprs(parts[1]) if len(parts) > 1 else set()
            if op.startswith("v_cmp") and op.endswith("_e32"):
                written = {-1, -2}
        history.append((worth, written, line))
        if len(history) > 16:
            history.pop(0)
    return findings


def _device_asm(unit, force):
    name, src, defs = unit
    out = os.path.join(OBJ, name + ".s")
    stamp = max(os.path.getmtime(src), _headers_mtime())
    if force or not os.path.exists(out) or os.path.getmtime(out) < stamp:
        cmd = [HIPCC] + [f for f in FLAGS if f != "-fPIC"] + defs + ["-S", "--cuda-device-only", src, "-o", out]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("hipcc -S failed for %s:\n%s" % (name, res.stdout))
    return out


def check_asm_hazards(force=False, jobs=None):
    """Compile every translation unit to device assembly (kept beside the objects, redone when a
    source is newer) and look for the hazard described above; returns the findings."""
    os.makedirs(OBJ, exist_ok=True)
    units = [u for u in _units() if u[0].startswith(("rowgemm", "tilegemm"))]   # the units with asm loads
    jobs = jobs or min(len(units), max(1, (os.cpu_count() or 2)), 8)
    with ThreadPoolExecutor(jobs) as pool:
        files = list(pool.map(lambda u: _device_asm(u, force), units))
    findings = []
    for unit, path in zip(units, files):
        with open(path) as f:
            findings += [(unit[0],) + hit for hit in find_asm_hazards(f.read())]
    return findings


if __name__ == "__main__":
    if "--check-hazards" in sys.argv:
        hits = check_asm_hazards(force="--force" in sys.argv)
        for hit in hits:
            print("%s: %s line %d: %s   <- %s" % hit)
        print("%d hazard(s)" % len(hits))
        sys.exit(1 if hits else 0)
    build(force="--force" in sys.argv, verbose=True)
    print(LIB)
