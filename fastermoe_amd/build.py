"""Builds ``fastermoe_amd/lib/libfmoe_hip.so`` (gfx950) with hipcc.

``python -m fastermoe_amd.build`` compiles every translation unit under
``csrc/`` in parallel and links them into one shared library that exports the
C ABI declared in ``include/fmoe_hip.h``.  The grouped-GEMM template is
compiled once per (element type, product) so that the nine variants build side
by side.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libfmoe_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: the packed fp32 VALU forms are not
# to be generated for this target.
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# extra -D switches for experiments, e.g. FMOE_EXTRA_FLAGS="-DFMOE_X=1"
FLAGS += os.environ.get("FMOE_EXTRA_FLAGS", "").split()

PLAIN_UNITS = ["error.cpp", "profile.cpp", "routing.hip", "segment_table.hip", "permute.hip", "combine.hip", "grouped_gemm.hip", "gemm_any.hip", "pipeline.hip"]
GEMM_TYPES = {0: "f32", 1: "bf16", 2: "f16"}
GEMM_PRODUCTS = {0: "fwd", 1: "dgrad", 2: "wgrad"}


def _units():
    units = []
    for src in PLAIN_UNITS:
        if os.path.exists(os.path.join(CSRC, src)):
            units.append((src, os.path.splitext(src)[0] + ".o", []))
    for t, tname in GEMM_TYPES.items():
        for p, pname in GEMM_PRODUCTS.items():
            units.append(("gemm_inst.hip", f"gemm_{tname}_{pname}.o",
                          [f"-DFMOE_GEMM_TYPE={t}", f"-DFMOE_GEMM_PRODUCT={p}"]))
    return units


def _compile(unit):
    src, obj, defs = unit
    cmd = [HIPCC] + FLAGS + defs + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", os.path.join(OBJ, obj)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    return proc.returncode, obj, log


def build(jobs=None, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    units = _units()
    jobs = jobs or min(8, os.cpu_count() or 1)
    failed = False
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for rc, obj, log in pool.map(_compile, units):
            if log.strip() and (verbose or rc != 0):
                print(f"--- {obj}\n{log}", file=sys.stderr)
            failed |= rc != 0
    if failed:
        raise RuntimeError("hipcc failed; see the log above")
    objs = [os.path.join(OBJ, u[1]) for u in units]
    link = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB] + objs
    subprocess.check_call(link)
    # a kernel the compiler dropped shows up as an undefined symbol when the library is loaded
    import ctypes
    ctypes.CDLL(LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
