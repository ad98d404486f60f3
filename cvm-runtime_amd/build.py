"""Build the gfx950 shared library in-tree: python cvm-runtime_amd/build.py

Every .hip / .cc file under csrc/ is compiled with hipcc for gfx950 and linked
into cvm-runtime_amd/libcvm_runtime_hip.so, the one library that exports both
the operator-level C ABI (include/cvm_hip_ops.h) and the model-level C ABI
(include/cvm_c_api.h).
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libcvm_runtime_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-fPIC", "-std=c++17", "-fsigned-char", "-fvisibility=hidden", "-I" + os.path.join(HERE, "..", "include")]
# extra preprocessor definitions for a measurement build, e.g. CVM_HIP_DEFINES="-DCVM_SEQ_STAMPS"
COMMON += os.environ.get("CVM_HIP_DEFINES", "").split()
# packed-fp32 code generation is switched off for all device code
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ, rel + ".o")
    cmd = [HIPCC] + COMMON + (DEVICE if src.endswith(".hip") else ["-x", "c++"]) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        sys.stderr.write(out + "\n")
    return obj


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "**", "*.cc"), recursive=True))
    with ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs + ["-Wl,-Bsymbolic"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
