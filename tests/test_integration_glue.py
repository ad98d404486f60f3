"""CPU-only: the glue a maintainer of the reference adds to run its own graph runtime on this library
(cvm-runtime_amd/integration/hip_device.cc) compiles against the reference's headers, and -- where the
reference runtime has been compiled (oracle/_ref) -- links with it and registers every operator name this
library's own registry lists, plus the device API, in the reference's registry.  Skipped where the
reference tree is absent (it does not travel)."""
import os
import subprocess

import pytest

import cvm_runtime_amd
from cvm_runtime_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GLUE = os.path.join(ROOT, "cvm-runtime_amd", "integration", "hip_device.cc")
REF = os.environ.get("CVM_REFERENCE", "/root/reference")
REF_LIB = os.path.join(ROOT, "oracle", "_ref", "libcvm_runtime_ref.so")

needs_ref = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "include", "cvm")), reason="reference headers not present")

LIST_MAIN = r"""
#include <cvm/runtime/registry.h>
#include <cstdio>
int main() {
  for (const std::string& n : cvm::runtime::Registry::ListNames())
    if (n.find("cvm.runtime.hip.") == 0 || n == "device_api.hip") std::printf("%s\n", n.c_str());
  const cvm::runtime::PackedFunc* f = cvm::runtime::Registry::Get("device_api.hip");
  return f ? 0 : 3;
}
"""


@needs_ref
def test_glue_compiles_against_the_reference_headers():
    r = subprocess.run(["g++", "-std=c++11", "-fsigned-char", "-Wall", "-Werror", "-fsyntax-only", "-I" + os.path.join(REF, "include"),
                        "-I" + os.path.join(ROOT, "include"), GLUE], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]


@needs_ref
@pytest.mark.skipif(not os.path.exists(REF_LIB), reason="compiled reference runtime (oracle/_ref) not present")
def test_glue_links_and_registers_every_operator(tmp_path):
    cvm_runtime_amd.lib()   # fails loudly when the library is not built
    libdir = os.path.join(ROOT, "cvm-runtime_amd")
    main = tmp_path / "list_main.cc"
    main.write_text(LIST_MAIN)
    exe = str(tmp_path / "list_hip_ops")
    cmd = ["g++", "-std=c++11", "-fsigned-char", "-O0", "-I" + os.path.join(REF, "include"), "-I" + os.path.join(ROOT, "include"),
           GLUE, str(main), "-o", exe, "-L" + os.path.dirname(REF_LIB), "-lcvm_runtime_ref", "-L" + libdir, "-lcvm_runtime_hip",
           "-Wl,-rpath," + os.path.dirname(REF_LIB), "-Wl,-rpath," + libdir, "-fopenmp", "-pthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stderr[-2000:])
    names = set(r.stdout.split())
    assert "device_api.hip" in names
    ops = {n for n in names if n.startswith("cvm.runtime.hip.")}
    assert ops == set(runtime.list_ops()) and len(ops) == 37, sorted(ops ^ set(runtime.list_ops()))
