"""Host-side checks that need no GPU: the shared library loads and exports every declared symbol,
the C++ header is source-compatible with the reference's driver, and the C++ MemRefFlatArray
reads/writes the same bytes as the Python tooling."""
import ctypes
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from nncv_amd import abi, modelbin, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_MAIN = "/root/reference/examples/Res18/main.cpp"


def test_library_exports_every_declared_symbol():
    if not os.path.exists(abi.LIB_PATH):
        pytest.skip("libnncv_hip.so not built here")
    header = open(os.path.join(ROOT, "include", "nncv_hip.h")).read()
    declared = set(re.findall(r"\b(_mlir_ciface_\w+|nncv_hip_\w+)\s*\(", header))
    declared -= {"nncv_hip_model", "nncv_hip_conv"}
    assert declared == set(abi.EXPORTS), declared ^ set(abi.EXPORTS)
    L = ctypes.CDLL(abi.LIB_PATH)  # load only; no compute call without a GPU
    for name in declared:
        assert hasattr(L, name), name


def test_descriptor_sizes():
    assert ctypes.sizeof(abi.MemRef1D) == 40
    assert ctypes.sizeof(abi.MemRef2D) == 56
    assert ctypes.sizeof(abi.MemRef4D) == 88


@pytest.mark.skipif(not os.path.exists(REF_MAIN) or shutil.which("g++") is None, reason="reference tree absent")
def test_reference_driver_compiles_against_this_header():
    """examples/Res18/main.cpp must compile unchanged with include/libnncv/DataType.hpp."""
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I" + os.path.join(ROOT, "include"),
                        "-I/root/reference/third_party/stb_image", REF_MAIN], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_cpp_flat_array_matches_python_tooling(tmp_path):
    src = tmp_path / "t.cpp"
    src.write_text(r'''
#include "libnncv/DataType.hpp"
#include <cstring>
using namespace nncv::rt;
int main(int argc, char** argv) {
  MemRefFlatArray in(dataType::kFloat32);
  if (!in.read(argv[1])) return 1;
  auto* d = in.getWrapedData<MemRefDescriptor<float, 1>>();
  if (d->sizes[0] != 76 || d->strides[0] != 1 || d->offset != 0) return 2;
  MemRefFlatArray out(dataType::kFloat32);
  size_t off = 0;
  for (const auto& ix : in.indexers()) {
    out.addMemRefIndexer(ix, d->aligned + off);
    size_t n = 1; for (size_t k = 0; k < ix.dims; ++k) n *= ix.shape[k];
    off += n;
  }
  if (!out.write(argv[2])) return 3;
  MemRefFlatArray bad(dataType::kFloat32);
  if (bad.read("/nonexistent/model.bin")) return 4;
  if (bad.read(argv[3])) return 5;   // truncated file must be refused
  return 0;
}''')
    exe = tmp_path / "t"
    lib_src = os.path.join(ROOT, "nncv_amd", "csrc", "datatype.cpp")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"), str(src), lib_src, "-o", str(exe)])
    ts = [("conv.weight", synth.normal(1, (2, 3, 3, 3))), ("bn.weight", synth.uniform(2, (2,), 0.5, 1.5)),
          ("fc.weight", synth.normal(3, (5, 4)))]
    a, b, c = str(tmp_path / "a.bin"), str(tmp_path / "b.bin"), str(tmp_path / "c.bin")
    modelbin.write(a, ts)
    raw = open(a, "rb").read()
    open(c, "wb").write(raw[:-10])
    assert subprocess.call([str(exe), a, b, c], stdout=subprocess.DEVNULL) == 0
    assert open(b, "rb").read() == raw
