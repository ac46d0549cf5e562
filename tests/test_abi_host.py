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


def test_arena_planner_known_answer_and_validity():
    """Greedy-by-size offset planning: the reference's own known-answer case
    (tests/MemSolver/test.cpp:17-37, the example of arXiv 2001.03288: total 124), then random
    cases checked for the two properties that matter: tensors live at the same time never share
    bytes, and the arena is never smaller than the largest set of simultaneously live tensors."""
    kat = [(0, 1, 32), (1, 4, 28), (2, 5, 36), (3, 5, 16), (4, 5, 8), (5, 7, 64), (6, 8, 10), (7, 8, 40)]
    total, off = abi.plan_arena(kat)
    assert total == 124
    rng = np.random.default_rng(5)
    for case in range(50):
        n = int(rng.integers(1, 40))
        lives = []
        for _ in range(n):
            a = int(rng.integers(0, 30))
            lives.append((a, a + int(rng.integers(0, 6)), int(rng.integers(1, 5000))))
        align = int(rng.choice([1, 16, 256]))
        total, off = abi.plan_arena(lives, align)
        up = lambda v: (v + align - 1) // align * align
        for i in range(n):
            assert off[i] % align == 0 and off[i] + lives[i][2] <= total
            for j in range(i):
                if max(lives[i][0], lives[j][0]) <= min(lives[i][1], lives[j][1]):
                    assert off[i] + up(lives[i][2]) <= off[j] or off[j] + up(lives[j][2]) <= off[i], (case, i, j)
        peak = max(sum(up(l[2]) for l in lives if l[0] <= op <= l[1]) for op in range(40))
        assert total >= peak
        assert total <= sum(up(l[2]) for l in lives)


def test_arena_planner_rejects_bad_input():
    with pytest.raises(abi.NncvHipError):
        abi.plan_arena([(3, 1, 16)])          # first operator after the last
    with pytest.raises(abi.NncvHipError):
        abi.plan_arena([(0, 1, 16)], align=24)  # alignment not a power of two
    assert abi.plan_arena([]) == (0, [])
