"""Builds libnncv_hip.so (gfx950) from nncv_amd/csrc with hipcc, in-tree.

    python -m nncv_amd.build          # compile what changed, link
    python -m nncv_amd.build --force  # recompile everything
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libnncv_hip.so")
RT_LIB = os.path.join(HERE, "lib", "libnncv_rt.so")
DRIVER = os.path.join(HERE, "lib", "res18_main")

DEVICE_SOURCES = ["igemm.hip", "igemm_fast.hip", "conv3x3_patch.hip", "conv3x3_f16.hip", "conv_pairs.hip", "stem_pool.hip", "gemm_nn.hip", "winograd.hip", "pool_layout.hip", "elementwise.hip", "noalloc.hip", "stream_probe.hip"]
HOST_SOURCES = ["model.cpp", "capi.cpp", "datatype.cpp", "profiler.cpp", "arena_plan.cpp", "graph.cpp", "hostcopy.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-Wall", "-Wno-unused-function"]
# packed-fp32 instruction selection is switched off for all device code
# the first kernel arguments (up to 14 dwords of scalars/pointers) arrive preloaded in SGPRs
# instead of through a scalar load at the top of every wave
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    newest = max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h")))
    newest = max(newest, os.path.getmtime(src), os.path.getmtime(os.path.join(ROOT, "include", "nncv_hip.h")),
                 os.path.getmtime(os.path.join(ROOT, "include", "libnncv", "DataType.hpp")))
    return os.path.getmtime(obj) < newest


def _compile(name, force):
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ, name + ".o")
    if not force and not _stale(src, obj):
        return obj
    cmd = [HIPCC] + COMMON + DEVICE + ["-x", "hip", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (name, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    names = DEVICE_SOURCES + HOST_SOURCES
    with ThreadPoolExecutor(max_workers=min(8, len(names))) as ex:
        objs = list(ex.map(lambda n: _compile(n, force), names))
    subprocess.check_call([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs)
    # host-only runtime library (model.bin reader/writer), the counterpart of the reference's nncv_rt
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-I" + os.path.join(ROOT, "include"),
                           "-o", RT_LIB, os.path.join(CSRC, "datatype.cpp")])
    # the example driver (the flow of the reference's examples/Res18/main.cpp): the C++ caller of the C ABI
    subprocess.check_call(["g++", "-O2", "-std=c++17", os.path.join(ROOT, "examples", "res18_main.cpp"),
                           "-I" + os.path.join(ROOT, "include"), "-L" + os.path.dirname(LIB), "-lnncv_hip",
                           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath-link,/opt/rocm/lib", "-o", DRIVER])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
