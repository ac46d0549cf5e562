"""Host-side checks of the 3x3 LDS-patch kernel's tile planner (no GPU needed: the planner is host arithmetic).

A plan that asks for more LDS cells than the instance owns, more patch pixels than its loader walks, or more pixel slots
than its waves hold would make the kernel write outside its LDS allocation, so the invariants are checked here for many
shapes, together with the plans the ResNet-18 layers are measured on."""
import ctypes

import numpy as np
import pytest

from nncv_amd import abi


@pytest.fixture(scope="module")
def plan():
    L = ctypes.CDLL(abi.LIB_PATH)
    L.nncv_hip_conv3x3_patch_plan.argtypes = [ctypes.c_int] * 6 + [ctypes.POINTER(ctypes.c_int)]
    L.nncv_hip_conv3x3_patch_plan.restype = ctypes.c_int

    def call(stride, N, OH, OW, F, slabs):
        out = (ctypes.c_int * 8)()
        if L.nncv_hip_conv3x3_patch_plan(stride, N, OH, OW, F, slabs, out) != 0:
            return None
        return dict(zip(("WS", "TN", "TH", "TW", "NTX", "lg", "cap", "cover"), out))
    return call


def check(p, stride, N, OH, OW, slabs):
    slots = 64 * p["WS"]
    assert p["WS"] in (1, 2, 4) and min(p["TN"], p["TH"], p["TW"], p["NTX"]) >= 1
    assert p["TN"] * p["TH"] * p["TW"] <= slots                      # every output pixel of a tile has an MFMA slot
    assert p["NTX"] * p["TW"] >= OW and p["TN"] <= N and p["TH"] <= OH
    assert p["NTX"] == 1 or p["TN"] == 1                             # column tiles never span images
    cols = p["TW"] + 2 if stride == 1 else 2 * p["TW"] + 1             # patch columns the loader walks
    cells = p["TW"] + 2 if stride == 1 else 2 * (p["TW"] + 1)          # LDS cells per patch row
    rows = p["TN"] * (p["TH"] + 2 if stride == 1 else 2 * p["TH"] + 1)
    assert cols <= (1 << p["lg"]) <= 64
    assert rows * cells <= p["cap"]                                  # the patch fits the instance's LDS
    assert (rows << p["lg"]) <= p["cover"]                           # ... and the loader's passes reach all of it
    # the widest instances keep no prefetch registers in the tap loop: single-slab layers only
    if stride == 1:
        assert p["WS"] != 4 or slabs == 1
    else:
        assert p["WS"] != 4 and (p["WS"] != 2 or slabs == 1)
    assert p["cap"] * 144 + 256 * 16 <= 80 * 1024                    # two workgroups per CU


def test_invariants_on_random_shapes(plan):
    rng = np.random.default_rng(20251125)
    found = 0
    for _ in range(20000):
        stride = int(rng.choice([1, 2]))
        N = int(rng.choice([1, 1, 2, 3, 4, 8, 16, 32, 64, 256]))
        OH, OW = int(rng.integers(1, 260)), int(rng.integers(1, 260))
        F = 8 * int(rng.integers(1, 129))
        slabs = int(rng.choice([1, 1, 2, 3, 4, 8, 16]))
        p = plan(stride, N, OH, OW, F, slabs)
        if p is None:
            continue
        found += 1
        check(p, stride, N, OH, OW, slabs)
    assert found > 19000  # rows of any width are cut into column tiles: nearly every shape has a plan


def test_edges(plan):
    for stride in (1, 2):
        for shape in [(1, 1, 1), (1, 1, 4096), (1, 4096, 1), (1, 62, 62), (1, 63, 63), (1, 64, 64), (7, 31, 31), (7, 32, 32),
                      (65535, 7, 7), (3, 2, 1000)]:
            for slabs in (1, 2, 16):
                p = plan(stride, shape[0], shape[1], shape[2], 64, slabs)
                assert p is not None, (stride, shape, slabs)
                check(p, stride, shape[0], shape[1], shape[2], slabs)
    assert plan(3, 1, 8, 8, 64, 1) is None and plan(1, 0, 8, 8, 64, 1) is None and plan(1, 1, 8, 8, 64, 0) is None


@pytest.mark.parametrize("args,want", [
    # ResNet-18 at batch 32, 224x224 (the bench workload): stride-1 layers of layer1..4, then the three stride-2 ones
    ((1, 32, 56, 56, 64, 1), dict(WS=4, TN=1, TH=4, TW=56, NTX=1)),
    ((1, 32, 28, 28, 128, 2), dict(WS=2, TN=1, TH=4, TW=28, NTX=1)),
    ((1, 32, 14, 14, 256, 4), dict(WS=2, TN=1, TH=7, TW=14, NTX=1)),
    ((1, 32, 7, 7, 512, 8), dict(WS=1, TN=1, TH=7, TW=7, NTX=1)),
    ((2, 32, 28, 28, 128, 1), dict(WS=2, TN=1, TH=4, TW=28, NTX=1)),
    ((2, 32, 14, 14, 256, 2), dict(WS=1, TN=1, TH=4, TW=14, NTX=1)),
    ((2, 32, 7, 7, 512, 4), dict(WS=1, TN=1, TH=7, TW=7, NTX=1)),
    # rows that are cut: 64 columns -> four tiles of 16 x 4 rows; 40 columns -> two tiles of 20 x 6 rows
    ((1, 1, 64, 64, 64, 2), dict(WS=1, TH=4, TW=16, NTX=4)),
    ((1, 16, 40, 40, 128, 2), dict(WS=2, TH=6, TW=20, NTX=2)),
])
def test_plans_the_measurements_were_taken_on(plan, args, want):
    p = plan(*args)
    assert p is not None
    assert {k: p[k] for k in want} == want, p
