"""Host-side checks of the fp16 3x3 stream kernel's launch planner (host arithmetic, no GPU needed).

A plan whose patch needs more row segments than a buffer holds, more pixel slots than the waves own, or whose
reciprocal divisions leave their exact range would make the kernel write outside its LDS allocation or address the
wrong pixels, so the invariants are checked here for many shapes, together with the plans of the ResNet-18 layers."""
import ctypes

import numpy as np
import pytest

from nncv_amd import abi

KEYS = ("TH", "S", "top", "aligned", "tiles", "NSEG", "PG", "WF", "WK", "FB", "Wpf", "segcap", "rowx", "patch_bytes")


@pytest.fixture(scope="module")
def plan():
    L = ctypes.CDLL(abi.LIB_PATH)
    L.nncv_hip_conv3x3_stream_plan.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_int)]
    L.nncv_hip_conv3x3_stream_plan.restype = ctypes.c_int

    def call(N, H, W, C, F):
        out = (ctypes.c_int * 14)()
        if L.nncv_hip_conv3x3_stream_plan(N, H, W, C, F, out) != 0:
            return None
        return dict(zip(KEYS, out))
    return call


def check(p, N, H, W, C, F):
    slots = 128 * p["PG"]
    assert p["PG"] in (1, 2) and p["WF"] * p["WK"] == 4 and p["segcap"] == 36 * p["PG"]
    assert F % (32 * p["WF"]) == 0 and p["FB"] * 32 * p["WF"] == F
    assert 1 <= p["TH"] and p["TH"] * W <= slots                         # every pixel of a tile has an MFMA slot
    assert p["NSEG"] * 7 >= W + 2                                        # a patch row holds the row and its two halo cells
    assert (p["TH"] + 2) * p["NSEG"] <= p["segcap"]                      # the patch fits one LDS buffer
    assert 2 * p["patch_bytes"] + 2 * 32 * p["WF"] * 4 <= (80 if p["PG"] == 1 else 160) * 1024  # two workgroups per CU (one of eight waves)
    # rows of the patch in LDS: NSEG segments of 1008 bytes and `rowx` spare bytes.  Every segment a wave may load (also
    # the ones below the patch, which load zeros) and the 16 bytes its last lane writes stay inside the buffer
    assert p["rowx"] % 16 == 0 and 0 <= p["rowx"] <= 256
    last = p["segcap"] - 1
    assert last * 1008 + (last // p["NSEG"]) * p["rowx"] + 1008 + 16 <= p["patch_bytes"]
    if p["rowx"]:
        # the pitch continues the bank sequence of a row: the slot after a row's last pixel is the next row's first
        assert ((p["NSEG"] * 1008 + p["rowx"]) // 16 - 9 * W) % 16 == 0
        slots_cells = []
        for s in range(slots):
            e = s
            if e >= p["TH"] * W:
                e = max(0, e - (((e - p["TH"] * W) >> 4) + 1) * 16)
            slots_cells.append(((e // W) * (p["NSEG"] * 1008 + p["rowx"]) + (e % W) * 144) // 16)
        if p["TH"] * W >= 16:
            for g0 in range(0, slots, 16):
                assert len({u % 16 for u in slots_cells[g0:g0 + 16]}) == 16, (N, H, W, g0)  # no two of 16 lanes share a bank group
    assert 2 <= p["S"] <= 255
    if p["aligned"]:
        assert p["top"] == 0 and p["S"] % p["TH"] == 0 and p["S"] >= H   # a whole number of tiles per image
        assert p["tiles"] == N * (p["S"] // p["TH"])
    else:
        assert p["top"] == 1 and p["S"] == H + 1                         # one shared zero row between images
        rows = N * (H + 1) - 1
        assert (p["tiles"] - 1) * p["TH"] < rows <= p["tiles"] * p["TH"]  # the tiles cover virtual rows 1 .. rows
    assert (N * p["S"] + p["TH"] + 2) * p["S"] < 2 ** 31                 # the reciprocal multiplications stay exact
    assert 1 <= p["Wpf"] <= p["tiles"] and p["Wpf"] < 65536
    # every tile is walked: a workgroup starts at tile i < Wpf and steps by Wpf
    assert (p["tiles"] + p["Wpf"] - 1) // p["Wpf"] >= 1


def test_invariants_on_random_shapes(plan):
    rng = np.random.default_rng(20251126)
    found = 0
    for _ in range(20000):
        N = int(rng.choice([1, 1, 2, 3, 4, 5, 8, 16, 32, 64, 256, 1000]))
        H, W = int(rng.integers(1, 200)), int(rng.integers(1, 200))
        C = 64 * int(rng.integers(1, 9))
        F = 32 * int(rng.integers(1, 17))
        p = plan(N, H, W, C, F)
        if p is None:
            # only what cannot fit is refused: a row wider than the slots or the buffer, more rows than the 8-bit fields
            # hold, one-row images (a single virtual row per image has no reciprocal), dividends beyond the exact range
            assert W > 128 or H > 254 or H == 1 or 3 * ((W + 2 + 6) // 7) > 36 or (N * (H + 1) + 200) * (H + 1) >= 2 ** 31, (N, H, W, C, F)
            continue
        found += 1
        check(p, N, H, W, C, F)
    assert found > 5000


@pytest.mark.parametrize("N,H,W,C,F,expect", [
    (32, 56, 56, 64, 64, dict(TH=2, aligned=1, tiles=896, WF=2, WK=2, Wpf=448)),      # layer1: 896 tiles, two per workgroup
    (32, 28, 28, 128, 128, dict(TH=4, aligned=1, tiles=224, WF=2, WK=2, FB=2)),       # layer2, the roofline kernel's shape
    (32, 14, 14, 256, 256, dict(TH=9, aligned=0, S=15, WF=2, FB=4)),                  # layer3: images one zero row apart
    (64, 28, 28, 128, 128, dict(TH=4, tiles=448, WF=4, WK=1, FB=1)),                  # batch 64: 128 filters per workgroup, no K groups
    (64, 14, 14, 256, 256, dict(TH=9, aligned=0, WF=4, WK=1, FB=2, Wpf=107)),         # four slabs per tile: 128 filters from 160 workgroups
    (1, 28, 28, 128, 128, dict(WF=1, WK=4)),                                          # batch 1: 32-filter blocks fill more CUs
])
def test_resnet18_plans(plan, N, H, W, C, F, expect):
    p = plan(N, H, W, C, F)
    assert p is not None
    check(p, N, H, W, C, F)
    for k, v in expect.items():
        assert p[k] == v, (k, p)


def test_invariants_hold_under_the_overlap_hint(plan):
    """nncv_hip_set_overlap_hint(4) makes the planner take the 128-filter form wherever the filter count allows it: the
    same invariants must hold for those plans, and the hint must not leak into later tests."""
    L = ctypes.CDLL(abi.LIB_PATH)
    L.nncv_hip_set_overlap_hint.argtypes = [ctypes.c_int]
    assert L.nncv_hip_set_overlap_hint(4) == 0
    try:
        rng = np.random.default_rng(20251127)
        wide = 0
        for _ in range(8000):
            N = int(rng.choice([1, 2, 3, 8, 16, 32, 64]))
            H, W = int(rng.integers(2, 130)), int(rng.integers(1, 129))
            C = 64 * int(rng.integers(1, 5))
            F = 32 * int(rng.integers(1, 13))
            p = plan(N, H, W, C, F)
            if p is None:
                continue
            check(p, N, H, W, C, F)
            if F % 128 == 0:
                assert (p["WF"], p["WK"]) == (4, 1), (N, H, W, C, F, p)
                wide += 1
        assert wide > 500
        p = plan(32, 14, 14, 256, 256)
        assert p["WF"] == 4 and p["FB"] == 2 and p["FB"] * p["Wpf"] == 108
    finally:
        assert L.nncv_hip_set_overlap_hint(1) == 0
    assert plan(32, 14, 14, 256, 256)["WF"] == 2


def _loader_offsets(p, N, H, W, C):
    """The byte offsets the kernel's patch loader forms (conv3x3_f16.hip, patch_tile / patch_piece_load), in the
    kernel's own 32-bit arithmetic: for every tile, the pass behind the last tile, every wave, piece, lane and slab."""
    M, OOB = 0xFFFFFFFF, 0x80000000
    TH, S, top, NSEG = p["TH"], p["S"], p["top"], p["NSEG"]
    mS32 = (M // S + 1) & M
    rnseg = 65535 // NSEG + 1 if NSEG > 1 else 0
    pixB = C * 2
    out = []
    for wave in range(4 * p["PG"]):
        cells = []  # (crow, ccol) of the cell each lane works out
        for lane in range(64):
            cseg = wave * 9 + ((lane * 37) >> 8)
            crow = cseg if NSEG == 1 else (cseg * rnseg) >> 16
            ccol = ((cseg - crow * NSEG) * 7 + (lane - ((lane * 37) >> 8) * 7) - 1) & M
            cells.append((crow, ccol))
        for t in list(range(p["tiles"])) + [None]:
            live = t is not None
            tt = t if live else p["tiles"] + 3
            v0 = (top + tt * TH) & M
            nt = (v0 * mS32) >> 32
            celloff = []
            for crow, ccol in cells:
                vS = (v0 - 1 + crow + S) & M
                nS = (vS * mS32) >> 32
                n = (nS - 1) & M
                y = (vS - nS * S - top) & M
                bad = y >= H or n >= N or ccol >= W or crow >= TH + 2 or (p["aligned"] == 1 and n != nt) or not live
                celloff.append(OOB if bad else (((n * H + y) * W + ccol) * pixB) & M)
            for pp in range(9):
                for lane in range(64):
                    lcell = (lane * 57) >> 9
                    lch = lane - 9 * lcell
                    lchoff = OOB if lch == 8 else lch * 16
                    vo = celloff[lcell + 7 * pp]
                    for slab in range(C // 64):
                        out.append((vo + lchoff + slab * 128) & M)
    return np.array(out, dtype=np.int64)


@pytest.mark.parametrize("shape", [(8, 28, 28, 128, 128), (16, 14, 14, 256, 256), (4, 56, 56, 64, 64), (3, 7, 7, 512, 512),
                                   (5, 20, 24, 64, 96), (2, 9, 100, 128, 32)])
def test_loader_offsets_are_out_of_range_or_inside_the_tensor(plan, shape):
    """The kernel addresses its input through a descriptor of 2^31 bytes (the tensor's size is not among the
    arguments that arrive preloaded), so the range check stops nothing below 2^31: every offset the loader forms must
    either carry the out-of-range flag or lie inside the tensor -- also for cells that do not exist, for the pad lane
    of such a cell (two flags that cancel) and for the pass behind the last tile."""
    N, H, W, C, F = shape
    p = plan(N, H, W, C, F)
    if p is None:
        pytest.skip("no stream plan for this shape")
    off = _loader_offsets(p, N, H, W, C)
    in_bytes = N * H * W * C * 2
    inside = off + 16 <= in_bytes
    flagged = off >= 0x80000000
    assert (inside | flagged).all(), (shape, [hex(int(v)) for v in off[~(inside | flagged)][:4]])
    assert inside.any() and flagged.any()
