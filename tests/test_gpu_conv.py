"""GPU parity of the convolution paths against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import oracle
from nncv_amd import abi, synth
from gpu_util import (Conv, dev, host, nhwc, nchw, max_rel, rel_l2, FP32_MAX_REL, FP16_REL_L2)

pytestmark = pytest.mark.gpu


def oracle_layer(x, w, stride, pad, bn=None, residual=None, relu=False):
    y = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, pad), w, stride=stride)
    if bn is not None:
        y = oracle.batchnorm(y, *bn)
    if residual is not None:
        y = y + residual
    if relu:
        y = oracle.relu(y)
    return y


def bn_params(seed, F):
    return (synth.uniform(seed, (F,), 0.5, 1.5), synth.normal(seed + 1, (F,), 0.1),
            synth.normal(seed + 2, (F,), 0.1), synth.uniform(seed + 3, (F,), 0.5, 1.5))


CASES = [  # N, C, F, H, W, R, stride, pad
    (2, 64, 64, 14, 14, 3, 1, 1),
    (1, 64, 128, 28, 28, 3, 2, 1),
    (3, 64, 128, 14, 14, 1, 2, 0),
    (2, 128, 64, 9, 13, 3, 1, 1),     # ragged: odd, non-square
    (1, 32, 200, 7, 7, 3, 1, 1),      # F not a multiple of the tile
    (5, 16, 8, 6, 5, 3, 2, 1),        # tiny
    # shapes that exercise the LDS-patch 3x3 kernel's wave arrangements and tile planner
    (4, 64, 64, 56, 56, 3, 1, 1),     # 4x2 waves, TH=4 row tiles, one channel slab
    (3, 128, 128, 28, 28, 3, 1, 1),   # 4x2 waves, TH=7, two slabs, two filter blocks
    (5, 256, 64, 14, 14, 3, 1, 1),    # few workgroups -> 2x4 waves, four slabs
    (9, 64, 128, 7, 7, 3, 1, 1),      # several images per tile, last tile short of images
    (2, 64, 72, 30, 62, 3, 1, 1),     # widest row the patch loader takes, F not a multiple of 64
    (1, 64, 64, 20, 64, 3, 1, 1),     # one row is wider than the patch loader takes: two column tiles of 32
    (2, 64, 72, 11, 150, 3, 1, 1),    # three column tiles of 50, the halo columns come from the neighbouring tiles
    (1, 128, 64, 40, 125, 3, 1, 1),   # column tiles of 42 + 42 + 41, two slabs
    (2, 64, 64, 23, 17, 3, 1, 1),     # ragged: H not a multiple of the row tile
    # stride 2 through the LDS-patch kernel (even / odd columns of the patch kept apart)
    (4, 64, 128, 56, 56, 3, 2, 1),    # 2x2 waves, TH=4, one slab
    (3, 128, 256, 28, 28, 3, 2, 1),   # 1x4 waves, TH=4, two slabs, last row tile short
    (5, 256, 64, 14, 14, 3, 2, 1),    # whole image per tile, four slabs
    (9, 64, 72, 7, 7, 3, 2, 1),       # several images per tile, F not a multiple of 64
    (2, 64, 64, 23, 17, 3, 2, 1),     # odd sizes: the last input row / column is read by the last output only
    (2, 128, 64, 30, 62, 3, 2, 1),    # widest row the loader takes at stride 2
    (1, 64, 64, 9, 63, 3, 2, 1),      # 32 output columns: two column tiles of 16
    (2, 128, 64, 33, 99, 3, 2, 1),    # stride 2, odd width: 50 output columns in two tiles of 25
]


@pytest.mark.parametrize("N,C,F,H,W,R,stride,pad", CASES)
@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
@pytest.mark.parametrize("algo", [abi.ALGO_IGEMM, abi.ALGO_WINOGRAD])
def test_conv_bn_relu_residual_nhwc(N, C, F, H, W, R, stride, pad, dt, algo):
    if algo == abi.ALGO_WINOGRAD and not (R == 3 and stride == 1):
        pytest.skip("Winograd F(4,3) covers 3x3 stride-1 only")
    print("case", N, C, F, H, W, R, stride, pad, dt, algo, flush=True)
    x = synth.normal(100, (N, C, H, W))
    w = synth.normal(101, (F, C, R, R), std=float(np.sqrt(2.0 / (C * R * R))))
    bn = bn_params(102, F)
    OH, OW = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - R) // stride + 1
    res = synth.normal(106, (N, F, OH, OW))
    if dt == abi.F16:
        x, w, res = synth.round_fp16(x), synth.round_fp16(w), synth.round_fp16(res)
        bn = tuple(synth.round_fp16(b) for b in bn)
    want = oracle_layer(x, w, stride, pad, bn, res, relu=True)
    layer = Conv(dt, w, stride, pad, bn=bn, relu=True, algo=algo)
    # a request for fp16 Winograd is served by the direct form (F(4,3) in half misses the fp16 bar)
    assert layer.algo == (abi.ALGO_IGEMM if (dt == abi.F16 and algo == abi.ALGO_WINOGRAD) else algo)
    got = nchw(host(layer(dev(nhwc(x), dt), abi.NHWC, residual=dev(nhwc(res), dt))))
    if dt == abi.F32:
        assert max_rel(got, want) < FP32_MAX_REL
    else:
        assert rel_l2(got, want) < FP16_REL_L2
    assert (got >= 0).all()


@pytest.mark.parametrize("algo", [abi.ALGO_IGEMM, abi.ALGO_WINOGRAD])
def test_conv_nchw_layout_plain(algo):
    """NCHW in/out (the layout of the reference's ABI), no epilogue."""
    x = synth.normal(110, (2, 16, 10, 11))
    w = synth.normal(111, (12, 16, 3, 3), std=0.1)
    want = oracle_layer(x, w, 1, 1)
    layer = Conv(abi.F32, w, 1, 1, algo=algo)
    got = host(layer(dev(x), abi.NCHW))
    assert max_rel(got, want) < FP32_MAX_REL


def test_relu_keeps_nan_and_conv_zero_halo():
    """`ugt` ReLU keeps NaN (Res18.mlir:139-141); the halo contributes exact zeros."""
    x = np.ones((1, 8, 4, 4), np.float32)
    w = np.ones((4, 8, 3, 3), np.float32)
    layer = Conv(abi.F32, w, 1, 1, relu=True, algo=abi.ALGO_IGEMM)
    got = nchw(host(layer(dev(nhwc(x)), abi.NHWC)))
    want = np.array([[32, 48, 48, 32], [48, 72, 72, 48], [48, 72, 72, 48], [32, 48, 48, 32]], np.float32)
    assert np.array_equal(got[0, 0], want)
    x[0, 0, 1, 1] = np.nan
    got = nchw(host(layer(dev(nhwc(x)), abi.NHWC)))
    assert np.isnan(got[0, :, 0:3, 0:3]).all() and not np.isnan(got[0, :, 3, 3]).any()


def test_cfg2_single_conv_winograd_vs_direct():
    """BASELINE config 2: 3x3 s1 p1 fp32, input [1,64,56,56], filter [64,64,3,3]."""
    x, w = synth.cfg2_conv()
    want = oracle_layer(x, w, 1, 1)
    for algo in (abi.ALGO_WINOGRAD, abi.ALGO_IGEMM):
        layer = Conv(abi.F32, w, 1, 1, algo=algo)
        got = nchw(host(layer(dev(nhwc(x)), abi.NHWC)))
        err = max_rel(got, want)
        print("cfg2 algo", algo, "max_rel", err, flush=True)
        assert err < FP32_MAX_REL


def test_conv_time_helper_reports_a_plausible_duration():
    """nncv_hip_conv_time (the roofline timer of bench.py) leaves the same output as one forward
    call and reports a per-launch time in a sane range."""
    import ctypes
    import torch
    x = synth.round_fp16(synth.normal(300, (2, 64, 14, 14)))
    w = synth.round_fp16(synth.normal(301, (64, 64, 3, 3), std=0.05))
    layer = Conv(abi.F16, w, 1, 1, relu=True)
    xd = dev(nhwc(x), abi.F16)
    want = host(layer(xd, abi.NHWC))
    out = torch.zeros((2, 14, 14, 64), dtype=torch.float16, device="cuda")
    avg = ctypes.c_float(0.0)
    abi.check(abi.lib().nncv_hip_conv_time(layer.h, xd.data_ptr(), 2, 14, 14, None, out.data_ptr(), 20, None, ctypes.byref(avg)))
    assert np.array_equal(out.cpu().numpy(), want)
    assert 1.0 < avg.value < 1000.0


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_random_layers(dt):
    """50 seeded random layers per element type: channel counts from one vector to 256, filters not multiples of the
    tiles, 1x1..7x7 windows, stride 1 / 2, with and without padding, BatchNorm, residual and any fused activation,
    odd and oblong images -- whichever kernel the dispatcher picks must agree with the oracle."""
    f16 = dt == abi.F16
    vn = 8 if f16 else 4
    done = 0
    for seed in range(9000, 9050):
        rng = np.random.default_rng(seed)
        C = vn * int(rng.choice([1, 2, 3, 4, 8, 8, 16, 16, 32]))
        F = 4 * int(rng.choice([1, 2, 3, 8, 16, 16, 18, 32, 50]))
        if f16:
            F = (F + 7) // 8 * 8
        R = int(rng.choice([1, 3, 3, 3, 5, 7]))
        stride = int(rng.choice([1, 1, 2]))
        pad = int(rng.choice([0, (R - 1) // 2, (R - 1) // 2]))
        H, W, N = int(rng.integers(R, 40)), int(rng.integers(R, 70)), int(rng.integers(1, 6))
        OH, OW = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - R) // stride + 1
        act = int(rng.choice([abi.ACT_NONE, abi.ACT_RELU, abi.ACT_RELU, abi.ACT_HARDSWISH, abi.ACT_SILU]))
        use_bn, use_res = rng.random() < 0.7, rng.random() < 0.4
        wino = R == 3 and stride == 1 and act <= abi.ACT_RELU and rng.random() < 0.25
        x = synth.normal(seed, (N, C, H, W))
        w = synth.normal(seed + 1, (F, C, R, R), std=float(np.sqrt(2.0 / (C * R * R))))
        bn = bn_params(seed + 2, F) if use_bn else None
        res = synth.normal(seed + 6, (N, F, OH, OW)) if use_res else None
        if f16:
            x, w = synth.round_fp16(x), synth.round_fp16(w)
            bn = tuple(synth.round_fp16(b) for b in bn) if bn else None
            res = synth.round_fp16(res) if res is not None else None
        print("seed", seed, (N, C, F, H, W, R, stride, pad), "act", act, "bn", use_bn, "res", use_res, "winograd", wino, flush=True)
        y = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, pad) if pad else x, w, stride)
        if bn:
            y = oracle.batchnorm(y, *bn)
        if res is not None:
            y = (y + res).astype(np.float32)
        want = oracle.ACTIVATIONS[act](y)
        conv = Conv(dt, w, stride, pad, bn=bn, relu=act, algo=abi.ALGO_WINOGRAD if wino else abi.ALGO_IGEMM)
        rd = dev(nhwc(res), dt) if res is not None else None
        got = nchw(host(conv(dev(nhwc(x), dt), abi.NHWC, residual=rd)))
        conv.close()
        if f16:
            assert rel_l2(got, want) < FP16_REL_L2, seed
        else:
            assert max_rel(got, want) < FP32_MAX_REL, seed
        done += 1
    assert done == 50


def test_fp32_k_split_over_workgroups_is_exact_and_repeatable():
    """A deep fp32 3x3 layer at batch 1 has too few workgroups for the chip, so the patch kernel splits its K walk over
    several per output tile; the last one to arrive adds the partial tiles in slab order.  Whichever arrives last, the bits
    must be the same on every launch (the tickets return to zero each time), and they must match the oracle."""
    N, C, F, H = 1, 512, 512, 7
    x = synth.normal(7100, (N, C, H, H))
    w = synth.normal(7101, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9))))
    bn = bn_params(7102, F)
    res = synth.normal(7106, (N, F, H, H))
    want = oracle_layer(x, w, 1, 1, bn, res, relu=True)
    layer = Conv(abi.F32, w, 1, 1, bn=bn, relu=True, algo=abi.ALGO_IGEMM)
    xd, rd = dev(nhwc(x), abi.F32), dev(nhwc(res), abi.F32)
    abi.profile_enable(True)
    try:
        abi.profile_report()
        first = host(layer(xd, abi.NHWC, residual=rd))
        tags = list(abi.profile_report())
    finally:
        abi.profile_enable(False)
    print("tags", tags, flush=True)
    assert any("splitk" in t for t in tags)
    assert max_rel(nchw(first), want) < FP32_MAX_REL
    for _ in range(20):
        again = host(layer(xd, abi.NHWC, residual=rd))
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
    # a stride-2 layer with several slabs takes the same path
    w2 = synth.normal(7111, (F, 256, 3, 3), std=float(np.sqrt(2.0 / (256 * 9))))
    x2 = synth.normal(7110, (2, 256, 14, 14))
    l2 = Conv(abi.F32, w2, 2, 1, bn=bn, relu=False, algo=abi.ALGO_IGEMM)
    got2 = nchw(host(l2(dev(nhwc(x2), abi.F32), abi.NHWC)))
    assert max_rel(got2, oracle_layer(x2, w2, 2, 1, bn, None, relu=False)) < FP32_MAX_REL
    layer.close()
    l2.close()


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_random_patch_kernel_layers(dt):
    """40 seeded random 3x3 pad-1 layers per element type inside the LDS-patch kernel's domain (whole channel slabs):
    stride 1 and 2, rows from 3 to 200 pixels wide (column tiles), batches that need several images per tile or the
    half-block / K-split forms, filters that are not multiples of 64, and (fp16) every fused activation with the residual
    before or after it.  Most of them must really have taken that kernel."""
    f16 = dt == abi.F16
    slab = 64 if f16 else 32
    routes = {}
    abi.profile_enable(True)
    try:
        abi.profile_report()
        for seed in range(9500, 9540):
            rng = np.random.default_rng(seed)
            C = slab * int(rng.choice([1, 1, 2, 2, 3, 4]))
            F = 8 * int(rng.choice([1, 4, 8, 8, 9, 16, 17, 32]))
            stride = int(rng.choice([1, 2, 2]))
            H, W = int(rng.integers(3, 48)), int(rng.integers(3, 200))
            N = int(rng.integers(1, 10))
            if N * H * W * C > 3e6:
                N = 1
            OH, OW = (H - 1) // stride + 1, (W - 1) // stride + 1
            acts = [abi.ACT_NONE, abi.ACT_RELU, abi.ACT_RELU] + ([abi.ACT_SILU, abi.ACT_HARDSWISH] if f16 else [])
            act = int(rng.choice(acts))
            use_bn, use_res = rng.random() < 0.7, rng.random() < 0.4
            x = synth.normal(seed, (N, C, H, W))
            w = synth.normal(seed + 1, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9))))
            bn = bn_params(seed + 2, F) if use_bn else None
            res = synth.normal(seed + 6, (N, F, OH, OW)) if use_res else None
            if f16:
                x, w = synth.round_fp16(x), synth.round_fp16(w)
                bn = tuple(synth.round_fp16(b) for b in bn) if bn else None
                res = synth.round_fp16(res) if res is not None else None
            print("seed", seed, (N, C, F, H, W, stride), "act", act, "bn", use_bn, "res", use_res, flush=True)
            y = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, 1), w, stride)
            if bn:
                y = oracle.batchnorm(y, *bn)
            if res is not None:
                y = (y + res).astype(np.float32)
            want = oracle.ACTIVATIONS[act](y)
            conv = Conv(dt, w, stride, 1, bn=bn, relu=act, algo=abi.ALGO_IGEMM)
            rd = dev(nhwc(res), dt) if res is not None else None
            got = nchw(host(conv(dev(nhwc(x), dt), abi.NHWC, residual=rd)))
            conv.close()
            for k, v in abi.profile_report().items():
                if "conv" in k or "igemm" in k:
                    routes[k] = routes.get(k, 0) + v["launches"]
            if f16:
                assert rel_l2(got, want) < FP16_REL_L2, seed
            else:
                assert max_rel(got, want) < FP32_MAX_REL, seed
    finally:
        abi.profile_enable(False)
    print("routes", routes, flush=True)
    patch = sum(v for k, v in routes.items() if k.startswith("conv3x3"))
    assert patch >= 0.8 * sum(routes.values()), routes


@pytest.mark.parametrize("C,F,N,H,W,act,res", [
    (16, 72, 2, 56, 56, abi.ACT_RELU, False),       # MobileNetV3 expansion: one K step, two 64-filter blocks
    (16, 16, 3, 9, 7, abi.ACT_NONE, True),          # projection with the block's residual, ragged pixel count
    (24, 88, 2, 28, 28, abi.ACT_RELU, False),       # 3 chunks: the second step's upper half is padding
    (40, 240, 1, 14, 14, abi.ACT_HARDSWISH, False),
    (48, 288, 2, 14, 14, abi.ACT_HARDSWISH, False),
    (72, 24, 2, 28, 28, abi.ACT_NONE, False),
    (88, 24, 2, 28, 28, abi.ACT_NONE, True),
    (120, 48, 2, 14, 14, abi.ACT_NONE, False),
    (144, 48, 3, 14, 14, abi.ACT_SILU, True),       # 18 chunks, activation before ... the residual is added first here
    (136, 40, 1, 5, 5, abi.ACT_RELU, True),         # 17 chunks: odd, the last step is half padding
])
def test_fp16_1x1_convolutions_with_a_short_k_axis(C, F, N, H, W, act, res):
    """1x1 layers whose channel count is a multiple of 8 but not of 32, up to 144: the kernel that holds the whole
    K axis in registers (`conv1x1_shortk`), against the oracle, with the route checked."""
    x = synth.round_fp16(synth.normal(7600 + C, (N, C, H, W)))
    w = synth.round_fp16(synth.normal(7601 + C, (F, C, 1, 1), std=float(np.sqrt(2.0 / C))))
    bn = tuple(synth.round_fp16(b) for b in bn_params(7602 + C, F))
    r = synth.round_fp16(synth.normal(7606 + C, (N, F, H, W))) if res else None
    y = oracle.batchnorm(oracle.conv2d_nchw_fchw(x, w, 1), *bn)
    if r is not None:
        y = (y + r).astype(np.float32)
    want = oracle.ACTIVATIONS[act](y)
    conv = Conv(abi.F16, w, 1, 0, bn=bn, relu=act, algo=abi.ALGO_IGEMM)
    rd = dev(nhwc(r), abi.F16) if r is not None else None
    print("1x1 short K", (C, F, N, H, W), act, res, flush=True)
    abi.profile_enable(True)
    abi.profile_report()
    got = nchw(host(conv(dev(nhwc(x), abi.F16), abi.NHWC, residual=rd)))
    tags = abi.profile_report()
    abi.profile_enable(False)
    conv.close()
    assert any(t.startswith("conv1x1_shortk<f16") for t in tags), sorted(tags)
    assert rel_l2(got, want) < 2e-3
    assert np.abs(got - want).max() < 2e-2 * max(1.0, np.abs(want).max())
