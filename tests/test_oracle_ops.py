"""Pins the CPU oracle (oracle/nncv_oracle.c) before anything is compared against it.

Each check is chosen so that a plausible mistake (dropped term, swapped index, wrong sign,
transposed operand) fails: an independent library routine (torch CPU functional ops), brute
force in numpy on tiny shapes, the closed-form fixtures the reference's own tests hold, and
algebraic identities.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from nncv_amd import synth


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def test_conv_brute_force_tiny():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, 7, 6)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 2)).astype(np.float32)
    init = rng.standard_normal((2, 4, 3, 3)).astype(np.float32)
    # stride 2 in both dims: OH = (7-3)//2+1 = 3, OW = (6-2)//2+1 = 3
    want = init.astype(np.float64).copy()
    for n in range(2):
        for f in range(4):
            for y in range(3):
                for xx in range(3):
                    for c in range(3):
                        for r in range(3):
                            for s in range(2):
                                want[n, f, y, xx] += float(x[n, c, 2 * y + r, 2 * xx + s]) * float(w[f, c, r, s])
    got = oracle.conv2d_nchw_fchw(x, w, stride=2, out=init)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("C,Fo,H,R,stride,pad", [
    (3, 8, 20, 7, 2, 3), (8, 8, 9, 3, 1, 1), (8, 16, 10, 3, 2, 1), (8, 16, 10, 1, 2, 0)])
def test_conv_vs_torch(C, Fo, H, R, stride, pad):
    x = synth.normal(11, (2, C, H, H + 1))
    w = synth.normal(12, (Fo, C, R, R), std=0.2)
    want = F.conv2d(t(x).double(), t(w).double(), stride=stride, padding=pad).numpy()
    got = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, pad), w, stride=stride)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6)


def test_split_params_fixture_closed_form():
    """tests/SplitParams/getParams.py: ones(1,3,224,224) -> conv1 picks 3 ones, conv2 a
    5-diagonal: every output equals 15.0, shape [1,1,218,218]."""
    w1 = np.zeros((1, 3, 3, 3), np.float32)
    w1[0, 0, 0, 0] = w1[0, 1, 1, 1] = w1[0, 2, 2, 2] = 1
    w2 = np.zeros((1, 1, 5, 5), np.float32)
    for i in range(5):
        w2[0, 0, i, i] = 1
    y = oracle.conv2d_nchw_fchw(oracle.conv2d_nchw_fchw(np.ones((1, 3, 224, 224), np.float32), w1), w2)
    assert y.shape == (1, 1, 218, 218)
    assert np.all(y == 15.0)


def test_winograd_ir_fixture_closed_form():
    """tests/ConvOptimization/conv2dNchwWinograd.mlir: NHWC 1x16x16x4 with filter dense<0.1>
    3x3x4x16: out = init + 0.1 * (sum over the 3x3x4 window), 14x14x16."""
    x = synth.normal(21, (1, 4, 16, 16))
    init = synth.normal(22, (1, 16, 14, 14))
    w = np.full((16, 4, 3, 3), 0.1, np.float32)
    got = oracle.conv2d_nchw_fchw(x, w, out=init)
    win = np.lib.stride_tricks.sliding_window_view(x.astype(np.float64), (3, 3), axis=(2, 3)).sum(axis=(1, 4, 5))
    want = init + np.float64(np.float32(0.1)) * win[:, None]
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    # and the Winograd route gives the same numbers (pad 0 form of the fixture)
    got_w = oracle.conv3x3_winograd43(x, w, pad=0) + init
    np.testing.assert_allclose(got_w, want, rtol=1e-5, atol=1e-5)


def test_matmul_accumulates():
    a = synth.uniform(31, (33, 17), -1, 1)
    b = synth.uniform(32, (17, 29), -1, 1)
    c = synth.uniform(33, (33, 29), -1, 1)
    want = c.astype(np.float64) + a.astype(np.float64) @ b.astype(np.float64)
    np.testing.assert_allclose(oracle.matmul(a, b, c), want, rtol=1e-6, atol=1e-6)


def test_batchnorm_formula_and_operand_order():
    x = synth.normal(41, (2, 5, 3, 4))
    g, b = synth.uniform(42, (5,), 0.5, 1.5), synth.normal(43, (5,), 0.1)
    m, v = synth.normal(44, (5,), 0.1), synth.uniform(45, (5,), 0.5, 1.5)
    want = F.batch_norm(t(x).double(), t(m).double(), t(v).double(), t(g).double(), t(b).double(),
                        training=False, eps=float(np.float32(1e-5))).numpy()
    np.testing.assert_allclose(oracle.batchnorm(x, g, b, m, v), want, rtol=1e-5, atol=1e-6)
    # exact fp32 op order of Res18.mlir:128-135
    r = np.float32(1.0) / np.sqrt(v + np.float32(1e-5), dtype=np.float32)
    exact = ((x - m[None, :, None, None]) * r[None, :, None, None]) * g[None, :, None, None] + b[None, :, None, None]
    assert np.array_equal(oracle.batchnorm(x, g, b, m, v), exact.astype(np.float32))


def test_relu_ugt_semantics():
    x = np.array([-1.0, -0.0, 0.0, 2.5, np.nan, -np.inf, np.inf], np.float32)
    y = oracle.relu(x)
    assert np.array_equal(y[[0, 1, 2, 3, 5, 6]], np.array([0, 0, 0, 2.5, 0, np.inf], np.float32))
    assert np.isnan(y[4])  # `ugt` is true for NaN: NaN passes through


def test_maxpool_vs_torch_and_nan():
    x = synth.normal(51, (2, 3, 9, 11))
    want = F.max_pool2d(t(x), 3, 2, 1).numpy()
    assert np.array_equal(oracle.maxpool3x3s2(x), want)
    x[0, 0, 3, 3] = np.nan  # arith.maximumf propagates NaN: rows/cols 3 feed outputs 1 and 2
    y = oracle.maxpool3x3s2(x)
    assert np.isnan(y[0, 0, 1:3, 1:3]).all() and np.isnan(y).sum() == 4


def test_avgpool_and_fc():
    x = synth.normal(61, (3, 8, 7, 7))
    want = x.astype(np.float64).sum(axis=(2, 3)) / 49.0
    np.testing.assert_allclose(oracle.global_avgpool(x), want, rtol=1e-6, atol=1e-7)
    p = synth.normal(62, (3, 8))
    w = synth.normal(63, (5, 8))
    b = synth.normal(64, (5,))
    np.testing.assert_allclose(oracle.fc(p, w, b), F.linear(t(p).double(), t(w).double(), t(b).double()).numpy(),
                               rtol=1e-6, atol=1e-6)


# ---- Winograd F(4x4,3x3) -------------------------------------------------------------------

def test_winograd_identity_single_tile_fp64():
    """A^T[(G g G^T) .* (B^T d B)]A == direct 3x3 correlation, exact in rationals."""
    rng = np.random.default_rng(5)
    d = rng.standard_normal((1, 1, 6, 6)).astype(np.float32)
    g = rng.standard_normal((1, 1, 3, 3)).astype(np.float32)
    U = oracle.wino43_filter_transform(g)
    V = oracle.wino43_input_transform(d, pad=0)
    assert U.shape == (36, 1, 1) and V.shape == (36, 1, 1)
    M = oracle.wino43_batched_gemm(V, U)
    y = oracle.wino43_output_transform(M, 1, 4, 4)
    want = np.zeros((4, 4))
    for a in range(4):
        for b in range(4):
            want[a, b] = (d[0, 0, a:a + 3, b:b + 3].astype(np.float64) * g[0, 0]).sum()
    np.testing.assert_allclose(y[0, 0], want, rtol=0, atol=2e-6)


def test_winograd_filter_transform_known_values():
    """G g G^T of the all-ones filter: row sums of G are (1/4,-1/2,-1/6,7/24,1/8,1)."""
    U = oracle.wino43_filter_transform(np.ones((1, 1, 3, 3), np.float32)).reshape(6, 6)
    s = np.array([1 / 4, -1 / 2, -1 / 6, 7 / 24, 1 / 8, 1.0])
    np.testing.assert_allclose(U, np.outer(s, s), rtol=1e-14)
    # a delta filter at (p,q) gives the outer product of columns p and q of G
    g = np.zeros((1, 1, 3, 3), np.float32)
    g[0, 0, 0, 2] = 1
    G = np.array([[1 / 4, 0, 0], [-1 / 6, -1 / 6, -1 / 6], [-1 / 6, 1 / 6, -1 / 6],
                  [1 / 24, 1 / 12, 1 / 6], [1 / 24, -1 / 12, 1 / 6], [0, 0, 1]])
    np.testing.assert_allclose(oracle.wino43_filter_transform(g).reshape(6, 6), np.outer(G[:, 0], G[:, 2]), rtol=1e-14)


@pytest.mark.parametrize("H,W", [(8, 8), (7, 7), (14, 14), (5, 9)])
def test_winograd_equals_direct_ragged(H, W):
    x = synth.normal(71, (2, 5, H, W))
    w = synth.normal(72, (6, 5, 3, 3), std=0.3)
    direct = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, 1), w)
    wino = oracle.conv3x3_winograd43(x, w, pad=1)
    np.testing.assert_allclose(wino, direct, rtol=1e-5, atol=1e-5)
    V = oracle.wino43_input_transform(x, pad=1)
    assert V.shape == (36, 2 * ((H + 3) // 4) * ((W + 3) // 4), 5)


@pytest.mark.parametrize("schedule", ["omp", "ref"])
@pytest.mark.parametrize("R,stride,pad", [(3, 1, 1), (3, 2, 1), (1, 2, 0), (7, 2, 3), (3, 1, 0)])
def test_hostwparallel_conv_matches_scalar_oracle(R, stride, pad, schedule):
    """Both AVX2 convolutions timed as CPU baselines (the OpenMP one and the reference's sequential tile order) compute
    the same convolution as the scalar oracle (fp32 vs fp64 accumulation: agreement to fp32 rounding), ragged sizes and
    filter counts that are not multiples of 8 included."""
    x = synth.normal(910, (2, 12, 19, 23))
    w = synth.normal(911, (10, 12, R, R), std=0.2)
    got = oracle.hwp_conv2d(x, w, stride, pad, schedule=schedule)
    want = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, pad), w, stride=stride)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("schedule", ["omp", "ref"])
def test_hostwparallel_resnet18_matches_scalar_oracle(schedule):
    blob = synth.resnet18_params()
    x = synth.uniform(912, (1, 3, 64, 96), 0.0, 1.0)
    got = oracle.hwp_resnet18_forward(x, blob, schedule=schedule)
    want = oracle.resnet18_forward(x, blob)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    assert got.argmax(1) == want.argmax(1)


def test_driver_preprocess_and_top1_restatements():
    """The numpy restatements of the driver's image preparation and top-1 scan against a plain
    per-element Python transcription of the same formulas and against numpy's argmax."""
    img = np.random.default_rng(1).integers(0, 256, size=(1, 5, 4, 3), dtype=np.uint8)
    got = oracle.preprocess_u8(img)
    mean, std = (0.485, 0.456, 0.406), (0.229, 0.224, 0.225)
    for c in range(3):
        for y in range(5):
            for x in range(4):
                v = np.float32(img[0, y, x, c]) / np.float32(255.0)
                v = (v - np.float32(mean[c])) / np.float32(std[c])
                assert got[0, c, y, x] == v
    z = np.random.default_rng(2).normal(size=(4, 50)).astype(np.float32)
    assert np.array_equal(oracle.top1_scan(z), z.argmax(1))  # no ties, all above -100
    assert oracle.top1_scan(np.full((1, 5), -200.0, np.float32))[0] == 0


def test_preprocess_u8_against_exact_arithmetic_and_properties():
    """oracle.preprocess_u8 pinned without retyping its float formula: against exact rational arithmetic on the
    driver's constants (examples/Res18/main.cpp:38-77) for every 8-bit value and channel, by the round trip back to
    the 8-bit value, by monotonicity, and by one-hot images for the HWC -> CHW placement (a fourth channel is ignored)."""
    from fractions import Fraction
    mean = [Fraction(float(np.float32(v))) for v in (0.485, 0.456, 0.406)]  # the float literals the driver compiles in
    std = [Fraction(float(np.float32(v))) for v in (0.229, 0.224, 0.225)]
    img = np.zeros((1, 256, 1, 3), np.uint8)
    img[0, :, 0, :] = np.arange(256, dtype=np.uint8)[:, None]
    got = oracle.preprocess_u8(img)  # [1,3,256,1]
    assert got.shape == (1, 3, 256, 1) and got.dtype == np.float32
    for c in range(3):
        col = got[0, c, :, 0]
        assert np.all(np.diff(col) > 0)  # strictly increasing in the pixel value
        for u in range(256):
            exact = (Fraction(u, 255) - mean[c]) / std[c]
            # three fp32 roundings on the way, the subtraction cancelling up to half of the operand: a few ulp of 0.5 / std
            assert abs(Fraction(float(col[u])) - exact) <= Fraction(1, 10 ** 6), (c, u)
            back = (Fraction(float(col[u])) * std[c] + mean[c]) * 255
            assert round(back) == u
    # ImageNet constants: a mid-grey pixel lands near zero in every channel, black and white at -mean/std and (1-mean)/std
    assert np.all(np.abs(got[0, :, 124, 0]) < 0.4)
    assert np.allclose(got[0, :, 0, 0], [-0.485 / 0.229, -0.456 / 0.224, -0.406 / 0.225], rtol=1e-6)
    assert np.allclose(got[0, :, 255, 0], [0.515 / 0.229, 0.544 / 0.224, 0.594 / 0.225], rtol=1e-6)
    # placement: a single bright sample at (y, x, c) changes exactly output [c, y, x]; alpha is ignored
    base = oracle.preprocess_u8(np.zeros((2, 3, 4, 4), np.uint8))
    for (n, y, x, c) in ((0, 0, 0, 0), (1, 2, 3, 1), (0, 1, 2, 2)):
        im = np.zeros((2, 3, 4, 4), np.uint8)
        im[n, y, x, c] = 200
        d = oracle.preprocess_u8(im) != base
        assert d.sum() == 1 and d[n, c, y, x]
    im = np.zeros((2, 3, 4, 4), np.uint8)
    im[..., 3] = 255
    assert np.array_equal(oracle.preprocess_u8(im), base)


def test_top1_scan_semantics():
    """The driver's scan (examples/Res18/main.cpp:103-111): strict `>` from -100 and index 0, left to right: the first of
    equal maxima wins, rows that never exceed -100 give 0, NaN never wins; without ties it is numpy's argmax."""
    z = np.random.default_rng(2).normal(size=(64, 1000)).astype(np.float32)
    assert np.array_equal(oracle.top1_scan(z), z.argmax(1))
    f = lambda row: int(oracle.top1_scan(np.array([row], np.float32))[0])
    assert f([1, 3, 3, 2]) == 1
    assert f([-200, -150, -100, -101]) == 0          # -100 itself does not exceed the initial maximum
    assert f([-200, -99.5, -300]) == 1
    assert f([np.nan, 1.0, 0.5]) == 1
    assert f([np.nan, -200, -300]) == 0
    assert f([2.0, np.nan, 5.0, np.nan]) == 2
    assert f([np.inf, np.inf]) == 0 and f([-np.inf, -np.inf]) == 0

