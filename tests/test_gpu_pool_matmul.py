"""Pooling kernels and the fp32 GEMM against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import dev, empty, host, nhwc, nchw, max_rel, FP32_MAX_REL

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
# the last three take the row form (a workgroup per output row, two output pixels per thread): odd and even widths,
# a last pair with one pixel, the stem's own shape
@pytest.mark.parametrize("N,C,H,W", [(2, 64, 16, 16), (1, 8, 9, 7), (3, 16, 5, 6), (2, 64, 37, 35), (3, 128, 20, 34), (1, 64, 112, 112)])
def test_maxpool(dt, N, C, H, W):
    x = synth.normal(300, (N, C, H, W))
    if dt == abi.F16:
        x = synth.round_fp16(x)
    x[0, 1, 2, 2] = np.nan  # arith.maximumf propagates NaN
    x[N - 1, C - 1, H - 1, W - 1] = np.nan
    x[0, 3, H // 2, :] = -np.inf  # a window of nothing but -inf stays -inf
    x[0, 3, H // 2 - 1, :] = -np.inf
    x[0, 3, H // 2 + 1, :] = -np.inf
    want = oracle.maxpool3x3s2(x)
    OH, OW = want.shape[2:]
    out = empty((N, OH, OW, C), dt)
    xd = dev(nhwc(x), dt)  # keep every device operand alive in a variable until the call returns
    abi.check(abi.lib().nncv_hip_maxpool3x3s2(dt, xd.data_ptr(), out.data_ptr(), N, H, W, C, None))
    got = nchw(host(out))
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.nan_to_num(got, nan=7.0), np.nan_to_num(want, nan=7.0))  # max is exact


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
@pytest.mark.parametrize("N,C,H,W", [(2, 512, 7, 7), (1, 512, 8, 8), (3, 96, 3, 5)])
def test_global_avgpool(dt, N, C, H, W):
    x = synth.normal(310, (N, C, H, W))
    if dt == abi.F16:
        x = synth.round_fp16(x)
    want = oracle.global_avgpool(x)
    out = empty((N, C), dt)
    xd = dev(nhwc(x), dt)
    abi.check(abi.lib().nncv_hip_global_avgpool(dt, xd.data_ptr(), out.data_ptr(), N, H, W, C, None))
    tol = 1e-6 if dt == abi.F32 else 1e-3  # fp16 result is rounded to half once
    assert np.abs(host(out) - want).max() <= tol * max(1.0, np.abs(want).max())


# linalg.matmul puts no condition on M, N, K: odd sizes (rows that are not 16-byte multiples) take the element-wise
# loader; the sizes also walk the launch shapes: 128x128 tiles, 64x64 tiles with 1, 2 and 4 K groups
@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (130, 68, 36), (64, 64, 16), (257, 512, 1000), (1, 4, 4),
                                   (33, 17, 5), (1, 1, 1), (65, 130, 259), (1000, 1001, 127), (2048, 2048, 64), (300, 200, 130),
                                   (1500, 1300, 200), (97, 1, 1031)])
def test_matmul_device(M, N, K):
    a = synth.uniform(320, (M, K), -1, 1)
    b = synth.uniform(321, (K, N), -1, 1)
    c0 = synth.uniform(322, (M, N), -1, 1)
    want = oracle.matmul(a, b, c0)
    ad, bd, c = dev(a), dev(b), dev(c0)
    abi.check(abi.lib().nncv_hip_matmul_f32(ad.data_ptr(), bd.data_ptr(), c.data_ptr(), M, N, K, None))
    err = max_rel(host(c), want)
    print("matmul", M, N, K, "max_rel", err, flush=True)
    assert err < FP32_MAX_REL


def test_cfg1_matmul_through_reference_abi():
    """BASELINE config 1 through _mlir_ciface_matmul: C (zeros) += A.B on host memrefs, plus a
    strided (transposed-view) operand, which the descriptor semantics must honour."""
    a, b = synth.cfg1_matmul()
    c = np.zeros((1024, 1024), np.float32)
    abi.matmul(a, b, c)
    want = oracle.matmul(a, b)
    assert max_rel(c, want) < FP32_MAX_REL
    at = np.ascontiguousarray(a.T).T  # same values, column-major strides
    assert at.strides != a.strides
    c2 = np.zeros((1024, 1024), np.float32)
    abi.matmul(at, b, c2)
    assert np.array_equal(c, c2)


def test_matmul_through_reference_abi_any_shape():
    """The reference's compiled linalg.matmul takes any M, N, K; so does the symbol here (no abort on rows that are
    not multiples of 16 bytes)."""
    for (M, N, K) in ((33, 17, 5), (7, 9, 3)):
        a = synth.uniform(330, (M, K), -1, 1)
        b = synth.uniform(331, (K, N), -1, 1)
        c = synth.uniform(332, (M, N), -1, 1)
        want = oracle.matmul(a, b, c)
        abi.matmul(a, b, c)
        assert max_rel(c, want) < FP32_MAX_REL


def test_matmul_k_groups_are_deterministic():
    """The K groups of a workgroup meet in a fixed order: two runs give the same bits."""
    a, b = synth.cfg1_matmul()
    ad, bd = dev(a), dev(b)
    outs = []
    for _ in range(2):
        c = dev(np.zeros((1024, 1024), np.float32))
        abi.check(abi.lib().nncv_hip_matmul_f32(ad.data_ptr(), bd.data_ptr(), c.data_ptr(), 1024, 1024, 1024, None))
        outs.append(host(c))
    assert np.array_equal(outs[0], outs[1])
