"""Each Winograd F(4x4,3x3) stage on the GPU against the oracle's stage (fp64), through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import dev, empty, host, nhwc, nchw, max_rel, rel_l2

pytestmark = pytest.mark.gpu

SHAPES = [(2, 8, 12, 8, 8), (1, 16, 8, 7, 7), (3, 4, 4, 5, 9), (1, 64, 64, 14, 14)]  # N, C, F, H, W


@pytest.mark.parametrize("N,C,F,H,W", SHAPES)
@pytest.mark.parametrize("layout", [abi.NHWC, abi.NCHW])
def test_stages_fp32(N, C, F, H, W, layout):
    print("case", N, C, F, H, W, layout, flush=True)
    L = abi.lib()
    x = synth.normal(200, (N, C, H, W))
    w = synth.normal(201, (F, C, 3, 3), std=0.2)
    TH, TW = (H + 3) // 4, (W + 3) // 4
    tiles = N * TH * TW
    # filter
    U = empty((36, F, C), abi.F32)
    wd = dev(w)  # every device operand stays alive in a variable until the call returns
    abi.check(L.nncv_hip_wino43_filter(abi.F32, wd.data_ptr(), U.data_ptr(), F, C, None))
    U_ref = oracle.wino43_filter_transform(w)
    assert max_rel(host(U), U_ref) < 1e-6
    # input
    xin = dev(nhwc(x) if layout == abi.NHWC else x)
    V = empty((36, tiles, C), abi.F32)
    abi.check(L.nncv_hip_wino43_input(abi.F32, xin.data_ptr(), layout, V.data_ptr(), N, C, H, W, 1, None))
    V_ref = oracle.wino43_input_transform(x, pad=1)
    assert max_rel(host(V), V_ref) < 1e-5
    # batched GEMM
    M = empty((36, tiles, F), abi.F32)
    abi.check(L.nncv_hip_wino43_gemm(abi.F32, V.data_ptr(), U.data_ptr(), M.data_ptr(), tiles, C, F, None))
    M_ref = oracle.wino43_batched_gemm(V_ref, U_ref)
    assert max_rel(host(M), M_ref) < 1e-5
    # output (+ scale/shift/residual/relu)
    scale = synth.uniform(202, (F,), 0.5, 1.5)
    shift = synth.normal(203, (F,), 0.1)
    res = synth.normal(204, (N, F, H, W))
    out = empty((N, H, W, F) if layout == abi.NHWC else (N, F, H, W), abi.F32)
    rdev = dev(nhwc(res) if layout == abi.NHWC else res)
    scd, shd = dev(scale), dev(shift)
    abi.check(L.nncv_hip_wino43_output(abi.F32, M.data_ptr(), out.data_ptr(), layout, N, F, H, W,
                                       scd.data_ptr(), shd.data_ptr(), rdev.data_ptr(), 1, None))
    y_ref = oracle.wino43_output_transform(M_ref, N, H, W).astype(np.float64)
    y_ref = np.maximum(y_ref * scale[None, :, None, None] + shift[None, :, None, None] + res, 0)
    got = host(out)
    got = nchw(got) if layout == abi.NHWC else got
    assert max_rel(got, y_ref) < 1e-5
    # and the whole route equals the direct convolution
    direct = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, 1), w)
    plain = empty(out.shape, abi.F32)
    abi.check(L.nncv_hip_wino43_output(abi.F32, M.data_ptr(), plain.data_ptr(), layout, N, F, H, W,
                                       None, None, None, 0, None))
    p = host(plain)
    p = nchw(p) if layout == abi.NHWC else p
    assert max_rel(p, direct) < 1e-4


def test_stages_fp16_storage():
    """fp16 storage of U, V, M with fp32 transform arithmetic and fp32 MFMA accumulation."""
    N, C, F, H, W = 2, 32, 32, 12, 12
    L = abi.lib()
    x = synth.round_fp16(synth.normal(210, (N, C, H, W)))
    w = synth.round_fp16(synth.normal(211, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9)))))
    tiles = N * 3 * 3
    U = empty((36, F, C), abi.F16)
    V = empty((36, tiles, C), abi.F16)
    M = empty((36, tiles, F), abi.F16)
    out = empty((N, H, W, F), abi.F16)
    wd, xd = dev(w, abi.F16), dev(nhwc(x), abi.F16)
    abi.check(L.nncv_hip_wino43_filter(abi.F16, wd.data_ptr(), U.data_ptr(), F, C, None))
    abi.check(L.nncv_hip_wino43_input(abi.F16, xd.data_ptr(), abi.NHWC, V.data_ptr(), N, C, H, W, 1, None))
    abi.check(L.nncv_hip_wino43_gemm(abi.F16, V.data_ptr(), U.data_ptr(), M.data_ptr(), tiles, C, F, None))
    abi.check(L.nncv_hip_wino43_output(abi.F16, M.data_ptr(), out.data_ptr(), abi.NHWC, N, F, H, W, None, None, None, 0, None))
    # stage-wise: each stored tensor is the oracle's value rounded to half (up to 1 half ulp)
    assert rel_l2(host(U), oracle.wino43_filter_transform(w)) < 1e-3
    assert rel_l2(host(V), oracle.wino43_input_transform(x, 1)) < 1e-3
    direct = oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, 1), w)
    err = rel_l2(nchw(host(out)), direct)
    print("fp16 winograd rel-L2 vs direct:", err, flush=True)
    assert err < 1e-2
