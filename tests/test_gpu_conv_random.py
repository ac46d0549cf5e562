"""fp16 3x3 convolutions of seeded random shapes against the oracle, whatever kernel the dispatcher picks for them
(stream kernel in its three forms, LDS-patch kernel at both strides, implicit GEMM for what neither takes), once with
the launch shapes of one pass at a time and once with those of several passes in flight (nncv_hip_set_overlap_hint).
The shapes are drawn once from a fixed seed: odd and oblong images, batches that do not divide into tiles, channel
counts from one to four 128-byte slabs, filter counts that are and are not multiples of 64 and 128."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import Conv, dev, host, nhwc, nchw, rel_l2, FP16_REL_L2

pytestmark = pytest.mark.gpu


def draw_cases(n):
    rng = np.random.default_rng(20251128)
    cases = []
    while len(cases) < n:
        N = int(rng.choice([1, 2, 3, 5, 7, 12, 19, 33]))
        H, W = int(rng.integers(5, 72)), int(rng.integers(5, 72))
        C = 64 * int(rng.integers(1, 5))
        F = 32 * int(rng.integers(1, 9))
        stride = int(rng.choice([1, 1, 2]))
        if 2.0 * N * H * W * C * F * 9 / stride ** 2 > 6e9:
            continue
        cases.append((N, H, W, C, F, stride, bool(rng.integers(0, 2))))
    return cases


CASES = draw_cases(18)


@pytest.mark.parametrize("hint", [1, 4])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(int(v)) for v in c))
def test_random_shape_matches_the_oracle(case, hint):
    N, H, W, C, F, stride, use_res = case
    seed = 12000 + CASES.index(case) * 10
    x = synth.round_fp16(synth.normal(seed, (N, C, H, W)))
    w = synth.round_fp16(synth.normal(seed + 1, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9)))))
    bn = tuple(synth.round_fp16(b) for b in (synth.uniform(seed + 2, (F,), 0.5, 1.5), synth.normal(seed + 3, (F,), std=0.1),
                                             synth.normal(seed + 4, (F,), std=0.1), synth.uniform(seed + 5, (F,), 0.5, 1.5)))
    OH, OW = (H - 1) // stride + 1, (W - 1) // stride + 1
    res = synth.round_fp16(synth.normal(seed + 6, (N, F, OH, OW))) if use_res else None
    y = oracle.batchnorm(oracle.hwp_conv2d(x, w, stride, 1), *bn)
    if res is not None:
        y = (y + res).astype(np.float32)
    want = oracle.ACTIVATIONS[abi.ACT_RELU](y)
    L = abi.lib()
    try:
        abi.check(L.nncv_hip_set_overlap_hint(hint))
        conv = Conv(abi.F16, w, stride, 1, bn=bn, relu=abi.ACT_RELU, algo=abi.ALGO_IGEMM)
        xd = dev(nhwc(x), abi.F16)
        rd = dev(nhwc(res), abi.F16) if res is not None else None
        conv(xd, abi.NHWC, residual=rd)
        torch.cuda.synchronize()
        abi.profile_enable(True)
        try:
            abi.profile_report()
            got = nchw(host(conv(xd, abi.NHWC, residual=rd)))
            rep = abi.profile_report()
        finally:
            abi.profile_enable(False)
        conv.close()
    finally:
        abi.check(L.nncv_hip_set_overlap_hint(1))
    err = rel_l2(got, want)
    print("case", case, "hint", hint, "->", list(rep), "rel_l2 %.2e" % err, flush=True)
    assert got.shape == want.shape
    assert err < FP16_REL_L2
    assert float(np.max(np.abs(got - want))) < 0.05 * max(1.0, float(np.max(np.abs(want))))
