"""The fp16 3x3 stride-1 stream kernel (conv3x3_f16.hip) against the oracle, on launches large enough for the dispatcher
to hand them to it: every tile geometry (tiles inside their image, tiles across images one zero row apart, odd and
oblong images), one to four channel slabs, workgroups that walk several tiles, all three workgroup forms (32, 64 and
128 filters), with and without BatchNorm and residual, ReLU and the other fused activations (residual before and
after).  The route is asserted from the launch tags, so a silent fall-back to another kernel fails the test.
Checker: the OpenMP x AVX2 convolution of the oracle (itself checked against the scalar one in test_oracle_ops.py),
then BatchNorm / residual / activation as the oracle's own functions spell them."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import Conv, dev, host, nhwc, nchw, rel_l2, FP16_REL_L2

pytestmark = pytest.mark.gpu

# N, H, W, C, F, BatchNorm, residual, activation, expected tag
CASES = [
    (8, 28, 28, 128, 128, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x1x4>"),      # 56 tiles x 4 filter groups, two slabs
    (12, 14, 14, 256, 256, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x1x4>"),     # images one zero row apart, four slabs
    (20, 56, 56, 64, 64, True, False, abi.ACT_RELU, "conv3x3_stream<f16,1x2x2,res>"),  # 560 tiles: workgroups walk two tiles; one slab: weights stay in registers
    (37, 56, 56, 64, 64, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x2x2,res>"),   # 1036 tiles: three tiles on the same fragments, residual
    (16, 56, 56, 64, 64, False, True, abi.ACT_NONE, "conv3x3_stream<f16,1x2x2,res>"),  # one tile per workgroup, no BatchNorm
    (58, 28, 28, 64, 128, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x4x1>"),      # 406 workgroups of 128 filters, no K groups
    (10, 23, 17, 192, 160, False, True, abi.ACT_NONE, "conv3x3_stream<f16,1x1x4>"),    # oblong, 32-filter groups only, no BatchNorm
    (6, 40, 40, 128, 128, True, False, abi.ACT_SILU, "conv3x3_stream<f16,1x2x2,act>"),
    (6, 40, 40, 128, 128, True, True, abi.ACT_HARDSWISH, "conv3x3_stream<f16,1x2x2,act>"),
    (6, 40, 40, 64, 96, True, True, abi.ACT_SIGMOID, "conv3x3_stream<f16,1x1x4,act>"),
    (3, 97, 31, 64, 96, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x1x4>"),        # 97 rows of 31: the last tile of an image is short
]


def bn_params(seed, F):
    return (synth.uniform(seed, (F,), 0.5, 1.5), synth.normal(seed + 1, (F,), std=0.1),
            synth.normal(seed + 2, (F,), std=0.1), synth.uniform(seed + 3, (F,), 0.5, 1.5))


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c[:5]) + "_act%d" % c[7])
def test_stream_kernel_matches_the_oracle(case):
    check_case(case, 9600 + CASES.index(case) * 10)


# With three or more passes in flight (nncv_hip_set_overlap_hint) the 128-filter form is taken wherever the filter count
# allows it, also on launches of a few dozen workgroups, and ReLU layers it does not fit go to the patch kernel.
OVERLAP_CASES = [
    (8, 28, 28, 128, 128, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x4x1>"),      # 56 workgroups, two slabs
    (12, 14, 14, 256, 256, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x4x1>"),     # 40 workgroups across image borders, four slabs
    (5, 97, 31, 64, 128, True, False, abi.ACT_RELU, "conv3x3_stream<f16,1x4x1>"),      # short last tile of an image
    (20, 56, 56, 64, 64, True, True, abi.ACT_RELU, "conv3x3_stream<f16,1x2x2,res>"),   # one slab: resident weights, 187 workgroups of three tiles
    (20, 56, 56, 128, 64, True, False, abi.ACT_RELU, "conv3x3_patch<f16,2,2>"),        # 64 filters, two slabs: the patch kernel
    (6, 40, 40, 128, 128, True, True, abi.ACT_HARDSWISH, "conv3x3_stream<f16,1x2x2,act>"),  # other activations keep their form
]


@pytest.mark.parametrize("case", OVERLAP_CASES, ids=lambda c: "x".join(str(v) for v in c[:5]) + "_act%d" % c[7])
def test_launch_shapes_under_the_overlap_hint_match_the_oracle(case):
    L = abi.lib()
    try:
        abi.check(L.nncv_hip_set_overlap_hint(4))
        check_case(case, 9900 + OVERLAP_CASES.index(case) * 10)
    finally:
        abi.check(L.nncv_hip_set_overlap_hint(1))


def check_case(case, seed):
    N, H, W, C, F, use_bn, use_res, act, tag = case
    print("stream case", case, flush=True)
    x = synth.round_fp16(synth.normal(seed, (N, C, H, W)))
    w = synth.round_fp16(synth.normal(seed + 1, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9)))))
    bn = tuple(synth.round_fp16(b) for b in bn_params(seed + 2, F)) if use_bn else None
    res = synth.round_fp16(synth.normal(seed + 6, (N, F, H, W))) if use_res else None
    y = oracle.hwp_conv2d(x, w, 1, 1)
    if bn:
        y = oracle.batchnorm(y, *bn)
    if res is not None:
        y = (y + res).astype(np.float32)
    want = oracle.ACTIVATIONS[act](y)
    conv = Conv(abi.F16, w, 1, 1, bn=bn, relu=act, algo=abi.ALGO_IGEMM)
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
    assert list(rep) == [tag], rep
    err = rel_l2(got, want)
    print("rel_l2", err, flush=True)
    assert err < FP16_REL_L2
    # every output pixel was written (a tile walked twice or not at all would leave zeros or doubled rows)
    assert np.isfinite(got).all()
    assert float(np.max(np.abs(got - want))) < 0.05 * max(1.0, float(np.max(np.abs(want))))


@pytest.mark.parametrize("shape", [(37, 56, 56, 64, 64), (24, 28, 28, 128, 128), (40, 14, 14, 256, 256)],
                         ids=lambda c: "x".join(str(v) for v in c))
@pytest.mark.parametrize("hint", [1, 4])
def test_stream_kernel_gives_the_same_bits_every_time(shape, hint):
    """The kernel's ordering of its own memory traffic is by hand (wait counts around the LDS DMA, resident weight
    fragments that nothing later waits for): the same launch twelve times over, with other work in between, must give
    the same bits as the first -- a load consumed before it landed would show here even where the error stays small."""
    N, H, W, C, F = shape
    seed = 9990
    x = synth.round_fp16(synth.normal(seed, (N, C, H, W)))
    w = synth.round_fp16(synth.normal(seed + 1, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9)))))
    bn = tuple(synth.round_fp16(b) for b in bn_params(seed + 2, F))
    res = synth.round_fp16(synth.normal(seed + 6, (N, F, H, W)))
    L = abi.lib()
    try:
        abi.check(L.nncv_hip_set_overlap_hint(hint))  # 4: the 128-filter form, resident weights on long-lived workgroups
        conv = Conv(abi.F16, w, 1, 1, bn=bn, relu=abi.ACT_RELU, algo=abi.ALGO_IGEMM)
        xd, rd = dev(nhwc(x), abi.F16), dev(nhwc(res), abi.F16)
        first = host(conv(xd, abi.NHWC, residual=rd)).view(np.uint16).copy()
        for rep in range(12):
            other = torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")  # evicts, shifts timing
            again = host(conv(xd, abi.NHWC, residual=rd if rep % 2 == 0 else None))
            if rep % 2 == 0:
                assert np.array_equal(again.view(np.uint16), first), rep
            assert other.shape == (512, 512)
        conv.close()
    finally:
        abi.check(L.nncv_hip_set_overlap_hint(1))


def test_bottleneck_and_concatenation_views_through_the_executor():
    """x + act(conv3x3(x)) written into a slice of a concatenated tensor: the graph executor folds the add into the
    convolution's epilogue (residual added after the activation) and lets the convolution read and write rows at the
    concatenated tensor's pixel pitch, so the stream kernel runs with pitches that differ from its channel counts."""
    from gpu_util import Graph
    C, N, H, W = 128, 6, 40, 40
    sizes, ops = [], []

    def take(n):
        off = sum(sizes)
        sizes.append(n)
        return off

    def conv(i, o, cin, F, k, act):
        w = take(F * cin * k * k)
        bnp = tuple(take(F) for _ in range(4))
        ops.append(abi.graph_op(abi.OP_CONV, [i, -1], o, F=F, K=k, stride=1, pad=(k - 1) // 2, act=act, eps=1e-3, w=w, bias=-1, bn=bnp))

    conv(0, 1, C, C, 1, abi.ACT_SILU)
    conv(0, 2, C, C, 1, abi.ACT_SILU)
    ops.append(abi.graph_op(abi.OP_CONCAT, [1, 2], 3))   # tensors 1 and 2 live in slices of tensor 3 ...
    conv(1, 4, C, C, 3, abi.ACT_SILU)                    # ... so this 3x3 reads rows at tensor 3's pitch and writes at tensor 6's
    conv(3, 5, 2 * C, C, 1, abi.ACT_SILU)
    ops.append(abi.graph_op(abi.OP_CONCAT, [4, 5], 6))
    conv(6, 7, 2 * C, C, 1, abi.ACT_NONE)
    conv(7, 8, C, C, 3, abi.ACT_SILU)                    # a Bottleneck: x + act(conv(x)), the add folded into the epilogue
    ops.append(abi.graph_op(abi.OP_ADD, [8, 7], 9))
    blob = synth.normal(9800, (sum(sizes),), std=0.05)
    for o in ops:
        if o.var >= 0:
            blob[o.var:o.var + o.F] = synth.uniform(9801, (o.F,), 0.5, 1.5)
    blob = synth.round_fp16(blob)
    x = synth.round_fp16(synth.normal(9802, (N, C, H, W)))
    g = Graph(ops, C, blob, abi.F16)
    xd = dev(x, abi.F16)
    g(xd)
    torch.cuda.synchronize()
    abi.profile_enable(True)
    try:
        abi.profile_report()
        got = host(g(xd))
        rep = abi.profile_report()
    finally:
        abi.profile_enable(False)
    g.close()
    print({k: v["launches"] for k, v in rep.items()}, flush=True)
    assert rep.get("conv3x3_stream<f16,1x2x2,act>", {}).get("launches") == 2
    assert not any(k.startswith("eltwise") or k.startswith("concat") for k in rep), "the add and the copies are folded away"
    want = oracle.run_graph(ops, x, blob, C)
    assert rel_l2(got, want) < FP16_REL_L2
