"""Operators of the reference's other fixtures (MobileNetV3.mlir, Yolov5s.mlir) and the graph
executor built from them, on the GPU through the C ABI, against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from nncv_amd import mobilenetv3_spec as spec
from gpu_util import Conv, Graph, dev, empty, host, nchw, nhwc, max_rel, rel_l2, FP32_MAX_REL, FP16_REL_L2

pytestmark = pytest.mark.gpu

ACTS = [abi.ACT_NONE, abi.ACT_RELU, abi.ACT_HARDSWISH, abi.ACT_HARDSIGMOID, abi.ACT_SILU, abi.ACT_SIGMOID]


def r16(a):
    return synth.round_fp16(a)


# ---------------------------------------------------------------------------------------------
# single operators
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
@pytest.mark.parametrize("k,stride,shape", [(3, 1, (2, 24, 13, 17)), (3, 2, (1, 16, 64, 64)), (5, 1, (3, 40, 9, 11)),
                                            (5, 2, (2, 96, 32, 31)), (5, 1, (1, 576, 8, 8)), (3, 2, (1, 8, 5, 4))])
def test_dwconv_vs_oracle(dt, k, stride, shape):
    N, C, H, W = shape
    pad = (k - 1) // 2
    x = synth.normal(7000 + k, shape)
    w = synth.normal(7001 + k, (C, 1, k, k), std=0.4)
    scale = synth.uniform(7002, (C,), 0.5, 1.5)
    shift = synth.normal(7003, (C,), std=0.2)
    if dt == abi.F16:
        x, w = r16(x), r16(w)
    conv = oracle.depthwise_conv2d_nchw_chw(oracle.pad_nchw(x, pad), w, stride)
    OH, OW = conv.shape[2:]
    xd, wd, sd, hd = dev(nhwc(x), dt), dev(w, dt), dev(scale), dev(shift)
    for act, affine in [(abi.ACT_NONE, False), (abi.ACT_HARDSWISH, True), (abi.ACT_RELU, True)]:
        want = conv * scale.reshape(1, C, 1, 1) + shift.reshape(1, C, 1, 1) if affine else conv
        want = oracle.ACTIVATIONS[act](want.astype(np.float32))
        out = empty((N, OH, OW, C), dt)
        print("dwconv", dt, k, stride, shape, act, affine, flush=True)
        abi.check(abi.lib().nncv_hip_dwconv(dt, xd.data_ptr(), wd.data_ptr(), sd.data_ptr() if affine else None,
                                            hd.data_ptr() if affine else None, out.data_ptr(), N, H, W, C, k, stride,
                                            pad, act, None))
        got = nchw(host(out))
        if dt == abi.F32:
            assert max_rel(got, want) < FP32_MAX_REL
        else:
            assert rel_l2(got, want) < 2e-3  # one rounding of the result to half


def test_dwconv_rejects_bad_arguments():
    x = empty((1, 4, 4, 12), abi.F16)
    L = abi.lib()
    assert L.nncv_hip_dwconv(abi.F16, x.data_ptr(), x.data_ptr(), None, None, x.data_ptr(), 1, 4, 4, 12, 3, 1, 1, 0, None) != 0
    assert b"multiple" in L.nncv_hip_last_error()  # 12 channels are not whole 16-byte vectors of halves
    assert L.nncv_hip_dwconv(abi.F16, x.data_ptr(), x.data_ptr(), None, None, x.data_ptr(), 1, 4, 4, 16, 4, 1, 1, 0, None) != 0
    assert L.nncv_hip_dwconv(abi.F16, x.data_ptr(), x.data_ptr(), None, None, x.data_ptr(), 1, 2, 2, 16, 5, 1, 0, 0, None) != 0


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_eltwise_activations_and_add(dt):
    special = np.float32([-3, 3, 0, -0.0, 6, -6, np.inf, -np.inf, np.nan, 1e-8, -1e-8, 2.999, -2.999])
    a = np.concatenate([synth.normal(7100, (4083,), std=3.0), special]).astype(np.float32)
    b = synth.normal(7101, a.shape, std=1.0)
    if dt == abi.F16:
        a, b = r16(a), r16(b)
    ad, bd = dev(a, dt), dev(b, dt)
    for act in ACTS:
        for add in (False, True):
            want = oracle.ACTIVATIONS[act]((a + b).astype(np.float32) if add else a)
            out = empty(a.shape, dt)
            abi.check(abi.lib().nncv_hip_eltwise(dt, ad.data_ptr(), bd.data_ptr() if add else None, out.data_ptr(), a.size, act, None))
            got = host(out)
            if dt == abi.F16:
                want = r16(want)
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(got), nan), (act, add)
            fin = np.isfinite(want)
            assert np.array_equal(got[~fin & ~nan], want[~fin & ~nan]), (act, add)
            tol = 2e-3 if dt == abi.F16 else 2e-6
            assert np.abs(got[fin] - want[fin]).max() <= tol * max(1.0, np.abs(want[fin]).max()), (act, add)
            if act in (abi.ACT_NONE, abi.ACT_RELU, abi.ACT_HARDSIGMOID) and not add and dt == abi.F32:
                assert np.array_equal(got[fin], want[fin])  # no transcendental, no product: bit exact


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_scale_concat_upsample_maxpool(dt):
    N, H, W, C = 2, 7, 5, 24
    x = synth.normal(7200, (N, C, H, W))
    g = synth.uniform(7201, (N, C), 0.0, 1.0)
    if dt == abi.F16:
        x, g = r16(x), r16(g)
    xd = dev(nhwc(x), dt)
    L = abi.lib()
    # squeeze-excitation gate
    out, gd = empty((N, H, W, C), dt), dev(g, dt)
    abi.check(L.nncv_hip_scale_channels(dt, xd.data_ptr(), gd.data_ptr(), out.data_ptr(), N, H * W, C, None))
    want = g.reshape(N, C, 1, 1) * x
    assert np.array_equal(nchw(host(out)), r16(want) if dt == abi.F16 else want)
    # concat of [x, y] into 24 + 16 channels, then a 2x up-sampled copy into another slice
    y = synth.normal(7202, (N, 16, H, W))
    y = r16(y) if dt == abi.F16 else y
    cat = torch.zeros((N, H, W, 40), dtype=xd.dtype, device="cuda")
    abi.check(L.nncv_hip_concat_slice(dt, xd.data_ptr(), cat.data_ptr(), N * H * W, 24, 40, 0, None))
    yd = dev(nhwc(y), dt)
    abi.check(L.nncv_hip_concat_slice(dt, yd.data_ptr(), cat.data_ptr(), N * H * W, 16, 40, 24, None))
    assert np.array_equal(nchw(host(cat)), np.concatenate([x, y], axis=1))
    up = torch.zeros((N, 2 * H, 2 * W, 40), dtype=xd.dtype, device="cuda")
    abi.check(L.nncv_hip_upsample2x(dt, xd.data_ptr(), up.data_ptr(), N, H, W, 24, 40, 16, None))
    got = nchw(host(up))
    assert np.array_equal(got[:, 16:], oracle.upsample2x_nearest(x)) and not got[:, :16].any()
    # max-pool windows of the fixtures: SPPF 5x5 s1 p2, the ResNet 3x3 s2 p1, a plain 2x2 s2
    for k, s, p in [(5, 1, 2), (3, 2, 1), (2, 2, 0)]:
        want = oracle.maxpool_nchw(x, k, s, p)
        out = empty((N, want.shape[2], want.shape[3], C), dt)
        abi.check(L.nncv_hip_maxpool(dt, xd.data_ptr(), out.data_ptr(), N, H, W, C, k, s, p, None))
        assert np.array_equal(nchw(host(out)), want)
    assert L.nncv_hip_concat_slice(dt, xd.data_ptr(), cat.data_ptr(), N * H * W, 24, 40, 20, None) != 0  # 20 + 24 > 40


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
@pytest.mark.parametrize("C,F,k,stride,H", [(96, 576, 1, 1, 8), (64, 64, 3, 1, 20), (40, 240, 1, 1, 16), (64, 128, 3, 2, 21)])
def test_conv_with_fused_activations(dt, C, F, k, stride, H):
    """hard-swish / SiLU / hard-sigmoid in the epilogue of the MFMA kernels (fast and generic tiles)."""
    x = synth.normal(7300, (2, C, H, H))
    w = synth.normal(7301, (F, C, k, k), std=float(np.sqrt(2.0 / (C * k * k))))
    bn = (synth.uniform(7302, (F,), 0.5, 1.5), synth.normal(7303, (F,), std=0.1), synth.normal(7304, (F,), std=0.1),
          synth.uniform(7305, (F,), 0.5, 1.5))
    if dt == abi.F16:
        x, w = r16(x), r16(w)
        bn = tuple(r16(b) for b in bn)
    pad = (k - 1) // 2
    pre = oracle.batchnorm(oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, pad) if pad else x, w, stride), *bn)
    xd = dev(nhwc(x), dt)
    for act in (abi.ACT_HARDSWISH, abi.ACT_SILU, abi.ACT_HARDSIGMOID):
        conv = Conv(dt, w, stride, pad, bn=bn, relu=act, algo=abi.ALGO_IGEMM)
        print("conv+act", dt, C, F, k, stride, H, act, flush=True)
        got = nchw(host(conv(xd, abi.NHWC)))
        want = oracle.ACTIVATIONS[act](pre)
        if dt == abi.F32:
            assert max_rel(got, want) < FP32_MAX_REL
        else:
            assert rel_l2(got, want) < FP16_REL_L2
        conv.close()


# ---------------------------------------------------------------------------------------------
# MobileNetV3-small through the graph executor
# ---------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def blob():
    return synth.mobilenetv3_params()


def tensors_of(blob):
    return {name: blob[o:o + spec.numel(shape)].reshape(shape) for name, (o, shape) in spec.offsets().items()}


@pytest.mark.parametrize("shape", [(2, 3, 64, 64), (1, 3, 256, 256), (3, 3, 100, 77)])
def test_mobilenetv3_fp32(blob, shape):
    ops, n = abi.mobilenetv3_small_ops()
    g = Graph(ops, 3, blob, abi.F32)
    assert abi.graph_output_shape(g.h, shape[2], shape[3]) == (1000, 1, 1)
    x = synth.uniform(7400, shape, 0.0, 1.0)
    print("mobilenetv3 fp32", shape, flush=True)
    got = host(g(dev(x))).reshape(shape[0], 1000)
    want = oracle.mobilenetv3_forward(x, tensors_of(blob))
    err = max_rel(got, want)
    print("logits max_rel", err, flush=True)
    assert err < FP32_MAX_REL
    assert np.array_equal(got.argmax(1), want.argmax(1))
    g.close()


@pytest.mark.parametrize("shape", [(2, 3, 64, 64), (32, 3, 224, 224), (3, 3, 100, 77)])  # odd width: no pixel pairs
def test_mobilenetv3_fp16(blob, shape):
    b16 = r16(blob)
    ops, n = abi.mobilenetv3_small_ops()
    g = Graph(ops, 3, b16, abi.F16)
    x = r16(synth.uniform(7401, shape, 0.0, 1.0))
    print("mobilenetv3 fp16", shape, flush=True)
    xd = dev(x, abi.F16)
    got = host(g(xd)).reshape(shape[0], 1000)
    want = oracle.mobilenetv3_forward(x, tensors_of(b16))
    err = rel_l2(got, want)
    print("logits rel_l2", err, flush=True)
    assert err < FP16_REL_L2
    assert np.array_equal(got.argmax(1), want.argmax(1))
    # later calls replay a captured HIP graph: every replay must reproduce the eager result, with
    # unrelated eager work and synchronisations in between
    for it in range(4):
        scratch = torch.randn(1 << 20, device="cuda").sum().item()
        again = host(g(xd)).reshape(shape[0], 1000)
        assert np.array_equal(again, got), it
    g.close()


def test_mobilenetv3_through_reference_abi(blob):
    """_mlir_ciface_forward recognises the network by the size of the params memref (host memory in,
    malloc'd [N,1000] out), as a program linked against the object for MobileNetV3.mlir would call it."""
    x = synth.uniform(7402, (1, 3, 256, 256), 0.0, 1.0)
    got = abi.forward(x, blob.copy())
    want = oracle.mobilenetv3_forward(x, tensors_of(blob))
    assert got.shape == (1, 1000)
    assert max_rel(got, want) < FP32_MAX_REL
    assert np.array_equal(got.argmax(1), want.argmax(1))
    # the half-precision symbol takes the same route (all three memrefs hold IEEE half bits)
    b16 = blob.astype(np.float16)
    x16 = x.astype(np.float16)
    got16 = abi.forward(x16, b16)
    want16 = oracle.mobilenetv3_forward(x16.astype(np.float32), tensors_of(b16.astype(np.float32)))
    assert got16.dtype == np.float16 and got16.shape == (1, 1000)
    assert rel_l2(got16.astype(np.float32), want16) < FP16_REL_L2
    assert np.array_equal(got16.argmax(1), want16.argmax(1))


# ---------------------------------------------------------------------------------------------
# executor: the YOLOv5-style operators, and what it refuses
# ---------------------------------------------------------------------------------------------
def small_net(C=16):
    """conv(SiLU) -> [5x5 max-pool x2, concat] -> conv 1x1 -> stride-2 conv -> upsample -> concat with the skip ->
    conv + residual add -> sigmoid: every operator kind the MobileNetV3 list does not use."""
    sizes, ops = [], []

    def take(n):
        off = sum(sizes)
        sizes.append(n)
        return off

    def conv(i, o, cin, F, k, stride, act, res=-1, bias=True, bn=False):
        w = take(F * cin * k * k)
        b = take(F) if bias else -1
        bnp = tuple(take(F) for _ in range(4)) if bn else None
        ops.append(abi.graph_op(abi.OP_CONV, [i, res], o, F=F, K=k, stride=stride, pad=(k - 1) // 2, act=act, eps=1e-3, w=w,
                                bias=b, bn=bnp))

    conv(0, 1, 3, C, 3, 1, abi.ACT_SILU, bn=True)
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [1], 2, K=5, stride=1, pad=2))
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [2], 3, K=5, stride=1, pad=2))
    ops.append(abi.graph_op(abi.OP_CONCAT, [1, 2, 3], 4))
    conv(4, 5, 3 * C, C, 1, 1, abi.ACT_SILU)
    conv(5, 6, C, 2 * C, 3, 2, abi.ACT_SILU, bias=False, bn=True)
    ops.append(abi.graph_op(abi.OP_UPSAMPLE2X, [6], 7))
    ops.append(abi.graph_op(abi.OP_CONCAT, [7, 5], 8))
    conv(8, 9, 3 * C, C, 3, 1, abi.ACT_NONE, res=5)
    ops.append(abi.graph_op(abi.OP_ADD, [9, 1], 10, act=abi.ACT_RELU))
    ops.append(abi.graph_op(abi.OP_ACT, [10], 11, act=abi.ACT_SIGMOID))
    n = sum(sizes)
    blob = synth.normal(7500, (n,), std=0.15)
    for o in ops:  # variances must be positive
        if o.var >= 0:
            blob[o.var:o.var + o.F] = synth.uniform(7501, (o.F,), 0.5, 1.5)
    return ops, blob


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_executor_on_yolo_style_operators(dt):
    ops, blob = small_net()
    x = synth.normal(7502, (2, 3, 20, 12))
    if dt == abi.F16:
        blob, x = r16(blob), r16(x)
    g = Graph(ops, 3, blob, dt)
    assert abi.graph_output_shape(g.h, 20, 12) == (16, 20, 12)
    got = host(g(dev(x, dt)))
    want = oracle.run_graph(ops, x, blob, 3)
    assert got.shape == want.shape
    if dt == abi.F32:
        assert max_rel(got, want) < FP32_MAX_REL
    else:
        assert rel_l2(got, want) < FP16_REL_L2
    # an odd-sized image cannot be up-sampled back onto its skip connection: refused with a message
    out = torch.empty(2 * 16 * 21 * 12, device="cuda")
    assert abi.lib().nncv_hip_graph_forward(g.h, out.data_ptr(), 2, 21, 12, out.data_ptr(), out.numel(), None) != 0
    assert b"different sizes" in abi.lib().nncv_hip_last_error()
    g.close()


def test_graph_create_refuses_malformed_lists():
    ops, blob = small_net()

    def refused(bad, blob=blob, cin=3):
        with pytest.raises(abi.NncvHipError) as e:
            abi.graph_create(bad, cin, blob)
        return str(e.value)

    def clone(i, **kw):
        c = [abi.GraphOp.from_buffer_copy(o) for o in ops]
        for k, v in kw.items():
            setattr(c[i], k, v)
        return c

    assert "defined earlier" in refused(clone(1, inputs=(ctypes.c_int32 * 4)(9, -1, -1, -1)))  # reads a later tensor
    assert "new tensor id" in refused(clone(2, out=2))                                          # writes a tensor twice
    assert "unknown kind" in refused(clone(3, kind=42))
    assert "outside the parameter blob" in refused(clone(4, w=blob.size - 3))
    assert "multiple" in refused(clone(0, F=10))                                                # a max-pool cannot read 10 (stored 12) channels
    assert "K must be 3 or 5" in refused(clone(1, kind=abi.OP_DWCONV, K=7, w=0))
    assert "unknown activation" in refused(clone(10, act=9))
    assert "channel" in refused(clone(8, inputs=(ctypes.c_int32 * 4)(8, 6, -1, -1)))            # residual with 2C channels


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
@pytest.mark.parametrize("C,SQ,H,W,N", [(16, 8, 56, 56, 2), (576, 144, 7, 7, 3), (240, 64, 14, 14, 1), (96, 24, 5, 3, 2)])
def test_squeeze_excitation_block(dt, C, SQ, H, W, N):
    """pool -> fc + ReLU -> fc + hard-sigmoid -> gate, which the executor runs as one launch."""
    sizes, ops = [], []

    def take(n):
        off = sum(sizes)
        sizes.append(n)
        return off

    ops.append(abi.graph_op(abi.OP_ACT, [0], 1, act=abi.ACT_NONE, stride=0))
    ops.append(abi.graph_op(abi.OP_GAVGPOOL, [1], 2, stride=0))
    ops.append(abi.graph_op(abi.OP_CONV, [2], 3, F=SQ, K=1, act=abi.ACT_RELU, w=take(SQ * C), bias=take(SQ)))
    ops.append(abi.graph_op(abi.OP_CONV, [3], 4, F=C, K=1, act=abi.ACT_HARDSIGMOID, w=take(C * SQ), bias=take(C)))
    ops.append(abi.graph_op(abi.OP_SCALE, [1, 4], 5, stride=0))
    blob = synth.normal(7600, (sum(sizes),), std=0.3)
    x = synth.normal(7601, (N, C, H, W))
    if dt == abi.F16:
        blob, x = r16(blob), r16(x)
    g = Graph(ops, C, blob, dt)
    print("se block", dt, C, SQ, H, W, N, flush=True)
    got = host(g(dev(x, dt)))
    want = oracle.run_graph(ops, x, blob, C)
    if dt == abi.F32:
        assert max_rel(got, want) < FP32_MAX_REL
    else:
        assert rel_l2(got, want) < 2e-3
    g.close()


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_resnet18_as_an_operator_list(dt):
    """tests/Nets/Res18.mlir through the generic executor: same logits as the oracle and as the hard-wired model."""
    from nncv_amd import resnet18_spec
    from gpu_util import Model
    blob = synth.resnet18_params()
    x = synth.uniform(7700, (2, 3, 96, 64), 0.0, 1.0)
    if dt == abi.F16:
        blob, x = r16(blob), r16(x)
    g = Graph(resnet18_spec.graph_ops(), 3, blob, dt)
    xd = dev(x, dt)
    got = host(g(xd)).reshape(2, 1000)
    want = oracle.resnet18_forward(x, blob)
    hard = host(Model(blob, dt)(xd))
    if dt == abi.F32:
        assert max_rel(got, want) < FP32_MAX_REL and max_rel(hard, want) < FP32_MAX_REL
    else:
        assert rel_l2(got, want) < FP16_REL_L2 and rel_l2(got, hard) < FP16_REL_L2
    assert np.array_equal(got.argmax(1), want.argmax(1))
    g.close()


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_nested_concatenation_views(dt):
    """Concatenations whose inputs are themselves concatenations, max-pools, adds and activations: tensors living in
    slices of slices, read at a pitch by 3x3 and 1x1 convolutions, against the dense evaluator."""
    sizes, ops = [], []

    def take(n):
        off = sum(sizes)
        sizes.append(n)
        return off

    def conv(i, o, cin, F, k, act=abi.ACT_RELU):
        ops.append(abi.graph_op(abi.OP_CONV, [i], o, F=F, K=k, stride=1, pad=(k - 1) // 2, act=act, w=take(F * cin * k * k), bias=take(F)))

    C = 16
    conv(0, 1, 3, C, 3)                                                   # a
    conv(0, 2, 3, 2 * C, 1, abi.ACT_HARDSWISH)                            # b
    ops.append(abi.graph_op(abi.OP_CONCAT, [1, 2], 3, stride=0))          # c1 = [a, b]            (3C)
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [1], 4, K=3, stride=1, pad=1))  # e = pool(a): reads a inside c1 inside c2
    ops.append(abi.graph_op(abi.OP_ACT, [2], 5, act=abi.ACT_SILU, stride=0))  # f = silu(b)
    ops.append(abi.graph_op(abi.OP_ADD, [4, 1], 6, act=abi.ACT_NONE, stride=0))  # g = e + a
    ops.append(abi.graph_op(abi.OP_CONCAT, [3, 6, 5], 7, stride=0))       # c2 = [c1, g, f]        (3C + C + 2C)
    conv(3, 8, 3 * C, C, 3)                                               # 3x3 over the slice c1 of c2
    conv(7, 9, 6 * C, 2 * C, 1, abi.ACT_NONE)                             # 1x1 over all of c2
    ops.append(abi.graph_op(abi.OP_CONCAT, [8, 9], 10, stride=0))         # output [C + 2C]
    blob = synth.normal(7800, (sum(sizes),), std=0.2)
    x = synth.normal(7801, (2, 3, 11, 14))
    if dt == abi.F16:
        blob, x = r16(blob), r16(x)
    g = Graph(ops, 3, blob, dt)
    assert abi.graph_output_shape(g.h, 11, 14) == (3 * C, 11, 14)
    got = host(g(dev(x, dt)))
    want = oracle.run_graph(ops, x, blob, 3)
    if dt == abi.F32:
        assert max_rel(got, want) < FP32_MAX_REL
    else:
        assert rel_l2(got, want) < FP16_REL_L2
    g.close()


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_random_operator_lists(dt):
    """40 seeded random graphs per element type against the evaluator (tests/graph_gen.py)."""
    from graph_gen import random_case
    f16 = dt == abi.F16
    done = 0
    for seed in range(5000, 5040):
        case = random_case(seed, f16)
        if case is None:
            continue
        ops, cin, blob, x = case
        print("seed", seed, "kinds", [int(o.kind) for o in ops], "input", x.shape, flush=True)
        g = Graph(ops, cin, blob, dt)
        got = host(g(dev(x, dt)))
        want = oracle.run_graph(ops, x, blob, cin)
        g.close()
        assert got.shape == want.shape and np.array_equal(np.isnan(got), np.isnan(want)), seed
        fin = np.isfinite(want) & np.isfinite(got)
        if fin.any():
            err = rel_l2(got[fin], want[fin]) if f16 else max_rel(got[fin], want[fin])
            assert err < (FP16_REL_L2 if f16 else FP32_MAX_REL), (seed, err)
        done += 1
    assert done >= 30


@pytest.mark.parametrize("k,pad,F,act,shape", [
    (6, 2, 32, abi.ACT_SILU, (2, 3, 64, 96)),         # YOLOv5s' first layer
    (6, 2, 32, abi.ACT_SILU, (1, 3, 38, 50)),         # pixel count not a multiple of the 256-pixel tile
    (6, 2, 64, abi.ACT_RELU, (3, 3, 20, 18)),         # two 32-filter halves per wave
    (6, 2, 48, abi.ACT_NONE, (1, 3, 16, 16)),         # filters that end inside the second half
    (3, 1, 16, abi.ACT_HARDSWISH, (2, 3, 64, 64)),    # MobileNetV3's first layer (half of the 32-filter block is padding)
    (3, 1, 24, abi.ACT_RELU, (1, 3, 33, 46)),         # odd height
    (3, 1, 64, abi.ACT_SILU, (2, 4, 12, 34)),         # four input channels
    (3, 1, 8, abi.ACT_NONE, (1, 1, 9, 10)),           # one input channel
])
def test_fp16_image_convolution_over_pixel_pairs(k, pad, F, act, shape):
    """A stride-2 convolution that is the only reader of an image with at most four channels and an even
    width runs over pixel pairs; 6x6 pad 2 and 3x3 pad 1 windows take the kernel that loads the whole K
    axis at once (`conv_pairs`).  One-operator graphs against the evaluator, with the route checked."""
    N, C, H, W = shape
    w = synth.normal(7900 + k, (F, C, k, k), std=float(np.sqrt(2.0 / (C * k * k))))
    bnp = (synth.uniform(7902, (F,), 0.5, 1.5), synth.normal(7903, (F,), std=0.1), synth.normal(7904, (F,), std=0.1),
           synth.uniform(7905, (F,), 0.5, 1.5))
    blob = r16(np.concatenate([w.ravel()] + list(bnp)))
    o = F * C * k * k
    ops = [abi.graph_op(abi.OP_CONV, [0, -1], 1, F=F, K=k, stride=2, pad=pad, act=act, eps=1e-3, w=0,
                        bn=(o, o + F, o + 2 * F, o + 3 * F))]
    x = r16(synth.uniform(7906, shape, -1.0, 1.0))
    print("pair stem", k, pad, F, act, shape, flush=True)
    g = Graph(ops, C, blob, abi.F16)
    abi.profile_enable(True)
    abi.profile_report()
    got = host(g(dev(x, abi.F16)))
    tags = abi.profile_report()
    abi.profile_enable(False)
    want = oracle.run_graph(ops, x, blob, C)
    g.close()
    assert any(t.startswith("conv_pairs<f16,%s" % ("6x3" if k == 6 else "3x2")) for t in tags), sorted(tags)
    assert got.shape == want.shape
    assert rel_l2(got, want) < 2e-3  # one layer: only the rounding of the result to half
    assert np.abs(got - want).max() < 2e-2 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
@pytest.mark.parametrize("shape,concat", [((2, 3, 20, 20), True), ((3, 3, 7, 13), True), ((1, 3, 40, 40), False), ((1, 3, 41, 40), True)])
def test_three_chained_5x5_max_pools_run_as_one_launch(dt, shape, concat):
    """SPPF: y1 = m(x), y2 = m(y1), y3 = m(y2), concatenated with x (or only y3 kept).  Maps of at most 1600 pixels take
    the fused kernel, larger ones three launches; both must equal the evaluator exactly (max of copies of the input)."""
    C = 16
    sizes, ops = [], []

    def take(n):
        off = sum(sizes)
        sizes.append(n)
        return off

    w = take(C * 3)
    ops.append(abi.graph_op(abi.OP_CONV, [0, -1], 1, F=C, K=1, stride=1, pad=0, act=abi.ACT_NONE, w=w, bias=take(C)))
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [1], 2, K=5, stride=1, pad=2))
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [2], 3, K=5, stride=1, pad=2))
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [3], 4, K=5, stride=1, pad=2))
    if concat:
        ops.append(abi.graph_op(abi.OP_CONCAT, [1, 2, 3, 4], 5))
    blob = synth.normal(7950, (sum(sizes),), std=0.5)
    x = synth.normal(7951, shape)
    if dt == abi.F16:
        blob, x = r16(blob), r16(x)
    g = Graph(ops, 3, blob, dt)
    abi.profile_enable(True)
    abi.profile_report()
    got = host(g(dev(x, dt)))
    tags = abi.profile_report()
    abi.profile_enable(False)
    want = oracle.run_graph(ops, x, blob, 3)
    fused = shape[2] * shape[3] <= 1600
    assert ("maxpool5_chain3" in tags) == fused and ("maxpool" in tags) == (not fused), sorted(tags)
    assert got.shape == want.shape
    if dt == abi.F32:
        assert max_rel(got, want) < FP32_MAX_REL
    else:
        assert rel_l2(got, want) < 2e-3
    # the pools themselves are exact: every pooled channel must be the maximum of the unpooled ones it covers
    if concat:
        y0, y1 = got[:, :C], got[:, C:2 * C]
        assert np.array_equal(y1, oracle.maxpool_nchw(y0, 5, 1, 2))
        assert np.array_equal(got[:, 2 * C:3 * C], oracle.maxpool_nchw(y1, 5, 1, 2))
        assert np.array_equal(got[:, 3 * C:], oracle.maxpool_nchw(got[:, 2 * C:3 * C], 5, 1, 2))
    # replays of the captured graph reproduce the eager result
    xd = dev(x, dt)
    first = host(g(xd))
    for it in range(3):
        assert np.array_equal(host(g(xd)), first), it
    g.close()


def test_two_graph_handles_on_two_streams_stay_exact():
    """Operator-list handles own their workspace like the ResNet-18 ones: two handles of the same network fed
    alternately on two caller streams, nothing ordering them, each reproduce the bits of a pass run alone; one handle
    on two streams is ordered by the library."""
    ops, blob = small_net()
    blob = r16(blob)
    xa, xb = r16(synth.normal(7601, (4, 3, 40, 24))), r16(synth.normal(7602, (4, 3, 40, 24)))
    ga, gb = Graph(ops, 3, blob, abi.F16), Graph(ops, 3, blob, abi.F16)
    xda, xdb = dev(xa, abi.F16), dev(xb, abi.F16)
    want_a, want_b = host(ga(xda)), host(gb(xdb))
    assert rel_l2(want_a, oracle.run_graph(ops, xa, blob, 3)) < FP16_REL_L2
    n = want_a.size
    oa, ob = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    L = abi.lib()
    torch.cuda.synchronize()
    for it in range(6):
        abi.check(L.nncv_hip_graph_forward(ga.h, xda.data_ptr(), 4, 40, 24, oa.data_ptr(), n, s1.cuda_stream))
        abi.check(L.nncv_hip_graph_forward(gb.h, xdb.data_ptr(), 4, 40, 24, ob.data_ptr(), n, s2.cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(oa.cpu().numpy().reshape(want_a.shape), want_a)
    assert np.array_equal(ob.cpu().numpy().reshape(want_b.shape), want_b)
    # one handle, two streams, two inputs: the second call waits for the first
    for it in range(4):
        abi.check(L.nncv_hip_graph_forward(ga.h, xda.data_ptr(), 4, 40, 24, oa.data_ptr(), n, s1.cuda_stream))
        abi.check(L.nncv_hip_graph_forward(ga.h, xdb.data_ptr(), 4, 40, 24, ob.data_ptr(), n, s2.cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(oa.cpu().numpy().reshape(want_a.shape), want_a)
    assert np.array_equal(ob.cpu().numpy().reshape(want_b.shape), host(ga(xdb)))
    ga.close()
    gb.close()
