"""ctypes front end of the CPU checker (oracle/nncv_oracle.c).

TEST INFRASTRUCTURE ONLY.  May be imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py — never by nncv_amd/ (the product fails loudly without its HIP
library instead of falling back to this).

Besides the C functions (pinning status in the header of nncv_oracle.c) this module restates in
numpy the operators of the reference's other network fixtures; what pins each:
  depthwise_conv2d_nchw_chw, batchnorm_eps, hardswish, hardsigmoid, silu, sigmoid, maxpool_nchw,
  upsample2x_nearest   torch CPU library routines in float64 (conv2d groups=C, batch_norm,
                       hardswish, hardsigmoid, silu, max_pool2d, interpolate), closed forms at the knees
                       and special values, a deliberately transposed filter that must fail
                       (tests/test_oracle_mobilenetv3.py)
  mobilenetv3_forward  a float64 torch composition of torchvision's mobilenet_v3_small.forward, block
                       by block; the tensor table against the fixture's 52 convolution shapes, its 210
                       constants and the published parameter count (same file)
  yolo_detect          closed forms on non-square grids (cell centres / anchors at sigmoid 0.5, the
                       extremes, one-hot channel placement) (tests/test_oracle_yolov5s.py)
  run_graph            reproduces the C ResNet-18 oracle over resnet18_spec.graph_ops()
                       (tests/test_oracle_resnet18.py), mobilenetv3_forward, and a float64 torch
                       composition of YOLOv5s whose 60 convolution shapes and 13 concatenations are
                       checked, in order, against tests/Nets/Yolov5s.mlir
  preprocess_u8, top1_scan, hwp_*   tests/test_oracle_ops.py
Parity unpinned, as for the C part: the exact fp32 summation order of the reference's compiled
object (it cannot be built here); the restatements keep the fixtures' operation order.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_HWP = None
_REF = None

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
_int = ctypes.c_int
_i64 = ctypes.c_int64


def build(force=False):
    """Compile the checker with the Makefile beside this file."""
    if force or not os.path.exists(os.path.join(_HERE, "liboracle.so")) \
            or not os.path.exists(os.path.join(_HERE, "libhostwparallel.so")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])


def lib():
    global _LIB
    if _LIB is None:
        build()
        L = ctypes.CDLL(os.path.join(_HERE, "liboracle.so"))
        L.orc_conv2d_nchw_fchw.argtypes = [_f32p, _f32p, _f32p] + [_int] * 9
        L.orc_matmul.argtypes = [_f32p, _f32p, _f32p, _int, _int, _int]
        L.orc_pad_nchw.argtypes = [_f32p, _f32p, _int, _int, _int, _int, _int, ctypes.c_float]
        L.orc_batchnorm_nchw.argtypes = [_f32p] * 6 + [_int] * 3
        L.orc_relu.argtypes = [_f32p, _f32p, _i64]
        L.orc_add.argtypes = [_f32p, _f32p, _f32p, _i64]
        L.orc_maxpool_nchw.argtypes = [_f32p, _f32p] + [_int] * 8
        L.orc_global_avgpool_nchw.argtypes = [_f32p, _f32p] + [_int] * 4
        L.orc_fc.argtypes = [_f32p] * 4 + [_int] * 3
        L.orc_wino43_filter_transform.argtypes = [_f32p, _f64p, _int, _int]
        L.orc_wino43_input_transform.argtypes = [_f32p, _f64p] + [_int] * 5
        L.orc_wino43_batched_gemm.argtypes = [_f64p, _f64p, _f64p, _i64, _int, _int]
        L.orc_wino43_output_transform.argtypes = [_f64p, _f32p] + [_int] * 4
        L.orc_conv3x3_winograd43.argtypes = [_f32p, _f32p, _f32p] + [_int] * 6
        L.orc_resnet18_forward.argtypes = [_f32p, _int, _int, _int, _f32p, _f32p, _int,
                                           ctypes.c_void_p]
        L.orc_resnet18_forward.restype = _int
        L.orc_resnet18_num_params.restype = _i64
        _LIB = L
    return _LIB


def _c(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def conv2d_nchw_fchw(x_padded, w, stride=1, out=None):
    """out + conv(x_padded, w); x is already padded (linalg.conv_2d_nchw_fchw)."""
    x_padded, w = _c(x_padded), _c(w)
    N, C, H, W = x_padded.shape
    F, C2, R, S = w.shape
    assert C == C2
    OH, OW = (H - R) // stride + 1, (W - S) // stride + 1
    y = np.zeros((N, F, OH, OW), np.float32) if out is None else _c(out).copy()
    assert y.shape == (N, F, OH, OW)
    lib().orc_conv2d_nchw_fchw(x_padded, w, y, N, C, H, W, F, R, S, stride, stride)
    return y


def pad_nchw(x, pad, value=0.0):
    x = _c(x)
    N, C, H, W = x.shape
    y = np.empty((N, C, H + 2 * pad, W + 2 * pad), np.float32)
    lib().orc_pad_nchw(x, y, N, C, H, W, pad, value)
    return y


def matmul(a, b, c=None):
    a, b = _c(a), _c(b)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    y = np.zeros((M, N), np.float32) if c is None else _c(c).copy()
    lib().orc_matmul(a, b, y, M, N, K)
    return y


def batchnorm(x, gamma, beta, mean, var):
    x = _c(x)
    N, C = x.shape[:2]
    y = np.empty_like(x)
    lib().orc_batchnorm_nchw(x, _c(gamma), _c(beta), _c(mean), _c(var), y, N, C,
                             int(np.prod(x.shape[2:])))
    return y


def relu(x):
    x = _c(x)
    y = np.empty_like(x)
    lib().orc_relu(x, y, x.size)
    return y


def maxpool3x3s2(x):
    """-inf pad 1, 3x3 window, stride 2 (Res18.mlir:144-151)."""
    xp = pad_nchw(x, 1, -np.inf)
    N, C, H, W = xp.shape
    OH, OW = (H - 3) // 2 + 1, (W - 3) // 2 + 1
    y = np.full((N, C, OH, OW), -np.inf, np.float32)
    lib().orc_maxpool_nchw(xp, y, N, C, H, W, 3, 3, 2, 2)
    return y


def global_avgpool(x):
    x = _c(x)
    N, C, H, W = x.shape
    y = np.empty((N, C), np.float32)
    lib().orc_global_avgpool_nchw(x, y, N, C, H, W)
    return y


def fc(x, w, b):
    x, w, b = _c(x), _c(w), _c(b)
    y = np.empty((x.shape[0], w.shape[0]), np.float32)
    lib().orc_fc(x, w, b, y, x.shape[0], x.shape[1], w.shape[0])
    return y


def wino43_filter_transform(w):
    w = _c(w)
    F, C = w.shape[:2]
    U = np.empty((36, F, C), np.float64)
    lib().orc_wino43_filter_transform(w, U, F, C)
    return U


def wino43_input_transform(x, pad=1):
    x = _c(x)
    N, C, H, W = x.shape
    OH, OW = H + 2 * pad - 2, W + 2 * pad - 2
    tiles = N * ((OH + 3) // 4) * ((OW + 3) // 4)
    V = np.empty((36, tiles, C), np.float64)
    lib().orc_wino43_input_transform(x, V, N, C, H, W, pad)
    return V


def wino43_batched_gemm(V, U):
    tiles, C = V.shape[1:]
    F = U.shape[1]
    M = np.empty((36, tiles, F), np.float64)
    lib().orc_wino43_batched_gemm(np.ascontiguousarray(V), np.ascontiguousarray(U), M, tiles, C, F)
    return M


def wino43_output_transform(M, N, OH, OW, out=None):
    F = M.shape[2]
    y = np.zeros((N, F, OH, OW), np.float32) if out is None else _c(out).copy()
    lib().orc_wino43_output_transform(np.ascontiguousarray(M), y, N, F, OH, OW)
    return y


def conv3x3_winograd43(x, w, pad=1):
    x, w = _c(x), _c(w)
    N, C, H, W = x.shape
    F = w.shape[0]
    y = np.zeros((N, F, H + 2 * pad - 2, W + 2 * pad - 2), np.float32)
    lib().orc_conv3x3_winograd43(x, w, y, N, C, H, W, F, pad)
    return y


def resnet18_forward(x, params, tap_layer=-1):
    """x [N,3,H,W] fp32, params flat fp32 blob (canonical order) -> logits [N,1000]
    (and the tapped NCHW activation when tap_layer >= 0)."""
    x, params = _c(x), _c(params)
    N, C, H, W = x.shape
    assert C == 3 and params.size == lib().orc_resnet18_num_params()
    y = np.empty((N, 1000), np.float32)
    tap = None
    tp = None
    if tap_layer >= 0:
        ch = [64, 64, 128, 256, 512][tap_layer]
        down = lambda v: (v - 1) // 2 + 1  # every stride-2 stage (7x7 p3, 3x3 p1): ceil(v / 2)
        h, w = down(down(H)), down(down(W))
        for _ in range(max(0, tap_layer - 1)):
            h, w = down(h), down(w)
        tap = np.empty((N, ch, h, w), np.float32)
        tp = tap.ctypes.data_as(ctypes.c_void_p)
    rc = lib().orc_resnet18_forward(x, N, H, W, params, y, tap_layer, tp)
    assert rc == 0
    return (y, tap) if tap_layer >= 0 else y


# ---- operators of tests/Nets/MobileNetV3.mlir and Yolov5s.mlir, numpy (fp32 like the fixtures) ----
def batchnorm_eps(x, gamma, beta, mean, var, eps):
    """(x - mean) * rsqrt(var + f32(eps)) * gamma + beta, op by op (MobileNetV3.mlir:249-258)."""
    x = _c(x)
    sh = (1, -1) + (1,) * (x.ndim - 2)
    r = (np.float32(1.0) / np.sqrt(_c(var) + np.float32(eps))).astype(np.float32)
    return (((x - _c(mean).reshape(sh)) * r.reshape(sh)) * _c(gamma).reshape(sh) + _c(beta).reshape(sh)).astype(np.float32)


def depthwise_conv2d_nchw_chw(x_padded, w, stride=1):
    """linalg.depthwise_conv_2d_nchw_chw (MobileNetV3.mlir:290): out[n,c,oh,ow] += x[n,c,oh*s+kh,ow*s+kw] * w[c,kh,kw],
    accumulated over (kh, kw) in loop order, separate multiply and add."""
    x_padded, w = _c(x_padded), _c(w)
    N, C, H, W = x_padded.shape
    if w.ndim == 4:
        w = w.reshape(w.shape[0], w.shape[2], w.shape[3])  # tensor.collapse_shape of [C,1,K,K] (:289)
    assert w.shape[0] == C
    K1, K2 = w.shape[1:]
    OH, OW = (H - K1) // stride + 1, (W - K2) // stride + 1
    y = np.zeros((N, C, OH, OW), np.float32)
    for kh in range(K1):
        for kw in range(K2):
            win = x_padded[:, :, kh:kh + stride * (OH - 1) + 1:stride, kw:kw + stride * (OW - 1) + 1:stride]
            y = y + win * w[None, :, kh, kw, None, None]
    return y


def hardswish(x):
    """(min(relu_ugt(x + 3), 6) / 6) * x, the generics of MobileNetV3.mlir:259-293; the min is `olt` + select."""
    x = _c(x)
    t = relu(x + np.float32(3.0))
    t = np.where(t < np.float32(6.0), t, np.float32(6.0)).astype(np.float32)
    return ((t / np.float32(6.0)) * x).astype(np.float32)


def hardsigmoid(x):
    """max(0, min(1, (x + 3) / 6)) as MobileNetV3.mlir:349-379 spells it: olt(1, t) ? 1 : t, then ogt(0, m) ? 0 : m."""
    x = _c(x)
    t = ((x + np.float32(3.0)) / np.float32(6.0)).astype(np.float32)
    m = np.where(np.float32(1.0) < t, np.float32(1.0), t)
    return np.where(np.float32(0.0) > m, np.float32(0.0), m).astype(np.float32)


def sigmoid(x):
    """1 / (exp(-x) + 1)  (Yolov5s.mlir:158-165)"""
    x = _c(x)
    return (np.float32(1.0) / (np.exp(-x) + np.float32(1.0))).astype(np.float32)


def silu(x):
    """sigmoid(x) * x  (Yolov5s.mlir:158-171)"""
    return (sigmoid(x) * _c(x)).astype(np.float32)


ACTIVATIONS = {0: _c, 1: relu, 2: hardswish, 3: hardsigmoid, 4: silu, 5: sigmoid}


def maxpool_nchw(x, k, stride, pad):
    """linalg.pooling_nchw_max over a -inf halo (Yolov5s.mlir SPPF: 5x5 stride 1 pad 2)."""
    xp = pad_nchw(x, pad, -np.inf) if pad else _c(x)
    N, C, H, W = xp.shape
    OH, OW = (H - k) // stride + 1, (W - k) // stride + 1
    y = np.full((N, C, OH, OW), -np.inf, np.float32)
    lib().orc_maxpool_nchw(xp, y, N, C, H, W, k, k, stride, stride)
    return y


def upsample2x_nearest(x):
    """out[n,c,y,x] = in[n,c,y // 2,x // 2]  (the index arithmetic + tensor.extract generics of Yolov5s.mlir)"""
    return _c(x).repeat(2, axis=2).repeat(2, axis=3)


def yolo_detect(heads, anchors, strides, A, F):
    """YOLOv5 Detect decode as Yolov5s.mlir:1348-1448 (and :1449-1662 for the other levels) spells it.
    heads: NCHW [N, A*F, H_l, W_l] per level; anchors [L, A, 2] in units of the stride; strides [L]
    -> [N, sum_l A*H_l*W_l, F], boxes ordered (level, anchor, y, x)."""
    anchors, strides = _c(anchors), _c(strides)
    outs = []
    for l, h in enumerate(heads):
        h = _c(h)
        N, _, H, W = h.shape
        p = h.reshape(N, A, F, H, W).transpose(0, 1, 3, 4, 2)            # expand_shape + permuting generic
        s = sigmoid(p)
        gx = np.arange(W, dtype=np.float32) + np.float32(0.0)             # linalg.index + 0 (:1358-1366)
        gy = np.arange(H, dtype=np.float32) + np.float32(0.0)
        grid = np.stack(np.broadcast_arrays(gx[None, :], gy[:, None]), axis=-1) - np.float32(0.5)  # (x, y) - 0.5
        ag = (anchors[l] * strides[l]).astype(np.float32).reshape(1, A, 1, 1, 2)                    # anchors * stride
        xy = ((s[..., 0:2] * np.float32(2.0) + grid.reshape(1, 1, H, W, 2)) * strides[l]).astype(np.float32)
        wh = (np.power(s[..., 2:4] * np.float32(2.0), np.float32(2.0)) * ag).astype(np.float32)     # math.powf(., 2)
        outs.append(np.concatenate([xy, wh, s[..., 4:]], axis=-1).reshape(N, A * H * W, F))
    return np.concatenate(outs, axis=1)


def mobilenetv3_forward(x, tensors, taps=None):
    """MobileNetV3-small as tests/Nets/MobileNetV3.mlir computes it.  x [N,3,H,W] fp32; tensors: {name: ndarray} with
    torchvision state_dict names (nncv_amd.mobilenetv3_spec.tensor_table) -> logits [N,1000].
    `taps`, when a list, receives the NCHW output of every bottleneck block."""
    from nncv_amd import mobilenetv3_spec as spec
    T = tensors
    eps = spec.BN_EPS

    def bn(y, p):
        return batchnorm_eps(y, T[p + ".weight"], T[p + ".bias"], T[p + ".running_mean"], T[p + ".running_var"], eps)

    def conv(y, name, stride=1, pad=0):
        return conv2d_nchw_fchw(pad_nchw(y, pad) if pad else y, T[name + ".weight"], stride)

    def conv_bias(y, name):  # the bias initialises the accumulator (:331-335)
        w = _c(T[name + ".weight"])
        w = w.reshape(w.shape[0], w.shape[1], 1, 1)
        init = np.broadcast_to(_c(T[name + ".bias"]).reshape(1, -1, 1, 1), (y.shape[0], w.shape[0], 1, 1))
        return conv2d_nchw_fchw(y, w, 1, out=init)

    y = hardswish(bn(conv(x, "features.0.0", 2, 1), "features.0.1"))
    for i, (cin, k, exp, cout, se, hs, stride) in enumerate(spec.BNECK, start=1):
        p = "features.%d.block" % i
        act = hardswish if hs else relu
        block_in, j = y, 0
        if exp != cin:
            y = act(bn(conv(y, "%s.%d.0" % (p, j)), "%s.%d.1" % (p, j)))
            j += 1
        y = act(bn(depthwise_conv2d_nchw_chw(pad_nchw(y, (k - 1) // 2), T["%s.%d.0.weight" % (p, j)], stride), "%s.%d.1" % (p, j)))
        j += 1
        if se:
            N, C, H, W = y.shape
            g = global_avgpool(y).reshape(N, C, 1, 1)  # pooling_nchw_sum, then one divf by H*W (:322-328)
            g = relu(conv_bias(g, "%s.%d.fc1" % (p, j)))
            g = hardsigmoid(conv_bias(g, "%s.%d.fc2" % (p, j)))
            y = (g * y).astype(np.float32)
            j += 1
        y = bn(conv(y, "%s.%d.0" % (p, j)), "%s.%d.1" % (p, j))
        if stride == 1 and cin == cout:
            y = (y + block_in).astype(np.float32)
        if taps is not None:
            taps.append(y)
    y = hardswish(bn(conv(y, "features.12.0"), "features.12.1"))
    N, C = y.shape[:2]
    y = global_avgpool(y)
    y = hardswish(fc(y, T["classifier.0.weight"], T["classifier.0.bias"]))
    return fc(y, T["classifier.3.weight"], T["classifier.3.bias"])


def run_graph(ops, x, blob, in_channels, conv=None):
    """Evaluates a list of nncv_hip_graph_op-like records (attributes kind, inputs, out, F, K, stride, pad, act, eps,
    w, bias, gamma, beta, mean, var) with the operator restatements above; NCHW fp32.  Checker for the graph executor.  `conv(x, w, stride, pad)`
    replaces the scalar convolution (e.g. hwp_conv2d, the OpenMP x AVX2 restatement, for large images)."""
    blob = _c(blob)
    if conv is None:
        conv = lambda a, w, stride, pad: conv2d_nchw_fchw(pad_nchw(a, pad) if pad else a, w, stride)
    vals = {0: _c(x)}
    for o in ops:
        ins = [t for t in o.inputs if t >= 0]
        a = vals[ins[0]]
        act = ACTIVATIONS[o.act]
        if o.kind in (1, 2):
            C = a.shape[1]
            if o.kind == 1:
                F = o.F
                w = blob[o.w:o.w + F * C * o.K * o.K].reshape(F, C, o.K, o.K)
                y = conv(a, w, o.stride, o.pad)
            else:
                F = C
                w = blob[o.w:o.w + C * o.K * o.K].reshape(C, o.K, o.K)
                y = depthwise_conv2d_nchw_chw(pad_nchw(a, o.pad) if o.pad else a, w, o.stride)
            if o.bias >= 0:
                y = (y + blob[o.bias:o.bias + F].reshape(1, F, 1, 1)).astype(np.float32)
            if o.gamma >= 0:
                y = batchnorm_eps(y, blob[o.gamma:o.gamma + F], blob[o.beta:o.beta + F], blob[o.mean:o.mean + F],
                                  blob[o.var:o.var + F], o.eps)
            if o.kind == 1 and len(ins) > 1:
                y = (y + vals[ins[1]]).astype(np.float32)
            y = act(y)
        elif o.kind == 3:
            y = maxpool_nchw(a, o.K, o.stride, o.pad)
        elif o.kind == 4:
            y = global_avgpool(a).reshape(a.shape[0], a.shape[1], 1, 1)
        elif o.kind == 5:
            y = (vals[ins[1]] * a).astype(np.float32)
        elif o.kind == 6:
            y = act((a + vals[ins[1]]).astype(np.float32))
        elif o.kind == 7:
            y = act(a)
        elif o.kind == 8:
            y = np.concatenate([vals[t] for t in ins], axis=1)
        elif o.kind == 9:
            y = upsample2x_nearest(a)
        elif o.kind == 10:
            L = len(ins)
            y = yolo_detect([vals[t] for t in ins], blob[o.w:o.w + L * o.K * 2].reshape(L, o.K, 2), blob[o.bias:o.bias + L], o.K, o.F)
        else:
            raise ValueError("unknown operator kind %d" % o.kind)
        vals[o.out] = _c(y)
    return vals[ops[-1].out]


# ---- the reference driver's pre- and post-processing (examples/Res18/main.cpp), numpy ----
def preprocess_u8(img_hwc):
    """[N,H,W,ch>=3] uint8 -> [N,3,H,W] fp32: x = ((u8 / 255.f) - mean[c]) / std[c], every step in
    fp32 in the driver's order (main.cpp:38 `(float)data[i] / 255.f`, :57-77 `(v - mean) / std`)."""
    img = np.asarray(img_hwc)
    assert img.dtype == np.uint8 and img.ndim == 4 and img.shape[3] >= 3
    mean = np.array([0.485, 0.456, 0.406], np.float32)
    std = np.array([0.229, 0.224, 0.225], np.float32)
    v = img[..., :3].astype(np.float32) / np.float32(255.0)
    v = (v - mean) / std
    return np.ascontiguousarray(v.transpose(0, 3, 1, 2)).astype(np.float32)


def top1_scan(logits):
    """The driver's scan (main.cpp:103-111): max = -100.f; idx = 0; strict `>` left to right."""
    out = []
    for row in np.asarray(logits, np.float32):
        best, idx = np.float32(-100.0), 0
        for i, v in enumerate(row):
            if v > best:
                best, idx = v, i
        out.append(idx)
    return np.array(out, np.int32)


# ---- AVX2/OpenMP restatement of the HostWParallel schedule (hostwparallel.cpp): the timed CPU baseline ----
_HWP = None


def hwp_lib():
    global _HWP
    if _HWP is None:
        p = os.path.join(_HERE, "libhostwparallel.so")
        if not os.path.exists(p):
            raise RuntimeError("%s is missing: run `make -C oracle`" % p)
        L = ctypes.CDLL(p)
        L.hwp_conv2d_nchw_fchw.argtypes = [_f32p, _f32p, _f32p] + [ctypes.c_int] * 9
        L.hwp_conv2d_ref_schedule.argtypes = [_f32p, _f32p, _f32p] + [ctypes.c_int] * 9
        L.hwp_set_num_threads.argtypes = [ctypes.c_int]
        L.hwp_set_num_threads.restype = None
        _HWP = L
    return _HWP


def hwp_threads(n=None):
    """Threads the OpenMP x AVX2 restatement uses; n sets it for the calls that follow."""
    if n is not None:
        hwp_lib().hwp_set_num_threads(int(n))
    return int(hwp_lib().hwp_num_threads())


def hwp_conv2d(x, w, stride=1, pad=0, schedule="omp"):
    """conv_2d_nchw_fchw over a zero halo of `pad`, fp32 accumulation.  schedule "omp": this repository's own OpenMP x
    AVX2 routine; "ref": the reference's tile order, sequential (ModernTile.cpp:184-199, :330-331)."""
    x, w = _c(x), _c(w)
    N, C, H, W = x.shape
    F, C2, R, S = w.shape
    assert C == C2
    OH, OW = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    y = np.empty((N, F, OH, OW), np.float32)
    fn = hwp_lib().hwp_conv2d_nchw_fchw if schedule == "omp" else hwp_lib().hwp_conv2d_ref_schedule
    rc = fn(x, w, y, N, C, H, W, F, R, S, stride, pad)
    assert rc == 0
    return y


def hwp_resnet18_forward(x, params, schedule="omp"):
    """ResNet-18 of tests/Nets/Res18.mlir with the convolutions on one of the AVX2 routines above (`schedule` as in
    hwp_conv2d) and every other op on the scalar oracle's; same parameter blob order as resnet18_forward."""
    import functools
    hwp_conv2d = functools.partial(globals()["hwp_conv2d"], schedule=schedule)
    from nncv_amd import resnet18_spec as spec
    x, params = _c(x), _c(params)
    tensors, off = {}, 0
    for name, shape in spec.tensor_table():
        n = spec.numel(shape)
        tensors[name] = params[off:off + n].reshape(shape)
        off += n
    assert off == params.size

    def bn(y, prefix):
        return batchnorm(y, tensors[prefix + ".weight"], tensors[prefix + ".bias"], tensors[prefix + ".running_mean"],
                         tensors[prefix + ".running_var"])

    y = relu(bn(hwp_conv2d(x, tensors["conv1.weight"], 2, 3), "bn1"))
    y = maxpool3x3s2(y)
    cin = 64
    for li, f in enumerate(spec.WIDTHS, start=1):
        for blk in range(2):
            p = "layer%d.%d" % (li, blk)
            stride = 2 if (li > 1 and blk == 0) else 1
            t = relu(bn(hwp_conv2d(y, tensors[p + ".conv1.weight"], stride, 1), p + ".bn1"))
            t = bn(hwp_conv2d(t, tensors[p + ".conv2.weight"], 1, 1), p + ".bn2")
            idn = y
            if stride != 1 or cin != f:
                idn = bn(hwp_conv2d(y, tensors[p + ".downsample.0.weight"], stride, 0), p + ".downsample.1")
            y = relu(t + idn)
            cin = f
    return fc(global_avgpool(y), tensors["fc.weight"], tensors["fc.bias"])


# ---- reference-built model.bin reader/writer (oracle/_ref), present only where it was built ----
def ref_lib():
    global _REF
    if _REF is None:
        p = os.path.join(_HERE, "_ref", "libnncv_rt_ref.so")
        if not os.path.exists(p):
            return None
        R = ctypes.CDLL(p)
        R.ref_modelbin_read_f32.restype = ctypes.c_longlong
        R.ref_modelbin_read_f32.argtypes = [ctypes.c_char_p, _f32p, ctypes.c_longlong]
        R.ref_sizeof_descriptor.restype = ctypes.c_size_t
        R.ref_sizeof_indexer.restype = ctypes.c_size_t
        R.ref_sizeof_head.restype = ctypes.c_size_t
        _REF = R
    return _REF


def ref_modelbin_write_f32(path, tensors):
    """tensors: list of (name, ndarray fp32).  Uses the reference's own writer."""
    R = ref_lib()
    n = len(tensors)
    names = (ctypes.c_char_p * n)(*[t[0].encode() for t in tensors])
    dims = (ctypes.c_size_t * n)(*[t[1].ndim for t in tensors])
    shapes = (ctypes.c_size_t * (8 * n))()
    arrs = [np.ascontiguousarray(t[1], np.float32) for t in tensors]
    for i, a in enumerate(arrs):
        for d, s in enumerate(a.shape):
            shapes[i * 8 + d] = s
    ptrs = (ctypes.POINTER(ctypes.c_float) * n)(
        *[a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)) for a in arrs])
    return R.ref_modelbin_write_f32(path.encode(), n, names, dims, shapes, ptrs)


def ref_modelbin_read_f32(path, cap):
    R = ref_lib()
    out = np.zeros(cap, np.float32)
    n = R.ref_modelbin_read_f32(path.encode(), out, cap)
    return n, out
