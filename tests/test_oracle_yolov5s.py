"""YOLOv5s table and the Detect decode of the oracle: structure against the reference's fixture
tests/Nets/Yolov5s.mlir, the published parameter count, closed forms of the decode, and the
operator-list evaluator against a float64 torch composition of the network."""
import os
import re

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from nncv_amd import abi, synth
from nncv_amd import yolov5s_spec as spec

FIXTURE = "/root/reference/tests/Nets/Yolov5s.mlir"


def test_tensor_table_counts():
    t = spec.tensor_table()
    assert len(t) == spec.NUM_TENSORS == 122
    assert len(set(n for n, _ in t)) == 122
    assert sum(spec.numel(s) for _, s in t) == spec.NUM_ELEMENTS
    # ultralytics' model summary for yolov5s: 7 225 885 parameters (anchors and strides are buffers)
    assert spec.NUM_ELEMENTS - 18 - 3 == 7225885
    assert abs(spec.flops_per_image(640) / 1e9 - 16.4) < 0.1  # published: 16.4-16.5 GFLOPs at 640
    ops = spec.graph_ops()
    assert sum(1 for o in ops if o.kind == abi.OP_CONV) == 60
    assert sum(1 for o in ops if o.kind == abi.OP_CONCAT) == 13
    assert sum(1 for o in ops if o.kind == abi.OP_ADD) == 7
    # every parameter is referenced exactly once
    used = sorted([o.w for o in ops if o.w >= 0] + [o.bias for o in ops if o.bias >= 0])
    assert used == sorted(o for o, _ in spec.offsets().values())


@pytest.mark.skipif(not os.path.exists(FIXTURE), reason="reference checkout not present")
def test_structure_matches_the_reference_fixture():
    text = open(FIXTURE).read()
    assert text.count("dense_resource<__elided__>") == spec.NUM_TENSORS
    pat = re.compile(r"linalg\.conv_2d_nchw_fchw \{dilations = dense<1> : vector<2xi64>, strides = dense<(\d+)> : vector<2xi64>\} "
                     r"ins\(%\w+, %\w+ : tensor<1x(\d+)x(\d+)x(\d+)xf32>, tensor<(\d+)x(\d+)x(\d+)x(\d+)xf32>\)")
    got = [(int(m.group(2)), int(m.group(5)), int(m.group(7)), int(m.group(1)), int(m.group(3))) for m in pat.finditer(text)]
    # walk the operator list at 640x640 and collect (C, F, K, stride, padded input height) per convolution
    dims, want = {0: (3, 640)}, []
    for o in spec.graph_ops():
        ins = [t for t in o.inputs if t >= 0]
        c, h = dims[ins[0]]
        if o.kind == abi.OP_CONV:
            want.append((c, o.F, o.K, o.stride, h + 2 * o.pad))
            dims[o.out] = (o.F, (h + 2 * o.pad - o.K) // o.stride + 1)
        elif o.kind == abi.OP_CONCAT:
            assert len(set(dims[t][1] for t in ins)) == 1
            dims[o.out] = (sum(dims[t][0] for t in ins), h)
        elif o.kind == abi.OP_UPSAMPLE2X:
            dims[o.out] = (c, 2 * h)
        elif o.kind == abi.OP_YOLO_DETECT:
            boxes = sum(3 * dims[t][1] ** 2 for t in ins)
            assert boxes == 25200 and "tensor<1x25200x85xf32>" in text
        else:
            dims[o.out] = (c, h)
    assert got == want
    # the channel concatenations (dim 1) of the fixture, in order, join tensors of these channel counts
    cat = re.compile(r"tensor\.concat dim\(1\) [^:]+: \(([^)]*)\) -> tensor<1x(\d+)x(\d+)x\d+xf32>")
    got_cat = [([int(re.match(r"tensor<1x(\d+)x", p.strip()).group(1)) for p in m.group(1).split(", ")], int(m.group(3)))
               for m in cat.finditer(text)]
    want_cat, dims = [], {0: (3, 640)}
    for o in spec.graph_ops():
        ins = [t for t in o.inputs if t >= 0]
        c, h = dims[ins[0]]
        if o.kind == abi.OP_CONV:
            dims[o.out] = (o.F, (h + 2 * o.pad - o.K) // o.stride + 1)
        elif o.kind == abi.OP_CONCAT:
            want_cat.append(([dims[t][0] for t in ins], h))
            dims[o.out] = (sum(dims[t][0] for t in ins), h)
        elif o.kind == abi.OP_UPSAMPLE2X:
            dims[o.out] = (c, 2 * h)
        elif o.kind != abi.OP_YOLO_DETECT:
            dims[o.out] = (c, h)
    assert got_cat == want_cat


def test_detect_decode_closed_forms():
    A, Fv = 3, 7
    anchors = np.float32([[[1.25, 1.625], [2, 3.75], [4.125, 2.875]], [[1.875, 3.8125], [3.875, 2.8125], [3.6875, 7.4375]]])
    strides = np.float32([8, 16])
    shapes = [(4, 6), (2, 3)]  # non-square: an x/y mix-up cannot pass
    for fill, s in [(0.0, 0.5), (60.0, 1.0), (-60.0, 0.0)]:
        heads = [np.full((2, A * Fv, h, w), fill, np.float32) for h, w in shapes]
        out = oracle.yolo_detect(heads, anchors, strides, A, Fv)
        assert out.shape == (2, 3 * 24 + 3 * 6, Fv)
        box = 0
        for l, (h, w) in enumerate(shapes):
            for a in range(A):
                for y in range(h):
                    for x in range(w):
                        r = out[1, box]
                        # sigmoid 0.5: the centre of cell (x, y) in pixels and the anchor itself; 1 / 0: the extremes
                        assert np.allclose(r[0:2], [(2 * s + x - 0.5) * strides[l], (2 * s + y - 0.5) * strides[l]], rtol=1e-6)
                        assert np.allclose(r[2:4], (2 * s) ** 2 * anchors[l, a] * strides[l], rtol=1e-6, atol=1e-30)
                        assert np.allclose(r[4:], s, atol=1e-7)
                        box += 1
    # value k of anchor a of a head is channel a*F + k: a one-hot head channel lands in exactly that field
    head = np.zeros((1, A * Fv, 2, 3), np.float32)
    head[0, 1 * Fv + 5, 1, 2] = 3.0
    out = oracle.yolo_detect([head], anchors[1:], strides[1:], A, Fv)
    hot = np.argwhere(np.abs(out[0, :, 4:] - 0.5) > 1e-3)
    assert hot.tolist() == [[1 * 6 + 1 * 3 + 2, 1]]


def torch_yolov5s(x, blob):
    """ultralytics yolov5s (fused) forward in float64 functional ops, from the file-order blob."""
    off = spec.offsets()
    P = lambda n: torch.from_numpy(blob[off[n][0]:off[n][0] + spec.numel(off[n][1])].reshape(off[n][1]).astype(np.float64))

    def conv(y, name, k=1, s=1, p=None, act=True):
        y = F.conv2d(y, P(name + ".weight"), P(name + ".bias"), stride=s, padding=k // 2 if p is None else p)
        return F.silu(y) if act else y

    def c3(y, name, n, shortcut):
        a = conv(y, name + ".cv1.conv")
        for i in range(n):
            t = conv(conv(a, "%s.m.%d.cv1.conv" % (name, i)), "%s.m.%d.cv2.conv" % (name, i), 3)
            a = a + t if shortcut else t
        return conv(torch.cat([a, conv(y, name + ".cv2.conv")], 1), name + ".cv3.conv")

    y = torch.from_numpy(x.astype(np.float64))
    y = conv(y, "model.0.conv", 6, 2, 2)
    y = conv(y, "model.1.conv", 3, 2)
    y = c3(y, "model.2", 1, True)
    y = conv(y, "model.3.conv", 3, 2)
    p3 = y = c3(y, "model.4", 2, True)
    y = conv(y, "model.5.conv", 3, 2)
    p4 = y = c3(y, "model.6", 3, True)
    y = conv(y, "model.7.conv", 3, 2)
    y = c3(y, "model.8", 1, True)
    x1 = conv(y, "model.9.cv1.conv")
    y1 = F.max_pool2d(x1, 5, 1, 2)
    y2 = F.max_pool2d(y1, 5, 1, 2)
    y = conv(torch.cat([x1, y1, y2, F.max_pool2d(y2, 5, 1, 2)], 1), "model.9.cv2.conv")
    h10 = y = conv(y, "model.10.conv")
    y = c3(torch.cat([F.interpolate(y, scale_factor=2, mode="nearest"), p4], 1), "model.13", 1, False)
    h14 = y = conv(y, "model.14.conv")
    d3 = y = c3(torch.cat([F.interpolate(y, scale_factor=2, mode="nearest"), p3], 1), "model.17", 1, False)
    d4 = y = c3(torch.cat([conv(y, "model.18.conv", 3, 2), h14], 1), "model.20", 1, False)
    d5 = c3(torch.cat([conv(d4, "model.21.conv", 3, 2), h10], 1), "model.23", 1, False)
    z = []
    anchors, stride = P("model.24.anchors"), P("model.24.stride")
    for l, d in enumerate((d3, d4, d5)):
        t = F.conv2d(d, P("model.24.m.%d.weight" % l), P("model.24.m.%d.bias" % l))
        bs, _, ny, nx = t.shape
        t = t.view(bs, 3, 85, ny, nx).permute(0, 1, 3, 4, 2).sigmoid()
        yv, xv = torch.meshgrid(torch.arange(ny, dtype=torch.float64), torch.arange(nx, dtype=torch.float64), indexing="ij")
        grid = torch.stack((xv, yv), 2).expand(1, 3, ny, nx, 2) - 0.5
        ag = (anchors[l] * stride[l]).view(1, 3, 1, 1, 2)
        xy = (t[..., 0:2] * 2 + grid) * stride[l]
        wh = (t[..., 2:4] * 2) ** 2 * ag
        z.append(torch.cat((xy, wh, t[..., 4:]), 4).view(bs, 3 * ny * nx, 85))
    return torch.cat(z, 1).numpy()


def test_yolov5s_oracle_vs_torch():
    blob = synth.yolov5s_params()
    x = synth.uniform(8000, (2, 3, 64, 96), 0.0, 1.0)
    got = oracle.run_graph(spec.graph_ops(), x, blob, 3)
    want = torch_yolov5s(x, blob)
    assert got.shape == want.shape == (2, 3 * (8 * 12 + 4 * 6 + 2 * 3), 85)
    assert np.abs(got[..., :4] - want[..., :4]).max() <= 2e-5 * np.abs(want[..., :4]).max()
    assert np.abs(got[..., 4:] - want[..., 4:]).max() <= 2e-5
    # the OpenMP x AVX2 convolution gives the same network (used as the checker for full-size images)
    got2 = oracle.run_graph(spec.graph_ops(), x, blob, 3, conv=oracle.hwp_conv2d)
    assert np.abs(got2 - got).max() <= 2e-5 * np.abs(got).max()
