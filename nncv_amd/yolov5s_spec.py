"""Tensor table and operator list of YOLOv5s as exported in the reference's fixture
tests/Nets/Yolov5s.mlir (ultralytics yolov5s.yaml v6, BatchNorm already fused into the 60
convolutions, 80 classes, input 640x640 there): 57 Conv + SiLU, 3 Detect convolutions, three 5x5
max-pools (SPPF), two nearest 2x up-samplings, 13 channel concatenations, 7 residual adds, and the
Detect decode to [N, 25200, 85].

Parameter order = `state_dict` order of the fused model (`model.<i>...conv.weight`, `.conv.bias`;
Detect: `model.24.anchors` [3,3,2] in units of the stride, then `model.24.m.<l>.weight/.bias`),
followed by `model.24.stride` [3], which ultralytics keeps as an attribute and the fixture as a
constant (:1394).  122 tensors like the fixture's 122 constants; 7 225 906 elements (ultralytics
reports 7 225 885 parameters; + 18 anchor values + 3 strides).
"""
from . import abi

NUM_CLASSES = 80
ANCHORS_PER_LEVEL = 3
STRIDES = (8.0, 16.0, 32.0)
# pixels; `model.24.anchors` holds these divided by the level's stride
ANCHORS_PX = ((10, 13, 16, 30, 33, 23), (30, 61, 62, 45, 59, 119), (116, 90, 156, 198, 373, 326))


class _Builder:
    """Walks yolov5s.yaml once; records tensors (name, shape) and operators."""

    def __init__(self):
        self.tensors, self.ops, self.convs = [], [], []
        self.off = 0
        self.next_id = 1

    def _take(self, name, shape):
        n = 1
        for s in shape:
            n *= s
        self.tensors.append((name, tuple(shape)))
        o = self.off
        self.off += n
        return o

    def new_id(self):
        self.next_id += 1
        return self.next_id - 1

    def conv(self, x, name, c1, c2, k=1, s=1, p=None, act=abi.ACT_SILU, residual=-1):
        p = k // 2 if p is None else p
        w = self._take(name + ".weight", (c2, c1, k, k))
        b = self._take(name + ".bias", (c2,))
        out = self.new_id()
        self.ops.append(abi.graph_op(abi.OP_CONV, [x, residual], out, F=c2, K=k, stride=s, pad=p, act=act, w=w, bias=b))
        self.convs.append((c1, c2, k, s, p))
        return out

    def simple(self, kind, ins, **kw):
        out = self.new_id()
        self.ops.append(abi.graph_op(kind, ins, out, **kw))
        return out

    def c3(self, x, name, c1, c2, n, shortcut):
        c_ = c2 // 2
        y = self.conv(x, name + ".cv1.conv", c1, c_)
        for i in range(n):
            # Bottleneck: x + cv2(cv1(x)); the add comes after cv2's SiLU, so it is its own operator
            t = self.conv(y, "%s.m.%d.cv1.conv" % (name, i), c_, c_)
            t = self.conv(t, "%s.m.%d.cv2.conv" % (name, i), c_, c_, 3)
            y = self.simple(abi.OP_ADD, [y, t], stride=0) if shortcut else t
        z = self.conv(x, name + ".cv2.conv", c1, c_)
        cat = self.simple(abi.OP_CONCAT, [y, z], stride=0)
        return self.conv(cat, name + ".cv3.conv", 2 * c_, c2)


def _build():
    b = _Builder()
    # state_dict order inside a C3 is cv1, cv2, cv3, m.*; execution order is cv1, m.*, cv2, cv3.
    # The builder records tensors in execution order; `tensor_table` re-sorts them below.
    x = b.conv(0, "model.0.conv", 3, 32, 6, 2, 2)
    x = b.conv(x, "model.1.conv", 32, 64, 3, 2)
    x = b.c3(x, "model.2", 64, 64, 1, True)
    x = b.conv(x, "model.3.conv", 64, 128, 3, 2)
    p3 = x = b.c3(x, "model.4", 128, 128, 2, True)
    x = b.conv(x, "model.5.conv", 128, 256, 3, 2)
    p4 = x = b.c3(x, "model.6", 256, 256, 3, True)
    x = b.conv(x, "model.7.conv", 256, 512, 3, 2)
    x = b.c3(x, "model.8", 512, 512, 1, True)
    # SPPF
    x1 = b.conv(x, "model.9.cv1.conv", 512, 256)
    y1 = b.simple(abi.OP_MAXPOOL, [x1], K=5, stride=1, pad=2)
    y2 = b.simple(abi.OP_MAXPOOL, [y1], K=5, stride=1, pad=2)
    y3 = b.simple(abi.OP_MAXPOOL, [y2], K=5, stride=1, pad=2)
    x = b.conv(b.simple(abi.OP_CONCAT, [x1, y1, y2, y3], stride=0), "model.9.cv2.conv", 1024, 512)
    # head
    h10 = x = b.conv(x, "model.10.conv", 512, 256)
    x = b.simple(abi.OP_CONCAT, [b.simple(abi.OP_UPSAMPLE2X, [x], stride=0), p4], stride=0)
    x = b.c3(x, "model.13", 512, 256, 1, False)
    h14 = x = b.conv(x, "model.14.conv", 256, 128)
    x = b.simple(abi.OP_CONCAT, [b.simple(abi.OP_UPSAMPLE2X, [x], stride=0), p3], stride=0)
    d3 = x = b.c3(x, "model.17", 256, 128, 1, False)
    x = b.conv(x, "model.18.conv", 128, 128, 3, 2)
    x = b.simple(abi.OP_CONCAT, [x, h14], stride=0)
    d4 = x = b.c3(x, "model.20", 256, 256, 1, False)
    x = b.conv(x, "model.21.conv", 256, 256, 3, 2)
    x = b.simple(abi.OP_CONCAT, [x, h10], stride=0)
    d5 = b.c3(x, "model.23", 512, 512, 1, False)
    # Detect
    no = ANCHORS_PER_LEVEL * (5 + NUM_CLASSES)
    anchors = b._take("model.24.anchors", (3, ANCHORS_PER_LEVEL, 2))
    heads = [b.conv(d, "model.24.m.%d" % l, c, no, act=abi.ACT_NONE) for l, (d, c) in enumerate(((d3, 128), (d4, 256), (d5, 512)))]
    strides = b._take("model.24.stride", (3,))
    b.ops.append(abi.graph_op(abi.OP_YOLO_DETECT, heads, b.new_id(), F=5 + NUM_CLASSES, K=ANCHORS_PER_LEVEL, stride=0,
                              w=anchors, bias=strides))
    return b


def _sort_key(name):
    """state_dict order: module index, then within C3 cv1 < cv2 < cv3 < m.*; stride last."""
    parts = name.split(".")
    idx = int(parts[1])
    if name == "model.24.stride":
        return (99, 0, 0, 0)
    if name == "model.24.anchors":
        return (24, -1, 0, 0)
    sub = parts[2]
    order = {"conv": 0, "cv1": 0, "cv2": 1, "cv3": 2, "m": 3}[sub]
    inner = (int(parts[3]), {"cv1": 0, "cv2": 1, "weight": 0, "bias": 1}[parts[4]]) if sub == "m" and idx != 24 else \
        ((int(parts[3]), 0) if sub == "m" else (0, 0))
    return (idx, order, inner, 0 if name.endswith("weight") else 1)


def tensor_table():
    """[(name, shape)] in file order."""
    return sorted(_build().tensors, key=lambda t: _sort_key(t[0]))


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


def offsets():
    out, off = {}, 0
    for name, shape in tensor_table():
        out[name] = (off, shape)
        off += numel(shape)
    return out


def graph_ops():
    """[abi.GraphOp] with parameter offsets into the file-order blob."""
    b = _build()
    exec_off, o = {}, 0
    for name, shape in b.tensors:
        exec_off[o] = name
        o += numel(shape)
    file_off = offsets()
    ops = []
    for op in b.ops:
        c = abi.GraphOp.from_buffer_copy(op)
        if c.w >= 0:
            c.w = file_off[exec_off[op.w]][0]
        if c.bias >= 0:
            c.bias = file_off[exec_off[op.bias]][0]
        ops.append(c)
    return ops


def conv_table():
    """[(C, F, K, stride, pad)] of the 60 convolutions in execution order."""
    return list(_build().convs)


NUM_TENSORS = 122
NUM_ELEMENTS = sum(numel(s) for _, s in _build().tensors)


def flops_per_image(h, w=None):
    """2*MACs of the 60 convolutions for an h x w image (both multiples of 32)."""
    w = h if w is None else w
    ops, total = graph_ops(), 0
    dims = {0: (3, h, w)}
    for o in ops:
        ins = [t for t in o.inputs if t >= 0]
        c, hh, ww = dims[ins[0]]
        if o.kind == abi.OP_CONV:
            oh, ow = (hh + 2 * o.pad - o.K) // o.stride + 1, (ww + 2 * o.pad - o.K) // o.stride + 1
            total += 2 * oh * ow * o.F * c * o.K * o.K
            dims[o.out] = (o.F, oh, ow)
        elif o.kind == abi.OP_CONCAT:
            dims[o.out] = (sum(dims[t][0] for t in ins), hh, ww)
        elif o.kind == abi.OP_UPSAMPLE2X:
            dims[o.out] = (c, 2 * hh, 2 * ww)
        else:
            dims[o.out] = (c, hh, ww)
    return total
