"""Canonical tensor table and operator list of a MobileNetV3-small `model.bin`.

The network is the one of the reference's fixture tests/Nets/MobileNetV3.mlir (torch-mlir export
of torchvision's `mobilenet_v3_small`, 256x256 input there): 52 convolutions of which 11
depthwise (:245, :290 ...), 9 squeeze-excitation blocks (:322-384), BatchNorm with epsilon 1e-3
(:228), hard-swish / hard-sigmoid spelled with add / max / min / div generics (:259-293, :349-379)
and two Linear layers.  As for ResNet-18 the parameter order is torchvision `state_dict` order
without `num_batches_tracked`.  210 tensors (the fixture holds 210 constants), 2 554 968 elements
(2 542 856 trainable + 12 112 running statistics).
"""
from . import abi

# (input channels, kernel, expanded channels, output channels, squeeze-excitation, hard-swish, stride)
BNECK = [
    (16, 3, 16, 16, True, False, 2),
    (16, 3, 72, 24, False, False, 2),
    (24, 3, 88, 24, False, False, 1),
    (24, 5, 96, 40, True, True, 2),
    (40, 5, 240, 40, True, True, 1),
    (40, 5, 240, 40, True, True, 1),
    (40, 5, 120, 48, True, True, 1),
    (48, 5, 144, 48, True, True, 1),
    (48, 5, 288, 96, True, True, 2),
    (96, 5, 576, 96, True, True, 1),
    (96, 5, 576, 96, True, True, 1),
]
BN_EPS = 1e-3
NUM_TENSORS = 210
NUM_ELEMENTS = 2554968


def make_divisible(v, divisor=8):
    """torchvision.ops.misc._make_divisible with min_value = divisor"""
    new_v = max(divisor, int(v + divisor / 2) // divisor * divisor)
    if new_v < 0.9 * v:
        new_v += divisor
    return new_v


def squeeze_channels(expanded):
    return make_divisible(expanded // 4, 8)


def _bn(prefix, c):
    return [(prefix + ".weight", (c,)), (prefix + ".bias", (c,)),
            (prefix + ".running_mean", (c,)), (prefix + ".running_var", (c,))]


def tensor_table():
    """[(name, shape)] in file order."""
    t = [("features.0.0.weight", (16, 3, 3, 3))] + _bn("features.0.1", 16)
    for i, (cin, k, exp, cout, se, hs, stride) in enumerate(BNECK, start=1):
        p = "features.%d.block" % i
        j = 0
        if exp != cin:
            t += [("%s.%d.0.weight" % (p, j), (exp, cin, 1, 1))] + _bn("%s.%d.1" % (p, j), exp)
            j += 1
        t += [("%s.%d.0.weight" % (p, j), (exp, 1, k, k))] + _bn("%s.%d.1" % (p, j), exp)
        j += 1
        if se:
            sq = squeeze_channels(exp)
            t += [("%s.%d.fc1.weight" % (p, j), (sq, exp, 1, 1)), ("%s.%d.fc1.bias" % (p, j), (sq,)),
                  ("%s.%d.fc2.weight" % (p, j), (exp, sq, 1, 1)), ("%s.%d.fc2.bias" % (p, j), (exp,))]
            j += 1
        t += [("%s.%d.0.weight" % (p, j), (cout, exp, 1, 1))] + _bn("%s.%d.1" % (p, j), cout)
    t += [("features.12.0.weight", (576, 96, 1, 1))] + _bn("features.12.1", 576)
    t += [("classifier.0.weight", (1024, 576)), ("classifier.0.bias", (1024,)),
          ("classifier.3.weight", (1000, 1024)), ("classifier.3.bias", (1000,))]
    return t


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


def offsets():
    """{name: (element offset, shape)}"""
    out, off = {}, 0
    for name, shape in tensor_table():
        out[name] = (off, shape)
        off += numel(shape)
    return out


def graph_ops():
    """The network as [abi.GraphOp] over tensor ids (0 = input), built from the tensor table."""
    off = offsets()
    ops = []
    nxt = [1]

    def new_id():
        nxt[0] += 1
        return nxt[0] - 1

    def conv_bn(x, conv, bn, k, stride, depthwise, act, residual=-1):
        F = off[conv + ".weight"][1][0]
        o = abi.graph_op(abi.OP_DWCONV if depthwise else abi.OP_CONV, [x, residual], new_id(), F=F, K=k, stride=stride,
                         pad=(k - 1) // 2, act=act, eps=BN_EPS, w=off[conv + ".weight"][0],
                         bn=tuple(off[bn + s][0] for s in (".weight", ".bias", ".running_mean", ".running_var")))
        ops.append(o)
        return o.out

    def fc(x, name, act):
        F = off[name + ".weight"][1][0]
        o = abi.graph_op(abi.OP_CONV, [x], new_id(), F=F, K=1, act=act, w=off[name + ".weight"][0], bias=off[name + ".bias"][0])
        ops.append(o)
        return o.out

    def simple(kind, a, b=-1):
        o = abi.graph_op(kind, [a, b], new_id(), stride=0)
        ops.append(o)
        return o.out

    x = conv_bn(0, "features.0.0", "features.0.1", 3, 2, False, abi.ACT_HARDSWISH)
    for i, (cin, k, exp, cout, se, hs, stride) in enumerate(BNECK, start=1):
        p = "features.%d.block" % i
        act = abi.ACT_HARDSWISH if hs else abi.ACT_RELU
        block_in, y, j = x, x, 0
        if exp != cin:
            y = conv_bn(y, "%s.%d.0" % (p, j), "%s.%d.1" % (p, j), 1, 1, False, act)
            j += 1
        y = conv_bn(y, "%s.%d.0" % (p, j), "%s.%d.1" % (p, j), k, stride, True, act)
        j += 1
        if se:
            g = simple(abi.OP_GAVGPOOL, y)
            g = fc(g, "%s.%d.fc1" % (p, j), abi.ACT_RELU)
            g = fc(g, "%s.%d.fc2" % (p, j), abi.ACT_HARDSIGMOID)
            y = simple(abi.OP_SCALE, y, g)
            j += 1
        res = block_in if (stride == 1 and cin == cout) else -1
        x = conv_bn(y, "%s.%d.0" % (p, j), "%s.%d.1" % (p, j), 1, 1, False, abi.ACT_NONE, res)
    x = conv_bn(x, "features.12.0", "features.12.1", 1, 1, False, abi.ACT_HARDSWISH)
    x = simple(abi.OP_GAVGPOOL, x)
    x = fc(x, "classifier.0", abi.ACT_HARDSWISH)
    x = fc(x, "classifier.3", abi.ACT_NONE)
    return ops


def conv_table(h):
    """[(kind, C, F, K, stride, H_in)] of the 52 convolutions for an h x h image (kind "conv" | "dw");
    the squeeze-excitation and classifier layers are 1x1 convolutions over a 1x1 image."""
    out = [("conv", 3, 16, 3, 2, h)]
    cur = (h + 2 - 3) // 2 + 1
    for cin, k, exp, cout, se, hs, stride in BNECK:
        if exp != cin:
            out.append(("conv", cin, exp, 1, 1, cur))
        out.append(("dw", exp, exp, k, stride, cur))
        cur = (cur + 2 * ((k - 1) // 2) - k) // stride + 1
        if se:
            sq = squeeze_channels(exp)
            out += [("conv", exp, sq, 1, 1, 1), ("conv", sq, exp, 1, 1, 1)]
        out.append(("conv", exp, cout, 1, 1, cur))
    out.append(("conv", 96, 576, 1, 1, cur))
    return out


def flops_per_image(h):
    """2*MACs of the convolutions and Linear layers for an h x h image."""
    total = 0
    for kind, c, f, k, s, hin in conv_table(h):
        oh = (hin + 2 * ((k - 1) // 2) - k) // s + 1
        total += 2 * oh * oh * f * (1 if kind == "dw" else c) * k * k
    return total + 2 * (576 * 1024 + 1024 * 1000)
