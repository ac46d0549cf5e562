"""Canonical tensor table of a ResNet-18 `model.bin`.

nncv's `-split-params` pass appends every `memref.global` of the bufferized module to one flat
array and bakes element offsets into the compiled object
(src/nncv/compiler/Conversion/Transforms/SplitParamsFlatArray.cpp:99-206); the order is an
artefact of MLIR's module walk and no file in the reference pins it.  A library has to fix one:
torchvision `state_dict` order without `num_batches_tracked`, each BatchNorm contributing
weight (gamma), bias (beta), running_mean, running_var.  102 tensors, 11 699 112 elements.
"""

WIDTHS = (64, 128, 256, 512)


def _bn(prefix, c):
    return [(prefix + ".weight", (c,)), (prefix + ".bias", (c,)),
            (prefix + ".running_mean", (c,)), (prefix + ".running_var", (c,))]


def tensor_table():
    """[(name, shape)] in file order."""
    t = [("conv1.weight", (64, 3, 7, 7))] + _bn("bn1", 64)
    cin = 64
    for li, f in enumerate(WIDTHS, start=1):
        for blk in range(2):
            p = "layer%d.%d" % (li, blk)
            stride = 2 if (li > 1 and blk == 0) else 1
            t += [(p + ".conv1.weight", (f, cin, 3, 3))] + _bn(p + ".bn1", f)
            t += [(p + ".conv2.weight", (f, f, 3, 3))] + _bn(p + ".bn2", f)
            if stride != 1 or cin != f:
                t += [(p + ".downsample.0.weight", (f, cin, 1, 1))] + _bn(p + ".downsample.1", f)
            cin = f
    t += [("fc.weight", (1000, 512)), ("fc.bias", (1000,))]
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


NUM_TENSORS = 102
NUM_ELEMENTS = 11699112


def conv_layers(h):
    """[(name, C, F, R, stride, pad, H_in)] of the 20 convs for an h x h input image."""
    out = [("conv1", 3, 64, 7, 2, 3, h)]
    cur = h // 4
    cin = 64
    for li, f in enumerate(WIDTHS, start=1):
        for blk in range(2):
            p = "layer%d.%d" % (li, blk)
            stride = 2 if (li > 1 and blk == 0) else 1
            out.append((p + ".conv1", cin, f, 3, stride, 1, cur))
            if stride != 1 or cin != f:
                out.append((p + ".downsample.0", cin, f, 1, stride, 0, cur))
            cur //= stride
            out.append((p + ".conv2", f, f, 3, 1, 1, cur))
            cin = f
    return out


def flops_per_image(h):
    """2*MACs of the convs + FC for an h x h image (direct-convolution count)."""
    total = 0
    for _, c, f, r, s, p, hin in conv_layers(h):
        oh = (hin + 2 * p - r) // s + 1
        total += 2 * oh * oh * f * c * r * r
    return total + 2 * 512 * 1000


def graph_ops():
    """The same network as an operator list for the generic executor (nncv_hip_graph_*): what the
    hard-wired ResNet18 object computes, without its fused stem / shortcut / head kernels."""
    from . import abi
    off = offsets()
    ops = []
    nxt = [1]

    def new_id():
        nxt[0] += 1
        return nxt[0] - 1

    def conv_bn(x, conv, bn, k, stride, pad, act, residual=-1):
        o = abi.graph_op(abi.OP_CONV, [x, residual], new_id(), F=off[conv + ".weight"][1][0], K=k, stride=stride, pad=pad, act=act,
                         eps=1e-5, w=off[conv + ".weight"][0],
                         bn=tuple(off[bn + s][0] for s in (".weight", ".bias", ".running_mean", ".running_var")))
        ops.append(o)
        return o.out

    x = conv_bn(0, "conv1", "bn1", 7, 2, 3, abi.ACT_RELU)
    ops.append(abi.graph_op(abi.OP_MAXPOOL, [x], new_id(), K=3, stride=2, pad=1))
    x = ops[-1].out
    cin = 64
    for li, f in enumerate(WIDTHS, start=1):
        for blk in range(2):
            p = "layer%d.%d" % (li, blk)
            stride = 2 if (li > 1 and blk == 0) else 1
            idn = x
            y = conv_bn(x, p + ".conv1", p + ".bn1", 3, stride, 1, abi.ACT_RELU)
            if stride != 1 or cin != f:
                idn = conv_bn(x, p + ".downsample.0", p + ".downsample.1", 1, stride, 0, abi.ACT_NONE)
            x = conv_bn(y, p + ".conv2", p + ".bn2", 3, 1, 1, abi.ACT_RELU, residual=idn)
            cin = f
    ops.append(abi.graph_op(abi.OP_GAVGPOOL, [x], new_id(), stride=0))
    ops.append(abi.graph_op(abi.OP_CONV, [ops[-1].out], new_id(), F=1000, K=1, w=off["fc.weight"][0], bias=off["fc.bias"][0]))
    return ops
