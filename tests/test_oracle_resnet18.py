"""Whole-network oracle vs an independent composition of torch CPU functional ops, following
the op order of tests/Nets/Res18.mlir (stem, maxpool, 8 BasicBlocks, avgpool, FC)."""
import numpy as np
import torch
import torch.nn.functional as F

import oracle
from nncv_amd import resnet18_spec as spec
from nncv_amd import synth


def torch_resnet18(x, blob):
    """float64 torch composition; BN eps = float32(1e-5)."""
    off = spec.offsets()
    eps = float(np.float32(1e-5))

    def P(name):
        o, shape = off[name]
        return torch.from_numpy(blob[o:o + spec.numel(shape)].reshape(shape).astype(np.float64))

    def bn(y, p):
        return F.batch_norm(y, P(p + ".running_mean"), P(p + ".running_var"), P(p + ".weight"),
                            P(p + ".bias"), False, 0.0, eps)

    y = torch.from_numpy(x.astype(np.float64))
    y = F.relu(bn(F.conv2d(y, P("conv1.weight"), stride=2, padding=3), "bn1"))
    y = F.max_pool2d(y, 3, 2, 1)
    taps = [y]
    cin = 64
    for li, f in enumerate(spec.WIDTHS, start=1):
        for blk in range(2):
            p = "layer%d.%d" % (li, blk)
            s = 2 if (li > 1 and blk == 0) else 1
            idn = y
            o = F.relu(bn(F.conv2d(y, P(p + ".conv1.weight"), stride=s, padding=1), p + ".bn1"))
            o = bn(F.conv2d(o, P(p + ".conv2.weight"), stride=1, padding=1), p + ".bn2")
            if s != 1 or cin != f:
                idn = bn(F.conv2d(y, P(p + ".downsample.0.weight"), stride=s), p + ".downsample.1")
            y = F.relu(o + idn)
            cin = f
        taps.append(y)
    y = y.mean(dim=(2, 3))
    return F.linear(y, P("fc.weight"), P("fc.bias")).numpy(), [a.numpy() for a in taps]


def test_resnet18_oracle_vs_torch_small_image():
    blob = synth.resnet18_params()
    # give the FC a non-zero bias here so a dropped bias term is caught
    blob = blob.copy()
    blob[-1000:] = synth.normal(9, (1000,), std=0.05)
    x = synth.uniform(3001, (2, 3, 64, 64), 0.0, 1.0)
    want, taps = torch_resnet18(x, blob)
    got, tap2 = oracle.resnet18_forward(x, blob, tap_layer=2)
    assert got.shape == (2, 1000)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() / scale < 1e-5
    assert np.abs(tap2 - taps[2]).max() / np.abs(taps[2]).max() < 1e-5
    assert (got.argmax(1) == want.argmax(1)).all()


def test_resnet18_oracle_non_square_batch_independent():
    """Images of a batch do not interact: forward(batch)[i] == forward(image i)."""
    blob = synth.resnet18_params()
    x = synth.uniform(3002, (2, 3, 64, 96), 0.0, 1.0)
    both = oracle.resnet18_forward(x, blob)
    one = oracle.resnet18_forward(x[1:2], blob)
    assert np.array_equal(both[1:2], one)


def test_operator_list_evaluator_reproduces_the_network_oracle():
    """oracle.run_graph over resnet18_spec.graph_ops() (the checker of the generic executor) against the
    C restatement of the whole network, which the tests above pin: two independently written walks of
    tests/Nets/Res18.mlir must agree."""
    blob = synth.resnet18_params()
    x = synth.uniform(3009, (2, 3, 72, 56), 0.0, 1.0)
    got = oracle.run_graph(spec.graph_ops(), x, blob, 3).reshape(2, 1000)
    want = oracle.resnet18_forward(x, blob)
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
