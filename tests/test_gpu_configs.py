"""BASELINE configurations at their full sizes on the GPU.

The oracle is too slow for whole batches, so every full-size case is checked two ways: the first
images of the batch against the oracle (a convolution / the network treats images independently),
and size-independent properties of the full batch (batch independence, permutation equivariance).
"""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import Conv, Model, dev, host, nhwc, nchw, rel_l2, FP16_REL_L2

pytestmark = pytest.mark.gpu


def _oracle_layer(x, w, stride, bn, res):
    y = oracle.batchnorm(oracle.conv2d_nchw_fchw(oracle.pad_nchw(x, 1), w, stride=stride), *bn)
    if res is not None:
        y = y + res
    return oracle.relu(y)


@pytest.mark.parametrize("i", range(len(synth.CFG5_LAYERS)))
def test_conv3x3_layer_sweep_fp16_batch64(i):
    """3x3 conv + BN + ReLU (+ residual) of every ResNet-18 stage, fp16, batch 64."""
    c, k, h, s = synth.CFG5_LAYERS[i]
    x, w, bn, res = synth.cfg5_layer(i, 64)
    bn = tuple(synth.round_fp16(b) for b in bn)
    layer = Conv(abi.F16, w, s, 1, bn=bn, relu=True)
    xd = dev(nhwc(x), abi.F16)
    rd = dev(nhwc(res), abi.F16) if res is not None else None
    got = nchw(host(layer(xd, abi.NHWC, residual=rd)))
    # first two images against the oracle
    want = _oracle_layer(x[:2], w, s, bn, res[:2] if res is not None else None)
    err = rel_l2(got[:2], want)
    print("layer", (c, k, h, s), "rel_l2", err, flush=True)
    assert err < FP16_REL_L2
    assert np.isfinite(got).all() and (got >= 0).all()
    # permutation equivariance over the batch, bit for bit (same launch geometry)
    perm = np.random.default_rng(i).permutation(64)
    xp = dev(nhwc(x[perm]), abi.F16)
    rp = dev(nhwc(res[perm]), abi.F16) if res is not None else None
    got_p = nchw(host(layer(xp, abi.NHWC, residual=rp)))
    assert np.array_equal(got_p, got[perm])


def test_resnet18_fp16_batch32_full_size():
    """BASELINE config 4 at its real size: [32,3,224,224] fp16."""
    hb = synth.round_fp16(synth.resnet18_params())
    x = synth.round_fp16(synth.cfg4_input(32))
    m = Model(hb, abi.F16)
    got = host(m(dev(x, abi.F16)))
    assert got.shape == (32, 1000) and np.isfinite(got).all()
    want = oracle.resnet18_forward(x[:2], hb)
    err = rel_l2(got[:2], want)
    print("bs32 first two images rel_l2", err, "top1", got[:2].argmax(1), want.argmax(1), flush=True)
    assert err < FP16_REL_L2
    assert (got[:2].argmax(1) == want.argmax(1)).all()
    # batch 1 (other tile shapes and K-group counts, hence another summation order) agrees closely
    one = host(m(dev(x[5:6], abi.F16)))
    assert rel_l2(one, got[5:6]) < 2e-3
    assert one.argmax(1) == got[5:6].argmax(1)
    # permuting the batch permutes the logits, bit for bit
    perm = np.random.default_rng(7).permutation(32)
    got_p = host(m(dev(x[perm], abi.F16)))
    assert np.array_equal(got_p, got[perm])


def _tags_and_logits(m, xd):
    """One eager pass under the event profiler: the logits and how often each kernel instance was launched."""
    host(m(xd))
    abi.profile_enable(True)
    try:
        abi.profile_report()
        got = host(m(xd))
        rep = abi.profile_report()
    finally:
        abi.profile_enable(False)
    return got, {k: v["launches"] for k, v in rep.items()}


@pytest.mark.parametrize("passes", [1, 4])
def test_resnet18_fp16_every_image_of_the_batch_against_the_oracle(passes):
    """BASELINE config 4, all 32 images (examples/Res18/main.cpp:103-111 takes the top-1 of every image): every row of the
    logits within the fp16 bar of the CPU oracle (its OpenMP x AVX2 convolution, itself checked against the scalar one)
    and the same top-1 on every image -- with the launch shapes of one pass at a time, and with the shapes a handle
    planned for four passes in flight takes (the ones the benchmark's headline runs), asserted from the launch tags.
    The same for batch 1."""
    hb = synth.round_fp16(synth.resnet18_params())
    x = synth.round_fp16(synth.cfg4_input(32))
    want = oracle.hwp_resnet18_forward(x, hb)
    m = Model(hb, abi.F16, abi.ALGO_AUTO, passes=passes)
    got, rep = _tags_and_logits(m, dev(x, abi.F16))
    print("passes", passes, rep, flush=True)
    count = lambda prefix: sum(v for k, v in rep.items() if k.startswith(prefix))
    if passes == 4:
        assert rep.get("conv3x3_stream<f16,1x4x1>", 0) == 6 and rep.get("conv3x3_stream<f16,1x2x2,res>", 0) == 4
        assert count("conv3x3_stream") == 10 and count("conv3x3_patch") == 3
        assert "avgpool_fc" not in rep and rep.get("global_avgpool", 0) == 1
    else:
        # layer1's 64 channels are one slab: the form that keeps its weight fragments in registers
        assert rep.get("conv3x3_stream<f16,1x2x2,res>", 0) == 4 and rep.get("conv3x3_stream<f16,1x2x2>", 0) == 6
        assert count("conv3x3_stream") == 10 and count("conv3x3_patch") == 3 and rep.get("avgpool_fc", 0) == 1
    assert count("conv3x3s2_patch") == 3 and rep.get("stem_conv7x7_bn_relu_maxpool<f16>", 0) == 1
    errs = [rel_l2(got[i], want[i]) for i in range(32)]
    print("worst image rel_l2 %.2e" % max(errs), flush=True)
    assert max(errs) < FP16_REL_L2
    assert np.array_equal(got.argmax(1), want.argmax(1))
    one, rep1 = _tags_and_logits(m, dev(x[7:8], abi.F16))
    assert rel_l2(one, want[7:8]) < FP16_REL_L2 and one.argmax(1) == want[7:8].argmax(1)
    m.close()
