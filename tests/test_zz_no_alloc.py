"""The entry point that allocates nothing, nncv_hip_conv_forward_noalloc, against nncv_hip_conv_forward on the same
inputs: two calls in a row through the C ABI, the second with a smaller input (the scratch array keeps the first
call's contents), then a request beyond the scratch array's size, which must fail with a message and change nothing.
The layers are fp32 3x3 ones of the K-split kind (the partial sums and tickets are what the scratch array holds) and
one fp16 layer that needs no workspace at all."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import Conv, dev, empty, host

pytestmark = pytest.mark.gpu

FP32_MAX_REL = 1e-4  # fp32 bar of the parity suite: normwise max relative error
FP16_REL_L2 = 1e-2


def max_rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b)) / max(float(np.max(np.abs(b))), 1e-30))


def run_pair(layer, dt, N, H, W, seed):
    C, F = layer.C, layer.F
    x = synth.normal(seed, (N, H, W, C))
    res = synth.normal(seed + 1, (N, H, W, F))
    if dt == abi.F16:
        x, res = synth.round_fp16(x), synth.round_fp16(res)
    xd, rd = dev(x, dt), dev(res, dt)
    want = host(layer(xd, abi.NHWC, rd))
    out = empty((N, H, W, F), dt)
    out.zero_()
    torch.cuda.synchronize()
    abi.check(abi.lib().nncv_hip_conv_forward_noalloc(layer.h, xd.data_ptr(), N, H, W, rd.data_ptr(), out.data_ptr(), None))
    return host(out), want


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_noalloc_matches_conv_forward_twice(dt):
    C = F = 512
    w = synth.normal(9100, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9))))
    if dt == abi.F16:
        w = synth.round_fp16(w)
    bn = (np.linspace(0.5, 1.5, F).astype(np.float32), np.linspace(-0.1, 0.1, F).astype(np.float32),
          np.linspace(-0.2, 0.2, F).astype(np.float32), np.linspace(0.5, 1.5, F).astype(np.float32))
    if dt == abi.F16:
        bn = tuple(synth.round_fp16(b) for b in bn)
    layer = Conv(dt, w, 1, 1, bn=bn, relu=True, algo=abi.ALGO_IGEMM)
    for (N, H, W, seed) in ((1, 8, 8, 9200), (1, 4, 4, 9300)):  # the K-split shape of config 3's last stage, then a smaller one
        print("noalloc case", dt, N, H, W, flush=True)
        got, want = run_pair(layer, dt, N, H, W, seed)
        # against the CPU oracle as well, so that this file stands on its own: conv + BatchNorm + residual + ReLU
        x = synth.normal(seed, (N, H, W, C))
        res = synth.normal(seed + 1, (N, H, W, F))
        if dt == abi.F16:
            x, res = synth.round_fp16(x), synth.round_fp16(res)
        ref = oracle.conv2d_nchw_fchw(oracle.pad_nchw(np.ascontiguousarray(x.transpose(0, 3, 1, 2)), 1), w, stride=1)
        ref = oracle.relu(oracle.batchnorm(ref, *bn) + res.transpose(0, 3, 1, 2)).transpose(0, 2, 3, 1)
        if dt == abi.F32:
            assert max_rel(got, ref) < FP32_MAX_REL
        else:
            assert float(np.linalg.norm(got - ref) / np.linalg.norm(ref)) < FP16_REL_L2
        if dt == abi.F32:
            assert max_rel(got, want) < FP32_MAX_REL
        else:
            assert float(np.linalg.norm(got - want) / np.linalg.norm(want)) < FP16_REL_L2
        assert np.array_equal(got, want), "same kernels, same order of the K groups' sums: the results are the same bits"
    layer.close()


def test_noalloc_refuses_what_the_scratch_cannot_hold():
    C = F = 64
    w = synth.normal(9400, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9))))
    layer = Conv(abi.F32, w, 1, 1, relu=True, algo=abi.ALGO_WINOGRAD)  # its transformed tensors are the workspace
    N, H, W = 8, 56, 56  # 36 * tiles * (C + F) * 4 bytes = 29 MB
    xd = dev(synth.normal(9401, (N, H, W, C)), abi.F32)
    out = empty((N, H, W, F), abi.F32)
    out.fill_(7.0)
    torch.cuda.synchronize()
    rc = abi.lib().nncv_hip_conv_forward_noalloc(layer.h, xd.data_ptr(), N, H, W, None, out.data_ptr(), None)
    assert rc != 0
    msg = abi.lib().nncv_hip_last_error().decode()
    assert "scratch" in msg and "nncv_hip_conv_forward" in msg
    assert float(out.min()) == 7.0 and float(out.max()) == 7.0
    # a small case of the same layer fits: 36 * 4 tiles * 128 * 4 bytes
    got, want = run_pair(layer, abi.F32, 1, 8, 8, 9500)
    assert max_rel(got, want) < FP32_MAX_REL
    layer.close()


@pytest.mark.parametrize("dt", [abi.F32, abi.F16])
def test_noalloc_under_graph_capture(dt):
    """Two calls of the entry point recorded into one HIP graph on a capturing stream (kernel nodes only: the tickets are
    cleared by a fill kernel, the library neither waits for nor records events on a capturing stream), replayed three
    times with eager work and synchronisations in between; every replay gives the bits of nncv_hip_conv_forward."""
    C = F = 512
    w = synth.normal(9600, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9))))
    if dt == abi.F16:
        w = synth.round_fp16(w)
    layer = Conv(dt, w, 1, 1, relu=True, algo=abi.ALGO_IGEMM)
    shapes = ((1, 8, 8, 9700), (1, 4, 4, 9800))
    xs, wants, outs = [], [], []
    for (N, H, W, seed) in shapes:
        x = synth.normal(seed, (N, H, W, C))
        if dt == abi.F16:
            x = synth.round_fp16(x)
        xd = dev(x, dt)
        xs.append(xd)
        wants.append(host(layer(xd, abi.NHWC)))
        out = empty((N, H, W, F), dt)
        # once eagerly: one-time kernel attribute set-up must not fall into the capture
        abi.check(abi.lib().nncv_hip_conv_forward_noalloc(layer.h, xd.data_ptr(), N, H, W, None, out.data_ptr(), None))
        outs.append(out)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.graph(g, stream=side):
        s = torch.cuda.current_stream().cuda_stream
        for (N, H, W, _), xd, out in zip(shapes, xs, outs):
            abi.check(abi.lib().nncv_hip_conv_forward_noalloc(layer.h, xd.data_ptr(), N, H, W, None, out.data_ptr(), s))
    for rep in range(3):
        for out in outs:
            out.fill_(float(rep + 3))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for out, want in zip(outs, wants):
            assert np.array_equal(host(out), want), ("replay", rep)
        # the library's own eager work between replays
        assert np.array_equal(host(layer(xs[0], abi.NHWC)), wants[0])
    layer.close()
