"""YOLOv5s (the network of the reference's fixture tests/Nets/Yolov5s.mlir) through the graph
executor on the GPU against the oracle's operator-list evaluator."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from nncv_amd import yolov5s_spec as spec
from gpu_util import Graph, dev, host, max_rel, rel_l2, FP32_MAX_REL, FP16_REL_L2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def blob():
    return synth.yolov5s_params()


def check_fp32(got, want):
    assert got.shape == want.shape
    # boxes (pixels) and scores (sigmoids in [0,1]) are judged each against its own scale
    e_box, e_sc = max_rel(got[..., :4], want[..., :4]), float(np.abs(got[..., 4:] - want[..., 4:]).max())
    print("box max_rel", e_box, "score max abs", e_sc, flush=True)
    assert e_box < FP32_MAX_REL and e_sc < FP32_MAX_REL


@pytest.mark.parametrize("shape", [(2, 3, 64, 96), (1, 3, 160, 128)])
def test_yolov5s_fp32_small(blob, shape):
    g = Graph(spec.graph_ops(), 3, blob, abi.F32)
    H, W = shape[2:]
    boxes = 3 * ((H // 8) * (W // 8) + (H // 16) * (W // 16) + (H // 32) * (W // 32))
    assert abi.graph_output_shape(g.h, H, W) == (boxes, 85, 1)
    x = synth.uniform(8200, shape, 0.0, 1.0)
    print("yolov5s fp32", shape, flush=True)
    got = host(g(dev(x))).reshape(shape[0], boxes, 85)
    check_fp32(got, oracle.run_graph(spec.graph_ops(), x, blob, 3))
    g.close()


def test_yolov5s_fp32_fixture_shape(blob):
    """[1,3,640,640] -> [1,25200,85], the signature of the fixture's @forward."""
    g = Graph(spec.graph_ops(), 3, blob, abi.F32)
    x = synth.uniform(8201, (1, 3, 640, 640), 0.0, 1.0)
    print("yolov5s fp32 640", flush=True)
    got = host(g(dev(x))).reshape(1, 25200, 85)
    check_fp32(got, oracle.run_graph(spec.graph_ops(), x, blob, 3, conv=oracle.hwp_conv2d))
    g.close()


def test_yolov5s_fp16(blob):
    b16 = synth.round_fp16(blob)
    g = Graph(spec.graph_ops(), 3, b16, abi.F16)
    shape = (2, 3, 320, 256)
    x = synth.round_fp16(synth.uniform(8202, shape, 0.0, 1.0))
    print("yolov5s fp16", shape, flush=True)
    xd = dev(x, abi.F16)
    got = host(g(xd)).reshape(2, -1, 85)
    want = oracle.run_graph(spec.graph_ops(), x, b16, 3, conv=oracle.hwp_conv2d)
    e_box, e_sc = rel_l2(got[..., :4], want[..., :4]), rel_l2(got[..., 4:], want[..., 4:])
    print("box rel_l2", e_box, "score rel_l2", e_sc, flush=True)
    assert e_box < FP16_REL_L2 and e_sc < FP16_REL_L2
    # the most confident box of every image is the same one
    assert np.array_equal(got[..., 4].argmax(1), want[..., 4].argmax(1))
    for it in range(3):  # HIP-graph replays reproduce the eager pass
        torch.randn(1 << 18, device="cuda").sum().item()
        assert np.array_equal(host(g(xd)).reshape(2, -1, 85), got), it
    g.close()


def test_yolov5s_fp16_batch8_at_640_every_image(blob):
    """Launches of several rounds of workgroups per CU (batch 8 at 640x640): a launch that wrote over
    its own input would only show at such sizes, where the workgroups of one launch no longer all run
    at the same time.  Image 0 of the batch against the oracle, every image against the same image
    sent alone (images are independent of each other)."""
    b16 = synth.round_fp16(blob)
    g = Graph(spec.graph_ops(), 3, b16, abi.F16)
    x = synth.round_fp16(synth.uniform(8203, (8, 3, 640, 640), 0.0, 1.0))
    print("yolov5s fp16 batch 8 at 640", flush=True)
    got = host(g(dev(x, abi.F16))).reshape(8, 25200, 85)
    assert np.isfinite(got).all()
    for n in range(8):
        alone = host(g(dev(x[n:n + 1], abi.F16))).reshape(25200, 85)
        e = rel_l2(got[n], alone)
        print("image", n, "batched vs alone rel_l2", e, flush=True)
        assert e < 2e-3, n
    want = oracle.run_graph(spec.graph_ops(), x[:1], b16, 3, conv=oracle.hwp_conv2d)[0]
    e_box, e_sc = rel_l2(got[0][:, :4], want[:, :4]), rel_l2(got[0][:, 4:], want[:, 4:])
    print("image 0 vs oracle: box rel_l2", e_box, "score rel_l2", e_sc, flush=True)
    assert e_box < FP16_REL_L2 and e_sc < FP16_REL_L2
    g.close()


def test_detect_refuses_being_in_the_middle(blob):
    ops = spec.graph_ops()
    extra = abi.graph_op(abi.OP_ACT, [ops[-1].out], ops[-1].out + 1, stride=0)
    with pytest.raises(abi.NncvHipError) as e:
        abi.graph_create(ops + [extra], 3, blob)
    assert "last operator" in str(e.value)
