"""The graph executor's workspace plan, checked on the host (nncv_hip_graph_plan touches no device).

The planner is the greedy-by-size offset calculation of the reference's MemSolver
(src/nncv/compiler/Utils/MemSolver.cpp:15-47); what is checked here is the executor's use of it: a launch
must never write memory that it reads.  Merged launches (convolution + ADD, squeeze-excitation blocks, the
chained 5x5 max-pools) write their result earlier than the operator list says, and the lifetimes handed to
the planner have to follow the launches, not the list.  The check below is written independently of the
library's own: it recomputes, from the operator list alone, which tensors each launch reads and writes.
"""
import numpy as np
import pytest

from nncv_amd import abi, mobilenetv3_spec, resnet18_spec, yolov5s_spec

import graph_gen


def _ranges_clash(info, a, b):
    ra, oa, ba, ca = info[a]
    rb, ob, bb, cb = info[b]
    if ra == rb:
        return True  # same block: the caller decides (slices of one concatenated tensor)
    return ba > 0 and bb > 0 and oa < ob + bb and ob < oa + ba


def _check(ops, cin, dt, N, H, W):
    total, info, dst = abi.graph_plan(ops, cin, dt, N, H, W)
    es = 2 if dt == abi.F16 else 4
    n = len(ops)
    # block start = offset of the tensor minus its channel offset inside the block
    blk = [(r, o - c0 * es, b, c0) for (r, o, b, c0) in info]
    for t, (r, o, b, c0) in enumerate(blk):
        assert o >= 0 and o + b <= total, "tensor %d lies outside the workspace" % t
    for i, op in enumerate(ops):
        d = dst[i]
        if d < 0:
            continue
        reads = [t for t in op.inputs if t >= 0]
        if d != op.out:  # merged launch: it also reads what the merged operators read from outside
            j = i + 1
            while j < n and dst[j] < 0 and ops[j].kind != abi.OP_YOLO_DETECT:
                reads += [t for t in ops[j].inputs if t >= 0 and t not in [o2.out for o2 in ops[i:j + 1]]]
                j += 1
        for t in reads:
            if blk[t][0] == blk[d][0]:
                # slices of one concatenated tensor (or the very same tensor, which no launch may do)
                assert t != d, "operator %d reads and writes tensor %d" % (i, d)
                continue
            assert not _ranges_clash(blk, d, t), (
                "operator %d (%s): result tensor %d at [%d, +%d) overlaps its input tensor %d at [%d, +%d)"
                % (i, op.kind, d, blk[d][1], blk[d][2], t, blk[t][1], blk[t][2]))
    return total


@pytest.mark.parametrize("dt", [abi.F16, abi.F32])
@pytest.mark.parametrize("shape", [(1, 640, 640), (16, 640, 640), (2, 320, 256), (1, 64, 96), (8, 640, 640)])
def test_yolov5s_plan_never_lays_a_result_over_an_input(dt, shape):
    N, H, W = shape
    total = _check(yolov5s_spec.graph_ops(), 3, dt, N, H, W)
    assert total > 0


@pytest.mark.parametrize("dt", [abi.F16, abi.F32])
@pytest.mark.parametrize("shape", [(1, 224, 224), (32, 224, 224), (3, 100, 77), (1, 256, 256)])
def test_mobilenetv3_and_resnet18_plans(dt, shape):
    N, H, W = shape
    assert _check(mobilenetv3_spec.graph_ops(), 3, dt, N, H, W) > 0
    assert _check(resnet18_spec.graph_ops(), 3, dt, N, H, W) > 0


def test_random_operator_lists_plan_cleanly():
    done = 0
    for seed in range(400):
        for f16 in (False, True):
            case = graph_gen.random_case(9000 + seed, f16)
            if case is None:
                continue
            ops, cin, blob, x = case
            _check(ops, cin, abi.F16 if f16 else abi.F32, x.shape[0], x.shape[2], x.shape[3])
            done += 1
    assert done > 300


def test_merged_bottleneck_result_is_live_from_the_convolution():
    """x -> conv1x1 -> conv3x3 -> ADD(x, .) (a YOLOv5 Bottleneck): the 3x3 convolution's launch writes the
    ADD's tensor, so that tensor must not reuse the memory of the 3x3 convolution's input, which dies at
    the same launch."""
    C = 64
    ops, off = [], [0]

    def take(n):
        o = off[0]; off[0] += n; return o

    ops.append(abi.graph_op(abi.OP_CONV, [0, -1], 1, F=C, K=3, stride=1, pad=1, act=abi.ACT_SILU, w=take(C * 8 * 9), bias=take(C)))
    ops.append(abi.graph_op(abi.OP_CONV, [1, -1], 2, F=C, K=1, stride=1, pad=0, act=abi.ACT_SILU, w=take(C * C), bias=take(C)))
    ops.append(abi.graph_op(abi.OP_CONV, [2, -1], 3, F=C, K=3, stride=1, pad=1, act=abi.ACT_SILU, w=take(C * C * 9), bias=take(C)))
    ops.append(abi.graph_op(abi.OP_ADD, [1, 3], 4))
    ops.append(abi.graph_op(abi.OP_CONV, [4, -1], 5, F=C, K=1, stride=1, pad=0, act=abi.ACT_NONE, w=take(C * C), bias=take(C)))
    total, info, dst = abi.graph_plan(ops, 8, abi.F16, 4, 40, 40)
    assert dst[2] == 4 and dst[3] == -1, "the ADD should ride in the convolution's epilogue"
    o2, b2 = info[2][1], info[2][2]
    o4, b4 = info[4][1], info[4][2]
    assert o4 + b4 <= o2 or o2 + b2 <= o4, "the merged result shares memory with the convolution's input"
    _check(ops, 8, abi.F16, 4, 40, 40)
