"""Seeded random operator lists for the graph executor's parity tests: convolutions (1x1 / 3x3 / 5x5, stride 1 / 2, with
bias and / or BatchNorm, any fused activation, optional residual), depthwise convolutions, max-pools, adds, activations,
channel concatenations of 2-4 earlier tensors, up-sampling and squeeze-excitation blocks, wired to random earlier
tensors -- so concatenation views, add fusion, SE fusion and their fallbacks meet in combinations no network has."""
import numpy as np

from nncv_amd import abi, synth


def random_graph(rng, vn):
    """-> ops, blob size, input shape.  Tensors are tracked as id -> (C, H, W) for a fixed input size."""
    cin = int(rng.choice([3, vn, 2 * vn]))
    H, W = int(rng.integers(9, 25)), int(rng.integers(9, 25))
    dims = {0: (cin, H, W)}
    ops, sizes = [], []

    def take(n):
        off = sum(sizes); sizes.append(n); return off

    nxt = 1
    chans = [vn, 2 * vn, 3 * vn, 4 * vn]
    for step in range(int(rng.integers(4, 14))):
        ids = list(dims)
        kind = rng.choice(["conv", "conv", "conv", "dw", "pool", "add", "act", "cat", "up", "se", "convres"])
        a = int(rng.choice(ids))
        C, h, w = dims[a]
        out = nxt
        if kind in ("conv", "convres"):
            F = int(rng.choice(chans)); k = int(rng.choice([1, 1, 3, 3, 5])); s = int(rng.choice([1, 1, 2]))
            p = (k - 1) // 2
            oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
            if oh < 1 or ow < 1: continue
            res = -1
            if kind == "convres":
                cands = [t for t in ids if dims[t] == (F, oh, ow) and t != 0]
                if not cands: continue
                res = int(rng.choice(cands))
            bn = tuple(take(F) for _ in range(4)) if rng.random() < 0.5 else None
            bias = take(F) if (bn is None or rng.random() < 0.3) else -1
            ops.append(abi.graph_op(abi.OP_CONV, [a, res], out, F=F, K=k, stride=s, pad=p, act=int(rng.integers(0, 6)), eps=1e-3,
                                    w=take(F * C * k * k), bias=bias, bn=bn))
            dims[out] = (F, oh, ow)
        elif kind == "dw":
            if a == 0 or C % vn: continue
            k = int(rng.choice([3, 5])); s = int(rng.choice([1, 2])); p = (k - 1) // 2
            oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
            if oh < 1 or ow < 1: continue
            bn = tuple(take(C) for _ in range(4))
            ops.append(abi.graph_op(abi.OP_DWCONV, [a], out, F=C, K=k, stride=s, pad=p, act=int(rng.integers(0, 5)), eps=1e-3,
                                    w=take(C * k * k), bn=bn))
            dims[out] = (C, oh, ow)
        elif kind == "pool":
            if a == 0 or C % vn: continue
            k, s, p = [(3, 2, 1), (5, 1, 2), (2, 2, 0), (3, 1, 1)][int(rng.integers(0, 4))]
            if h + 2 * p < k or w + 2 * p < k: continue
            ops.append(abi.graph_op(abi.OP_MAXPOOL, [a], out, K=k, stride=s, pad=p))
            dims[out] = (C, (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1)
        elif kind == "add":
            cands = [t for t in ids if dims[t] == dims[a] and t != 0]
            if a == 0 or not cands or C % vn: continue
            ops.append(abi.graph_op(abi.OP_ADD, [a, int(rng.choice(cands))], out, act=int(rng.integers(0, 3)), stride=0))
            dims[out] = dims[a]
        elif kind == "act":
            if a == 0 or C % vn: continue
            ops.append(abi.graph_op(abi.OP_ACT, [a], out, act=int(rng.integers(1, 6)), stride=0))
            dims[out] = dims[a]
        elif kind == "cat":
            cands = [t for t in ids if dims[t][1:] == (h, w) and t != 0 and dims[t][0] % vn == 0]
            if a == 0 or C % vn or len(cands) < 2: continue
            n_in = int(rng.integers(2, min(4, len(cands)) + 1))
            ins = [int(t) for t in rng.choice(cands, size=n_in, replace=False)]
            ops.append(abi.graph_op(abi.OP_CONCAT, ins, out, stride=0))
            dims[out] = (sum(dims[t][0] for t in ins), h, w)
        elif kind == "up":
            if a == 0 or C % vn or h * w > 400: continue
            ops.append(abi.graph_op(abi.OP_UPSAMPLE2X, [a], out, stride=0))
            dims[out] = (C, 2 * h, 2 * w)
        elif kind == "se":
            if a == 0 or C % vn: continue
            sq = vn * int(rng.integers(1, 3))
            ops.append(abi.graph_op(abi.OP_GAVGPOOL, [a], out, stride=0))
            ops.append(abi.graph_op(abi.OP_CONV, [out], out + 1, F=sq, K=1, act=abi.ACT_RELU, w=take(sq * C), bias=take(sq)))
            ops.append(abi.graph_op(abi.OP_CONV, [out + 1], out + 2, F=C, K=1, act=abi.ACT_HARDSIGMOID, w=take(C * sq), bias=take(C)))
            ops.append(abi.graph_op(abi.OP_SCALE, [a, out + 2], out + 3, stride=0))
            dims[out] = dims[out + 1] = dims[out + 2] = (C, 1, 1)  # placeholders: only out+3 is offered to later ops
            dims.pop(out); dims.pop(out + 1); dims.pop(out + 2)
            dims[out + 3] = (C, h, w)
            nxt += 3
        nxt += 1
    if not ops or ops[-1].out not in dims:
        return None
    return ops, sum(sizes), (cin, H, W)


def random_case(seed, f16):
    """-> (ops, in_channels, blob, x) or None when the seed produced no usable graph."""
    rng = np.random.default_rng(seed)
    g = random_graph(rng, 8 if f16 else 4)
    if g is None:
        return None
    ops, nparam, (cin, H, W) = g
    blob = synth.normal(seed, (max(nparam, 1),), std=0.25)
    for o in ops:
        if o.var >= 0:
            blob[o.var:o.var + o.F] = synth.uniform(seed + 1, (o.F,), 0.5, 1.5)
    x = synth.normal(seed + 2, (int(rng.integers(1, 4)), cin, H, W))
    if f16:
        blob, x = synth.round_fp16(blob), synth.round_fp16(x)
    return ops, cin, blob, x
