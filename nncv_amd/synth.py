"""Seeded synthetic inputs and weights for the benchmark configurations.

A self-contained counter-based generator (splitmix64 -> uniform / Box-Muller normal, evaluated in
numpy float64 and rounded once to float32) so that fixtures do not depend on any library's RNG
stream.  Element i of stream `seed` depends only on (seed, i).
"""
import numpy as np

from . import resnet18_spec as spec

_G = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(x):
    with np.errstate(over="ignore"):
        z = x + _G
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _bits(seed, n, lane):
    """n 64-bit words of stream (seed, lane)."""
    with np.errstate(over="ignore"):
        key = _mix(np.uint64(seed) * np.uint64(2) + np.uint64(lane))
        ctr = np.arange(n, dtype=np.uint64) * _G
        return _mix(key + ctr)


def uniform01(seed, shape):
    n = int(np.prod(shape))
    u = (_bits(seed, n, 0) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    return u.reshape(shape)


def uniform(seed, shape, lo, hi):
    return (lo + (hi - lo) * uniform01(seed, shape)).astype(np.float32)


def normal(seed, shape, std=1.0, mean=0.0):
    n = int(np.prod(shape))
    u1 = ((_bits(seed, n, 0) >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / (1 << 53))
    u2 = (_bits(seed, n, 1) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (mean + std * z).astype(np.float32).reshape(shape)


def round_fp16(a):
    """Round-to-nearest-even to IEEE half, returned as float32."""
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


# ---- BASELINE configurations -------------------------------------------------------------------

def cfg1_matmul(n=1024):
    """fp32 C[n,n] = A.B, A and B uniform[-1,1]; C starts at zero (linalg.matmul accumulates)."""
    return uniform(1001, (n, n), -1.0, 1.0), uniform(1002, (n, n), -1.0, 1.0)


def cfg2_conv(n=1, c=64, h=56, f=64):
    """3x3 s1 p1 conv: input N(0,1), filter N(0,1)*sqrt(2/(c*9))."""
    x = normal(2001, (n, c, h, h))
    w = normal(2002, (f, c, 3, 3), std=float(np.sqrt(2.0 / (c * 9))))
    return x, w


def resnet18_params(seed_base=3100):
    """Flat fp32 parameter blob in the canonical order.

    conv: Kaiming normal, std = sqrt(2/fan_in), fan_in = C*R*S;  fc.weight N(0, 0.01), fc.bias 0;
    BN gamma U(0.5,1.5), beta N(0,0.1), running_mean N(0,0.1), running_var U(0.5,1.5).
    Tensor k of the table uses seed seed_base + k.
    """
    parts = []
    for k, (name, shape) in enumerate(spec.tensor_table()):
        seed = seed_base + k
        if name.endswith("conv1.weight") or name.endswith("conv2.weight") \
                or name.endswith("downsample.0.weight"):
            fan_in = shape[1] * shape[2] * shape[3]
            a = normal(seed, shape, std=float(np.sqrt(2.0 / fan_in)))
        elif name == "fc.weight":
            a = normal(seed, shape, std=0.01)
        elif name == "fc.bias":
            a = np.zeros(shape, np.float32)
        elif name.endswith("running_var"):
            a = uniform(seed, shape, 0.5, 1.5)
        elif name.endswith("running_mean"):
            a = normal(seed, shape, std=0.1)
        elif name.endswith(".weight"):  # BN gamma
            a = uniform(seed, shape, 0.5, 1.5)
        elif name.endswith(".bias"):  # BN beta
            a = normal(seed, shape, std=0.1)
        else:
            raise AssertionError(name)
        parts.append(a.reshape(-1))
    blob = np.concatenate(parts)
    assert blob.size == spec.NUM_ELEMENTS
    return blob


def mobilenetv3_params(seed_base=6100):
    """Flat fp32 parameter blob of MobileNetV3-small in the canonical order (mobilenetv3_spec).

    conv / Linear weights: Kaiming normal, std = sqrt(2/fan_in) (fan_in = K*K for depthwise filters);
    conv / Linear biases N(0, 0.1); BN as in resnet18_params.  Tensor k uses seed seed_base + k."""
    from . import mobilenetv3_spec as m
    parts = []
    for k, (name, shape) in enumerate(m.tensor_table()):
        seed = seed_base + k
        if len(shape) >= 2:
            fan_in = int(np.prod(shape[1:]))
            a = normal(seed, shape, std=float(np.sqrt(2.0 / fan_in)))
        elif name.endswith("running_var"):
            a = uniform(seed, shape, 0.5, 1.5)
        elif name.endswith("running_mean"):
            a = normal(seed, shape, std=0.1)
        elif name.endswith(".weight"):  # BN gamma
            a = uniform(seed, shape, 0.5, 1.5)
        elif name.endswith(".bias"):  # BN beta, squeeze-excitation and classifier biases
            a = normal(seed, shape, std=0.1)
        else:
            raise AssertionError(name)
        parts.append(a.reshape(-1))
    blob = np.concatenate(parts)
    assert blob.size == m.NUM_ELEMENTS
    return blob


def yolov5s_params(seed_base=8100):
    """Flat fp32 parameter blob of YOLOv5s in the canonical order (yolov5s_spec).  Convolution weights
    Kaiming normal std = sqrt(2/fan_in) (the BatchNorm is already fused in this network's table), biases
    N(0, 0.1) -- the three Detect biases N(0, 1) so that the decoded boxes spread over their range --,
    anchors and strides the published yolov5s.yaml values."""
    from . import yolov5s_spec as y
    parts = []
    for k, (name, shape) in enumerate(y.tensor_table()):
        seed = seed_base + k
        if name == "model.24.anchors":
            a = np.array([[v / y.STRIDES[l] for v in y.ANCHORS_PX[l]] for l in range(3)], np.float32).reshape(shape)
        elif name == "model.24.stride":
            a = np.array(y.STRIDES, np.float32)
        elif len(shape) == 4:
            a = normal(seed, shape, std=float(np.sqrt(2.0 / int(np.prod(shape[1:])))))
        else:
            a = normal(seed, shape, std=1.0 if name.startswith("model.24.") else 0.1)
        parts.append(a.reshape(-1))
    blob = np.concatenate(parts)
    assert blob.size == y.NUM_ELEMENTS
    return blob


def cfg3_input():
    return uniform(3000, (1, 3, 256, 256), 0.0, 1.0)


def cfg4_input(n=32):
    return uniform(4000, (n, 3, 224, 224), 0.0, 1.0)


CFG5_LAYERS = [  # (C, K, H, stride)
    (64, 64, 56, 1), (64, 128, 56, 2), (128, 128, 28, 1), (128, 256, 28, 2),
    (256, 256, 14, 1), (256, 512, 14, 2), (512, 512, 7, 1)]


def cfg5_layer(i, n=64):
    """Layer i of the fp16 3x3 sweep: x, w, BN (gamma, beta, mean, var), residual or None."""
    c, k, h, s = CFG5_LAYERS[i]
    seed = 5000 + 10 * i
    x = round_fp16(normal(seed, (n, c, h, h)))
    w = round_fp16(normal(seed + 1, (k, c, 3, 3), std=float(np.sqrt(2.0 / (c * 9)))))
    bn = (uniform(seed + 2, (k,), 0.5, 1.5), normal(seed + 3, (k,), std=0.1),
          normal(seed + 4, (k,), std=0.1), uniform(seed + 5, (k,), 0.5, 1.5))
    oh = (h + 2 - 3) // s + 1
    res = round_fp16(normal(seed + 6, (n, k, oh, oh))) if s == 1 else None
    return x, w, bn, res
