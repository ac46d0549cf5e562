"""ctypes binding of libnncv_hip.so (include/nncv_hip.h) — the same structs and entry points a
C or C++ caller of nncv uses, so tests read like calls into the reference's object.

There is no fallback: if the library is missing or cannot be loaded this module raises.
"""
import ctypes
import os
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnncv_hip.so")

F32, F16 = 1, 2
NCHW, NHWC = 0, 1
ALGO_AUTO, ALGO_WINOGRAD, ALGO_IGEMM = 0, 1, 2

c_intptr = ctypes.c_ssize_t


def _memref(rank):
    class MemRef(ctypes.Structure):
        _fields_ = [("allocated", ctypes.c_void_p), ("aligned", ctypes.c_void_p), ("offset", c_intptr),
                    ("sizes", c_intptr * rank), ("strides", c_intptr * rank)]
    MemRef.__name__ = "MemRef%dD" % rank
    return MemRef


MemRef1D, MemRef2D, MemRef4D = _memref(1), _memref(2), _memref(4)
assert ctypes.sizeof(MemRef1D) == 40 and ctypes.sizeof(MemRef2D) == 56 and ctypes.sizeof(MemRef4D) == 88

EXPORTS = [
    "_mlir_ciface_forward", "_mlir_ciface_forward_f16", "_mlir_ciface_matmul", "_mlir_ciface_batch_nchw_conv",
    "nncv_hip_init", "nncv_hip_last_error", "nncv_hip_device_arch",
    "nncv_hip_profile_enable", "nncv_hip_profile_report",
    "nncv_hip_resnet18_create", "nncv_hip_resnet18_clone", "nncv_hip_resnet18_destroy", "nncv_hip_resnet18_forward",
    "nncv_hip_resnet18_forward_tap",
    "nncv_hip_conv_create", "nncv_hip_conv_destroy", "nncv_hip_conv_algo", "nncv_hip_conv_forward", "nncv_hip_conv_forward_noalloc", "nncv_hip_conv_time", "nncv_hip_conv3x3_patch_plan", "nncv_hip_conv3x3_stream_plan", "nncv_hip_params_invalidate", "nncv_hip_set_overlap_hint", "nncv_hip_resnet18_create_ex", "nncv_hip_resnet18_passes_in_flight", "nncv_hip_pick_streams",
    "nncv_hip_plan_arena", "nncv_hip_preprocess_u8", "nncv_hip_argmax", "nncv_hip_resnet18_classify_u8",
    "nncv_hip_matmul_f32", "nncv_hip_matmul_time", "nncv_hip_wino43_filter", "nncv_hip_wino43_input", "nncv_hip_wino43_gemm",
    "nncv_hip_wino43_output", "nncv_hip_maxpool3x3s2", "nncv_hip_global_avgpool",
    "nncv_hip_graph_create", "nncv_hip_graph_destroy", "nncv_hip_graph_output_shape", "nncv_hip_graph_forward",
    "nncv_hip_graph_plan", "nncv_hip_mobilenetv3_small_ops", "nncv_hip_dwconv", "nncv_hip_scale_channels", "nncv_hip_eltwise",
    "nncv_hip_concat_slice", "nncv_hip_upsample2x", "nncv_hip_maxpool",
]

# operator kinds / activations of nncv_hip_graph_op (include/nncv_hip.h)
OP_CONV, OP_DWCONV, OP_MAXPOOL, OP_GAVGPOOL, OP_SCALE, OP_ADD, OP_ACT, OP_CONCAT, OP_UPSAMPLE2X, OP_YOLO_DETECT = range(1, 11)
ACT_NONE, ACT_RELU, ACT_HARDSWISH, ACT_HARDSIGMOID, ACT_SILU, ACT_SIGMOID = range(6)


class GraphOp(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("inputs", ctypes.c_int32 * 4), ("out", ctypes.c_int32), ("F", ctypes.c_int32),
                ("K", ctypes.c_int32), ("stride", ctypes.c_int32), ("pad", ctypes.c_int32), ("act", ctypes.c_int32),
                ("eps", ctypes.c_float), ("w", ctypes.c_int64), ("bias", ctypes.c_int64), ("gamma", ctypes.c_int64),
                ("beta", ctypes.c_int64), ("mean", ctypes.c_int64), ("var", ctypes.c_int64)]


assert ctypes.sizeof(GraphOp) == 96


def graph_op(kind, inputs, out, F=0, K=0, stride=1, pad=0, act=ACT_NONE, eps=0.0, w=-1, bias=-1, bn=None):
    """One nncv_hip_graph_op; bn = (gamma, beta, mean, var) element offsets."""
    o = GraphOp()
    o.kind, o.out, o.F, o.K, o.stride, o.pad, o.act, o.eps = kind, out, F, K, stride, pad, act, eps
    ins = list(inputs) + [-1] * (4 - len(inputs))
    for k in range(4):
        o.inputs[k] = ins[k]
    o.w, o.bias = w, bias
    o.gamma, o.beta, o.mean, o.var = bn if bn is not None else (-1, -1, -1, -1)
    return o

_lib = None


def lib():
    """Load the library (never builds, never falls back)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m nncv_amd.build` (needs hipcc)" % LIB_PATH)
        # A process must hold ONE HIP runtime.  PyTorch ships its own copy of it: imported AFTER this library was loaded
        # (which brings in the system's copy), torch finds "no HIP GPUs"; imported before, both use torch's copy.
        if "torch" not in sys.modules:
            try:
                import torch  # noqa: F401
            except ImportError:
                pass
        L = ctypes.CDLL(LIB_PATH)
        vp, i, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
        P = ctypes.POINTER
        L._mlir_ciface_forward.argtypes = [P(MemRef2D), P(MemRef4D), vp]
        L._mlir_ciface_forward.restype = None
        L._mlir_ciface_forward_f16.argtypes = [P(MemRef2D), P(MemRef4D), vp]
        L._mlir_ciface_forward_f16.restype = None
        L._mlir_ciface_matmul.argtypes = [P(MemRef2D)] * 4
        L._mlir_ciface_matmul.restype = None
        L._mlir_ciface_batch_nchw_conv.argtypes = [P(MemRef4D)] * 4
        L._mlir_ciface_batch_nchw_conv.restype = None
        L.nncv_hip_init.argtypes = [i]
        L.nncv_hip_params_invalidate.argtypes = [vp]
        L.nncv_hip_set_overlap_hint.argtypes = [i]
        L.nncv_hip_last_error.restype = ctypes.c_char_p
        L.nncv_hip_device_arch.restype = ctypes.c_char_p
        L.nncv_hip_profile_enable.argtypes = [i]
        L.nncv_hip_profile_enable.restype = None
        L.nncv_hip_profile_report.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
        L.nncv_hip_profile_report.restype = ctypes.c_size_t
        L.nncv_hip_resnet18_create.argtypes = [vp, i64, i, i]
        L.nncv_hip_resnet18_create.restype = vp
        L.nncv_hip_resnet18_clone.argtypes = [vp]
        L.nncv_hip_resnet18_clone.restype = vp
        L.nncv_hip_resnet18_create_ex.argtypes = [vp, i64, i, i, i]
        L.nncv_hip_resnet18_create_ex.restype = vp
        L.nncv_hip_resnet18_passes_in_flight.argtypes = [vp]
        L.nncv_hip_pick_streams.argtypes = [i, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_int)]
        L.nncv_hip_resnet18_destroy.argtypes = [vp]
        L.nncv_hip_resnet18_destroy.restype = None
        L.nncv_hip_resnet18_forward.argtypes = [vp, vp, i, i, i, vp, vp]
        L.nncv_hip_resnet18_forward_tap.argtypes = [vp, vp, i, i, i, vp, i, vp, vp]
        L.nncv_hip_conv_create.argtypes = [i, vp, i, i, i, i, i, i, vp, vp, vp, vp, i, i]
        L.nncv_hip_conv_create.restype = vp
        L.nncv_hip_conv_destroy.argtypes = [vp]
        L.nncv_hip_conv_destroy.restype = None
        L.nncv_hip_conv_algo.argtypes = [vp]
        L.nncv_hip_conv_forward.argtypes = [vp, vp, i, i, i, i, vp, vp, vp]
        L.nncv_hip_conv_forward_noalloc.argtypes = [vp, vp, i, i, i, vp, vp, vp]
        L.nncv_hip_conv_time.argtypes = [vp, vp, i, i, i, vp, vp, i, vp, P(ctypes.c_float)]
        L.nncv_hip_matmul_f32.argtypes = [vp, vp, vp, i, i, i, vp]
        L.nncv_hip_matmul_time.argtypes = [vp, vp, vp, i, i, i, i, vp, ctypes.POINTER(ctypes.c_float)]
        L.nncv_hip_plan_arena.argtypes = [i, P(i), P(i), P(ctypes.c_uint64), ctypes.c_uint64, P(ctypes.c_uint64)]
        L.nncv_hip_plan_arena.restype = ctypes.c_uint64
        L.nncv_hip_preprocess_u8.argtypes = [vp, i, i, i, i, i, vp, vp]
        L.nncv_hip_argmax.argtypes = [vp, i, i, vp, vp]
        L.nncv_hip_resnet18_classify_u8.argtypes = [vp, vp, i, i, i, i, vp, vp, vp]
        L.nncv_hip_wino43_filter.argtypes = [i, vp, vp, i, i, vp]
        L.nncv_hip_wino43_input.argtypes = [i, vp, i, vp, i, i, i, i, i, vp]
        L.nncv_hip_wino43_gemm.argtypes = [i, vp, vp, vp, i64, i, i, vp]
        L.nncv_hip_wino43_output.argtypes = [i, vp, vp, i, i, i, i, i, vp, vp, vp, i, vp]
        L.nncv_hip_maxpool3x3s2.argtypes = [i, vp, vp, i, i, i, i, vp]
        L.nncv_hip_global_avgpool.argtypes = [i, vp, vp, i, i, i, i, vp]
        L.nncv_hip_graph_create.argtypes = [P(GraphOp), i, i, vp, i64, i]
        L.nncv_hip_graph_create.restype = vp
        L.nncv_hip_graph_destroy.argtypes = [vp]
        L.nncv_hip_graph_destroy.restype = None
        L.nncv_hip_graph_output_shape.argtypes = [vp, i, i, P(i)]
        L.nncv_hip_graph_forward.argtypes = [vp, vp, i, i, i, vp, i64, vp]
        L.nncv_hip_graph_plan.argtypes = [P(GraphOp), i, i, i, i, i, i, P(i64), i, P(ctypes.c_int32)]
        L.nncv_hip_graph_plan.restype = i64
        L.nncv_hip_mobilenetv3_small_ops.argtypes = [P(GraphOp), i, P(i64)]
        L.nncv_hip_dwconv.argtypes = [i, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, i, vp]
        L.nncv_hip_scale_channels.argtypes = [i, vp, vp, vp, i, i, i, vp]
        L.nncv_hip_eltwise.argtypes = [i, vp, vp, vp, i64, i, vp]
        L.nncv_hip_concat_slice.argtypes = [i, vp, vp, i64, i, i, i, vp]
        L.nncv_hip_upsample2x.argtypes = [i, vp, vp, i, i, i, i, i, i, vp]
        L.nncv_hip_maxpool.argtypes = [i, vp, vp, i, i, i, i, i, i, i, vp]
        _lib = L
    return _lib


class NncvHipError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        raise NncvHipError(lib().nncv_hip_last_error().decode())


def profile_enable(on):
    lib().nncv_hip_profile_enable(1 if on else 0)


def profile_report():
    """-> {tag: {"launches", "ms", "flops", "bytes"}} since the last report."""
    import json
    buf = ctypes.create_string_buffer(1 << 16)
    lib().nncv_hip_profile_report(buf, len(buf))
    return json.loads(buf.value.decode())


def np_dtype(dt):
    return np.float16 if dt == F16 else np.float32


# ---- host memref helpers (for the reference ABI) ------------------------------------------------

def memref_of(a):
    """Descriptor over a numpy array (any strides); keeps no reference — keep `a` alive."""
    cls = {1: MemRef1D, 2: MemRef2D, 4: MemRef4D}[a.ndim]
    m = cls()
    m.allocated = m.aligned = a.ctypes.data
    m.offset = 0
    for k in range(a.ndim):
        m.sizes[k] = a.shape[k]
        m.strides[k] = a.strides[k] // a.itemsize
    return m


def memref_to_numpy(m, dtype):
    """View of a dense rank-2 result descriptor (the buffer was malloc'd by the callee)."""
    n = m.sizes[0] * m.sizes[1]
    buf = (ctypes.c_char * (n * np.dtype(dtype).itemsize)).from_address(m.aligned)
    return np.frombuffer(buf, dtype=dtype).reshape(m.sizes[0], m.sizes[1])


_libc = ctypes.CDLL(None)
_libc.free.argtypes = [ctypes.c_void_p]


def forward(x, params_blob):
    """_mlir_ciface_forward / _f16 on host arrays: x [N,3,H,W], params flat blob -> logits [N,1000].
    The element type (float32 / float16) selects the entry point."""
    assert x.dtype == params_blob.dtype and x.dtype in (np.float32, np.float16)
    src = memref_of(x)
    par = memref_of(params_blob)
    dst = MemRef2D()
    fn = lib()._mlir_ciface_forward if x.dtype == np.float32 else lib()._mlir_ciface_forward_f16
    fn(ctypes.byref(dst), ctypes.byref(src), ctypes.cast(ctypes.byref(par), ctypes.c_void_p))
    out = memref_to_numpy(dst, x.dtype).copy()
    _libc.free(dst.allocated)  # the caller owns the callee-allocated result
    return out


def matmul(a, b, c):
    """_mlir_ciface_matmul: c += a @ b in place (fp32 host arrays); returns the aliasing result view."""
    res = MemRef2D()
    ma, mb, mc = memref_of(a), memref_of(b), memref_of(c)
    lib()._mlir_ciface_matmul(ctypes.byref(res), ctypes.byref(ma), ctypes.byref(mb), ctypes.byref(mc))
    assert res.aligned == mc.aligned
    return c


def batch_nchw_conv(x_padded, w, out):
    """_mlir_ciface_batch_nchw_conv: out += conv(x_padded, w) in place (fp32 host arrays)."""
    res = MemRef4D()
    mi, mw, mo = memref_of(x_padded), memref_of(w), memref_of(out)
    lib()._mlir_ciface_batch_nchw_conv(ctypes.byref(res), ctypes.byref(mi), ctypes.byref(mw), ctypes.byref(mo))
    assert res.aligned == mo.aligned
    return out


def plan_arena(lives, align=1):
    """lives: [(first_op, last_op, bytes)] -> (total, [offsets]) by nncv_hip_plan_arena."""
    n = len(lives)
    first = (ctypes.c_int * n)(*[l[0] for l in lives])
    last = (ctypes.c_int * n)(*[l[1] for l in lives])
    size = (ctypes.c_uint64 * n)(*[l[2] for l in lives])
    off = (ctypes.c_uint64 * n)()
    total = lib().nncv_hip_plan_arena(n, first, last, size, align, off)
    if total == 2 ** 64 - 1:
        raise NncvHipError(lib().nncv_hip_last_error().decode())
    return int(total), [int(o) for o in off]


def mobilenetv3_small_ops():
    """-> ([GraphOp], n_elems): the library's built-in operator list of MobileNetV3-small."""
    n_elems = ctypes.c_int64()
    n = lib().nncv_hip_mobilenetv3_small_ops(None, 0, ctypes.byref(n_elems))
    arr = (GraphOp * n)()
    lib().nncv_hip_mobilenetv3_small_ops(arr, n, ctypes.byref(n_elems))
    return list(arr), int(n_elems.value)


def graph_create(ops, in_channels, params_blob):
    """nncv_hip_graph_create over a host blob (float32 / float16 numpy array); returns the handle."""
    dt = F16 if params_blob.dtype == np.float16 else F32
    arr = (GraphOp * len(ops))(*ops)
    blob = np.ascontiguousarray(params_blob)
    h = lib().nncv_hip_graph_create(arr, len(ops), in_channels, blob.ctypes.data, blob.size, dt)
    if not h:
        raise NncvHipError(lib().nncv_hip_last_error().decode())
    return h


def graph_plan(ops, in_channels, dt, N, H, W):
    """nncv_hip_graph_plan (host only) -> (total bytes, [(root, offset, root_bytes, c0)] per tensor, [dst] per operator)."""
    arr = (GraphOp * len(ops))(*ops)
    n_t = max(o.out for o in ops) + 1
    info = (ctypes.c_int64 * (4 * n_t))()
    dst = (ctypes.c_int32 * len(ops))()
    total = lib().nncv_hip_graph_plan(arr, len(ops), in_channels, dt, N, H, W, info, n_t, dst)
    if total < 0:
        raise NncvHipError(lib().nncv_hip_last_error().decode())
    return int(total), [tuple(int(v) for v in info[4 * t:4 * t + 4]) for t in range(n_t)], [int(d) for d in dst]


def graph_output_shape(h, H, W):
    shp = (ctypes.c_int * 3)()
    check(lib().nncv_hip_graph_output_shape(h, H, W, shp))
    return tuple(shp)
