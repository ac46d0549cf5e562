"""Helpers for the GPU parity tests: device memory through torch (plumbing only), calls through
the C ABI of libnncv_hip.so, comparison metrics with the tolerances of the acceptance criteria."""
import numpy as np
import torch

from nncv_amd import abi

# fp32: max |got - want| / max |want| (normwise max relative error) must stay below 1e-4
FP32_MAX_REL = 1e-4
# fp16: relative L2 error below 1e-2 (plus identical top-1 where logits are compared)
FP16_REL_L2 = 1e-2


def dev(a, dt=None):
    """numpy -> device tensor of the library dtype."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dt is not None:
        t = t.to(torch.float16 if dt == abi.F16 else torch.float32)
    return t.cuda()


def empty(shape, dt):
    return torch.empty(shape, dtype=torch.float16 if dt == abi.F16 else torch.float32, device="cuda")


def host(t):
    return t.detach().float().cpu().numpy()


def nhwc(a):
    """NCHW numpy -> contiguous NHWC numpy."""
    return np.ascontiguousarray(np.transpose(a, (0, 2, 3, 1)))


def nchw(a):
    return np.ascontiguousarray(np.transpose(a, (0, 3, 1, 2)))


def max_rel(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def max_rel_elementwise(got, want, floor=1e-2):
    """max over elements of |got - want| / max(|want|, floor * max|want|): the relative error of every element, with an
    absolute floor for elements near zero (an element one hundredth of the largest or smaller is held to the error a
    value of that size may have)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    denom = np.maximum(np.abs(want), floor * max(np.abs(want).max(), 1e-30))
    return float((np.abs(got - want) / denom).max())


def rel_l2(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def stream():
    return torch.cuda.current_stream().cuda_stream


class Conv:
    """nncv_hip_conv_* handle."""

    def __init__(self, dt, w, stride, pad, bn=None, relu=False, algo=abi.ALGO_AUTO):
        npdt = abi.np_dtype(dt)
        self.dt = dt
        w = np.ascontiguousarray(w, npdt)
        F, C, R, S = w.shape
        self.F, self.C, self.R, self.S, self.stride, self.pad = F, C, R, S, stride, pad
        ptrs = [None] * 4
        keep = []
        if bn is not None:
            keep = [np.ascontiguousarray(b, npdt) for b in bn]
            ptrs = [k.ctypes.data for k in keep]
        self.h = abi.lib().nncv_hip_conv_create(dt, w.ctypes.data, F, C, R, S, stride, pad, *ptrs, int(relu), algo)
        if not self.h:
            raise abi.NncvHipError(abi.lib().nncv_hip_last_error().decode())

    @property
    def algo(self):
        return abi.lib().nncv_hip_conv_algo(self.h)

    def __call__(self, x_dev, layout, residual=None):
        if layout == abi.NHWC:
            N, H, W, C = x_dev.shape
        else:
            N, C, H, W = x_dev.shape
        assert C == self.C
        OH = (H + 2 * self.pad - self.R) // self.stride + 1
        OW = (W + 2 * self.pad - self.S) // self.stride + 1
        shape = (N, OH, OW, self.F) if layout == abi.NHWC else (N, self.F, OH, OW)
        out = empty(shape, self.dt)
        torch.cuda.synchronize()
        abi.check(abi.lib().nncv_hip_conv_forward(self.h, x_dev.data_ptr(), N, H, W, layout,
                                                  residual.data_ptr() if residual is not None else None,
                                                  out.data_ptr(), None))
        return out

    def close(self):
        if self.h and abi is not None:
            abi.lib().nncv_hip_conv_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown: the modules this needs may be gone already
            pass


class Model:
    """nncv_hip_resnet18_* handle."""

    def __init__(self, blob, dt, algo=abi.ALGO_AUTO, passes=0):
        blob = np.ascontiguousarray(blob, abi.np_dtype(dt))
        self.dt = dt
        if passes:  # the handle plans for that many passes in flight (nncv_hip_resnet18_create_ex)
            self.h = abi.lib().nncv_hip_resnet18_create_ex(blob.ctypes.data, blob.size, dt, algo, passes)
        else:
            self.h = abi.lib().nncv_hip_resnet18_create(blob.ctypes.data, blob.size, dt, algo)
        if not self.h:
            raise abi.NncvHipError(abi.lib().nncv_hip_last_error().decode())

    def __call__(self, x_dev, tap_stage=None):
        N, C, H, W = x_dev.shape
        logits = torch.empty((N, 1000), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        if tap_stage is None:
            abi.check(abi.lib().nncv_hip_resnet18_forward(self.h, x_dev.data_ptr(), N, H, W, logits.data_ptr(), None))
            return logits
        ch = [64, 64, 128, 256, 512][tap_stage]
        down = lambda v: (v - 1) // 2 + 1  # every stride-2 stage halves, rounding up
        h, w = down(down(H)), down(down(W))
        for _ in range(max(0, tap_stage - 1)):
            h, w = down(h), down(w)
        tap = empty((N, h, w, ch), self.dt)
        abi.check(abi.lib().nncv_hip_resnet18_forward_tap(self.h, x_dev.data_ptr(), N, H, W, logits.data_ptr(),
                                                          tap_stage, tap.data_ptr(), None))
        return logits, tap

    def clone(self):
        """Another handle on the same device weights (nncv_hip_resnet18_clone), with a workspace of its own."""
        c = Model.__new__(Model)
        c.dt = self.dt
        c.h = abi.lib().nncv_hip_resnet18_clone(self.h)
        if not c.h:
            raise abi.NncvHipError(abi.lib().nncv_hip_last_error().decode())
        return c

    def close(self):
        if self.h and abi is not None:
            abi.lib().nncv_hip_resnet18_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown: the modules this needs may be gone already
            pass


class Graph:
    """nncv_hip_graph_* handle over an operator list and a host parameter blob."""

    def __init__(self, ops, in_channels, blob, dt):
        self.dt = dt
        self.h = abi.graph_create(ops, in_channels, np.ascontiguousarray(blob, abi.np_dtype(dt)))

    def __call__(self, x_dev):
        N, C, H, W = x_dev.shape
        c, oh, ow = abi.graph_output_shape(self.h, H, W)
        out = torch.empty((N, c, oh, ow), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        abi.check(abi.lib().nncv_hip_graph_forward(self.h, x_dev.data_ptr(), N, H, W, out.data_ptr(), out.numel(), None))
        return out

    def close(self):
        if self.h and abi is not None:
            abi.lib().nncv_hip_graph_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown: the modules this needs may be gone already
            pass
