"""ResNet-18 forward on the GPU against the oracle: device API, taps, and the reference ABI."""
import os

import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, modelbin, synth
from gpu_util import Model, dev, host, nchw, max_rel, max_rel_elementwise, rel_l2, FP32_MAX_REL, FP16_REL_L2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def blob():
    return synth.resnet18_params()


@pytest.mark.parametrize("algo", [abi.ALGO_WINOGRAD, abi.ALGO_IGEMM])
def test_fp32_small_image_with_taps(blob, algo):
    x = synth.uniform(3001, (2, 3, 64, 64), 0.0, 1.0)
    m = Model(blob, abi.F32, algo)
    xd = dev(x)
    for stage in (0, 1, 2, 3, 4):
        want_logits, want_tap = oracle.resnet18_forward(x, blob, tap_layer=stage)
        logits, tap = m(xd, tap_stage=stage)
        err = max_rel(nchw(host(tap)), want_tap)
        print("algo", algo, "stage", stage, "tap max_rel", err, flush=True)
        assert err < FP32_MAX_REL
    err = max_rel(host(logits), want_logits)
    print("logits max_rel", err, flush=True)
    assert err < FP32_MAX_REL
    # every logit on its own, not only against the largest one (elements below 1 % of the largest against that floor)
    assert max_rel_elementwise(host(logits), want_logits) < FP32_MAX_REL
    assert (host(logits).argmax(1) == want_logits.argmax(1)).all()


def test_cfg3_fp32_256_through_reference_abi(blob, tmp_path):
    """BASELINE config 3: [1,3,256,256] fp32, params read back from a -split-params style
    model.bin, called through _mlir_ciface_forward like examples/Res18/main.cpp does."""
    p = str(tmp_path / "model.bin")
    modelbin.write_resnet18(p, blob)
    index, params = modelbin.read(p)
    assert len(index) == 102
    params = np.array(params)  # own, writable copy like MemRefFlatArray's blob
    x = synth.cfg3_input()
    got = abi.forward(x, params)
    want = oracle.resnet18_forward(x, blob)
    err = max_rel(got, want)
    print("cfg3 logits max_rel", err, "top1", got.argmax(1), want.argmax(1), flush=True)
    assert got.shape == (1, 1000)
    assert err < FP32_MAX_REL
    assert max_rel_elementwise(got, want) < FP32_MAX_REL  # element by element, with a floor of 1 % of the largest logit
    assert (got.argmax(1) == want.argmax(1)).all()
    # second call hits the cached device model; a strided input view must give the same answer
    xs = np.zeros((1, 3, 256, 512), np.float32)[:, :, :, ::2]
    xs[...] = x
    assert not xs.flags["C_CONTIGUOUS"]
    again = abi.forward(xs, params)
    assert np.array_equal(again, got)
    # same address, new contents: the cache must notice
    params[-1000:] += 1.0  # fc.bias
    shifted = abi.forward(x, params)
    assert np.allclose(shifted, got + 1.0, atol=1e-5)
    # a change between the fingerprint's samples goes unnoticed until the caller says so (nncv_hip_params_invalidate):
    # that is the documented contract of the cache
    n = params.size
    step = max(1, n // 4096)
    i = n - 1000 + 7  # fc.bias[7]
    assert i % step != 0 and i != n - 1, "pick an element the fingerprint does not sample"
    params[i] += 2.0
    stale = abi.forward(x, params)
    assert np.array_equal(stale, shifted)
    assert abi.lib().nncv_hip_params_invalidate(params.ctypes.data) == 0
    fresh = abi.forward(x, params)
    want2 = shifted.copy()
    want2[:, 7] += 2.0
    assert np.allclose(fresh, want2, atol=1e-5)


def test_fp16_small_batch(blob):
    """fp16 storage, fp32 accumulate vs the fp32 oracle on half-rounded weights and input."""
    hb = synth.round_fp16(blob)
    x = synth.round_fp16(synth.uniform(4001, (4, 3, 224, 224), 0.0, 1.0))
    want = oracle.resnet18_forward(x, hb)
    for algo in (abi.ALGO_IGEMM, abi.ALGO_WINOGRAD):
        m = Model(hb, abi.F16, algo)
        got = host(m(dev(x, abi.F16)))
        err = rel_l2(got, want)
        print("fp16 algo", algo, "rel_l2", err, "top1", got.argmax(1), want.argmax(1), flush=True)
        assert err < FP16_REL_L2
        assert (got.argmax(1) == want.argmax(1)).all()


def test_fp16_layers_take_the_kernels_they_are_measured_on(blob):
    """The launch tags of one fp16 forward pass at 224x224: every 3x3 stride-1 layer goes through one of the two LDS-patch
    kernels (the stream form for layers of at most 256 channels, the patch form for the deepest ones), the three stride-2
    ones through the patch kernel's stride-2 form with the 1x1 shortcut riding along (no separate shortcut launch), so a
    silent fall-back to the implicit-GEMM kernels shows up here and not only in the timings."""
    hb = synth.round_fp16(blob)
    m = Model(hb, abi.F16, abi.ALGO_IGEMM)

    def tags(xd):
        m(xd)
        torch.cuda.synchronize()
        abi.profile_enable(True)
        try:
            abi.profile_report()
            got = host(m(xd))
            rep = abi.profile_report()
        finally:
            abi.profile_enable(False)
        print({k: v["launches"] for k, v in rep.items()}, flush=True)
        return got, rep, (lambda prefix: sum(v["launches"] for k, v in rep.items() if k.startswith(prefix)))

    # batch 32, the measured configuration (input values do not matter for the route)
    _, rep, count = tags(dev(synth.round_fp16(synth.uniform(4004, (32, 3, 224, 224), 0.0, 1.0)), abi.F16))
    assert count("conv3x3_patch") + count("conv3x3_stream") == 13
    assert count("conv3x3_stream") == 10  # layer1 (4), layer2 (3) and layer3 (3)
    assert count("conv3x3s2_patch") == 3
    assert count("igemm") == 0
    assert sum(v["launches"] for v in rep.values()) == 18  # + stem/pool and pool/FC
    # batch 4 against the oracle: the small launches of layer2 / layer3 stay with the patch kernel
    x = synth.round_fp16(synth.uniform(4003, (4, 3, 224, 224), 0.0, 1.0))
    got, rep, count = tags(dev(x, abi.F16))
    assert count("conv3x3_patch") + count("conv3x3_stream") == 13
    assert count("conv3x3_stream") == 4  # layer1
    assert count("conv3x3s2_patch") == 3 and count("igemm") == 0
    assert sum(v["launches"] for v in rep.values()) == 18
    assert rel_l2(got, oracle.resnet18_forward(x, hb)) < FP16_REL_L2


def test_fp16_stage_outputs_at_a_batch_whose_shortcuts_ride_along(blob):
    """Batch 20 at 224x224: the stride-2 launches carry their block's 1x1 shortcut inside the workgroups of the 3x3
    convolution, behind its epilogue.  Every stage's
    output against the oracle, so that a wrong shortcut shows where it enters and not only in the logits."""
    hb = synth.round_fp16(blob)
    x = synth.round_fp16(synth.uniform(4007, (20, 3, 224, 224), 0.0, 1.0))
    m = Model(hb, abi.F16, abi.ALGO_IGEMM)
    xd = dev(x, abi.F16)
    for stage in (1, 2, 3, 4):
        want_logits, want_tap = oracle.resnet18_forward(x, hb, tap_layer=stage)
        logits, tap = m(xd, tap_stage=stage)
        got = nchw(host(tap))
        errs = [rel_l2(got[i], want_tap[i]) for i in range(20)]
        print("stage", stage, "worst image rel_l2 %.2e" % max(errs), flush=True)
        assert max(errs) < FP16_REL_L2
    assert rel_l2(host(logits), want_logits) < FP16_REL_L2
    m.close()


def test_graph_replay_matches_eager_every_time(blob):
    """The device entry point captures the forward into a HIP graph on the second call with the
    same buffers and replays it afterwards: every replay must equal the eager result, also when the
    input buffer's contents change between replays and other work runs in between."""
    hb = synth.round_fp16(blob)
    m = Model(hb, abi.F16)
    xs = [synth.round_fp16(synth.uniform(4100 + i, (2, 3, 64, 64), 0.0, 1.0)) for i in range(3)]
    xd = dev(xs[0], abi.F16)
    logits = torch.empty((2, 1000), dtype=torch.float32, device="cuda")
    L = abi.lib()

    def run():
        abi.check(L.nncv_hip_resnet18_forward(m.h, xd.data_ptr(), 2, 64, 64, logits.data_ptr(), None))
        return logits.cpu().numpy().copy()

    eager = run()  # first sighting: eager
    want = oracle.resnet18_forward(xs[0], hb)
    assert rel_l2(eager, want) < FP16_REL_L2
    for rep in range(6):  # capture on the first of these, replay on the rest
        x = xs[rep % 3]
        xd.copy_(torch.from_numpy(x.astype(np.float16)))
        other = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")  # unrelated eager work
        torch.cuda.synchronize()
        got = run()
        ref = host(Model(hb, abi.F16)(dev(x, abi.F16)))  # a fresh handle never replays: eager result
        assert np.array_equal(got, ref), rep
        assert other.shape == (256, 256)


def _stage0(m, x16, N, H, W):
    """Pooled stem activation (NHWC) and logits through the tap entry point, any image size."""
    oh, ow = (H - 1) // 2 + 1, (W - 1) // 2 + 1
    ph, pw = (oh - 1) // 2 + 1, (ow - 1) // 2 + 1
    xd = dev(x16, abi.F16)
    logits = torch.empty((N, 1000), dtype=torch.float32, device="cuda")
    tap = torch.empty((N, ph, pw, 64), dtype=torch.float16, device="cuda")
    abi.check(abi.lib().nncv_hip_resnet18_forward_tap(m.h, xd.data_ptr(), N, H, W, logits.data_ptr(), 0, tap.data_ptr(), None))
    return host(logits), nchw(host(tap))


@pytest.mark.parametrize("shape", [(2, 64, 64), (1, 96, 160), (1, 70, 90), (3, 224, 224), (1, 34, 32), (2, 226, 250)])
def test_fp16_fused_stem_and_pool(blob, shape):
    """conv7x7 + BN + ReLU + max-pool in one launch: pooled activation and logits vs the oracle for
    square, wide, odd-sized and minimum images (partial tiles on every edge)."""
    N, H, W = shape
    hb = synth.round_fp16(blob)
    x = synth.round_fp16(synth.uniform(4200 + H, (N, 3, H, W), -1.0, 1.0))
    want_logits, want_tap = oracle.resnet18_forward(x, hb, tap_layer=0)
    m = Model(hb, abi.F16)
    logits, tap = _stage0(m, x, N, H, W)
    assert tap.shape == want_tap.shape
    e_tap, e_log = rel_l2(tap, want_tap), rel_l2(logits, want_logits)
    print("shape", shape, "stage0 rel_l2", e_tap, "logits rel_l2", e_log, flush=True)
    assert e_tap < 2e-3  # one fp16 rounding of an O(1) activation
    assert e_log < FP16_REL_L2


@pytest.mark.parametrize("dt", [abi.F16, abi.F32])
def test_head_on_a_final_image_of_many_pixels(blob, dt):
    """416x480 in: the last stage is 13x15 = 195 pixels, so the head's pooling walks several trips of sixteen pixels per
    wave with a ragged last one (at 224x224 it is 49 pixels, one trip)."""
    b = synth.round_fp16(blob) if dt == abi.F16 else blob
    x = synth.uniform(4400, (1, 3, 416, 480), 0.0, 1.0)
    if dt == abi.F16:
        x = synth.round_fp16(x)
    want = oracle.resnet18_forward(x, b)
    m = Model(b, dt)
    got = host(m(dev(x, dt)))
    err = rel_l2(got, want)
    print("head on 13x15, dtype", dt, "logits rel_l2 %.2e" % err, flush=True)
    assert err < (FP16_REL_L2 if dt == abi.F16 else 1e-4)
    assert got.argmax(1) == want.argmax(1)
    m.close()


def test_fp16_fused_stem_propagates_nan(blob):
    """arith.maximumf keeps NaN: a NaN pixel poisons exactly the pooled outputs whose windows see it."""
    hb = synth.round_fp16(blob)
    x = synth.round_fp16(synth.uniform(4300, (1, 3, 64, 64), -1.0, 1.0))
    x[0, 1, 20, 41] = np.nan
    want_logits, want_tap = oracle.resnet18_forward(x, hb, tap_layer=0)
    m = Model(hb, abi.F16)
    _, tap = _stage0(m, x, 1, 64, 64)
    assert np.isnan(want_tap).any() and not np.isnan(want_tap).all()
    assert np.array_equal(np.isnan(tap), np.isnan(want_tap))
    ok = ~np.isnan(want_tap)
    assert rel_l2(tap[ok], want_tap[ok]) < 2e-3


def test_fp16_fused_stem_nan_and_inf_at_tile_borders(blob):
    """NaNs and infinities where the fused kernel's tiles meet (a pooled tile is 7 rows x 8 columns: image rows 28 k,
    columns 32 k), in the image corners and in the last, partial tile: the same outputs are poisoned as in the oracle,
    +inf stays +inf, and every other value is untouched.  The pixels sit in odd columns: the kernel's K axis pads a
    filter row from seven to eight pixels with a zero weight on the even column left of the window, so a non-finite
    pixel in an even column also reaches the window one further right as 0 x inf = NaN (a documented difference from
    the reference, which images with finite pixels never see)."""
    hb = synth.round_fp16(blob)
    H, W = 120, 136
    x = synth.round_fp16(synth.uniform(4310, (2, 3, H, W), -1.0, 1.0))
    for (n, c, y, xx) in [(0, 0, 0, 1), (0, 2, 27, 31), (0, 1, 28, 33), (1, 0, 55, 63), (1, 2, H - 1, W - 1), (1, 1, 112, 5)]:
        x[n, c, y, xx] = np.nan
    x[0, 1, 60, 101] = np.inf
    x[1, 0, 3, 131] = -np.inf
    _, want_tap = oracle.resnet18_forward(x, hb, tap_layer=0)
    m = Model(hb, abi.F16)
    _, tap = _stage0(m, x, 2, H, W)
    assert np.isnan(want_tap).any() and not np.isnan(want_tap).all()
    assert np.array_equal(np.isnan(tap), np.isnan(want_tap))
    assert np.array_equal(np.isposinf(tap), np.isposinf(want_tap))
    ok = np.isfinite(want_tap)
    assert rel_l2(tap[ok], want_tap[ok]) < 2e-3


@pytest.mark.parametrize("shape", [(1, 3, 32, 32), (3, 3, 33, 47), (2, 3, 225, 223), (1, 3, 330, 70), (33, 3, 64, 64)])
def test_unusual_sizes_both_types(blob, shape):
    """Smallest image the network accepts, odd and very oblong images, a batch that is not a power of two:
    the tile planners, the fused stem (even widths only) and its fallback all see shapes they were not tuned for."""
    x = synth.uniform(3011, shape, 0.0, 1.0)
    print("sizes", shape, flush=True)
    m32 = Model(blob, abi.F32)
    got, want = host(m32(dev(x))), oracle.resnet18_forward(x, blob)
    assert max_rel(got, want) < FP32_MAX_REL and (got.argmax(1) == want.argmax(1)).all()
    m32.close()
    b16, x16 = synth.round_fp16(blob), synth.round_fp16(x)
    m16 = Model(b16, abi.F16)
    got16, want16 = host(m16(dev(x16, abi.F16))), oracle.resnet18_forward(x16, b16)
    assert rel_l2(got16, want16) < FP16_REL_L2 and (got16.argmax(1) == want16.argmax(1)).all()
    m16.close()
