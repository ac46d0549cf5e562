"""Device pre-/post-processing of the reference driver (examples/Res18/main.cpp:38-77, :103-111)."""
import numpy as np
import pytest
import torch

import oracle
from nncv_amd import abi, synth
from gpu_util import Model, host, rel_l2, FP16_REL_L2

pytestmark = pytest.mark.gpu


def _image(seed, shape):
    return np.random.default_rng(seed).integers(0, 256, size=shape, dtype=np.uint8)


@pytest.mark.parametrize("shape", [(1, 32, 32, 3), (2, 37, 53, 3), (3, 64, 48, 4)])
def test_preprocess_u8_bit_exact(shape):
    img = _image(11, shape)
    img[0, 0, 0, :3] = (0, 255, 128)
    want = oracle.preprocess_u8(img)
    N, H, W, ch = shape
    d_img = torch.from_numpy(img).cuda()
    for dt, tdt in ((abi.F32, torch.float32), (abi.F16, torch.float16)):
        out = torch.empty((N, 3, H, W), dtype=tdt, device="cuda")
        abi.check(abi.lib().nncv_hip_preprocess_u8(d_img.data_ptr(), N, H, W, ch, dt, out.data_ptr(), None))
        got = out.cpu().numpy()
        if dt == abi.F32:
            assert np.array_equal(got, want)  # same fp32 operations in the same order
        else:
            assert np.array_equal(got, want.astype(np.float16))  # one rounding of the fp32 value


def test_argmax_matches_the_drivers_scan():
    rng = np.random.default_rng(3)
    x = rng.normal(size=(9, 1000)).astype(np.float32)
    x[1, 17] = x[1, 400] = x[1].max() + 1.0           # tie: the first index wins
    x[2, :] = -150.0                                    # nothing above -100: index 0
    x[3, 5] = np.nan; x[3, 900] = 7.0                   # NaN never wins
    x[4, 999] = 50.0                                    # last element
    x[5, 0] = 50.0                                      # first element
    x[6, :] = -100.0                                    # equal to the initial maximum: index 0
    x[7, 300:310] = 3.5                                 # a run of equal maxima across lanes
    x[8, 256] = x[8, 0] = 9.0                           # tie between a thread's first and second element
    d = torch.from_numpy(x).cuda()
    idx = torch.empty((9,), dtype=torch.int32, device="cuda")
    abi.check(abi.lib().nncv_hip_argmax(d.data_ptr(), 9, 1000, idx.data_ptr(), None))
    assert np.array_equal(idx.cpu().numpy(), oracle.top1_scan(x))
    # other row lengths, including shorter than a workgroup
    for F in (1, 7, 255, 257, 4099):
        y = rng.normal(size=(3, F)).astype(np.float32)
        dy = torch.from_numpy(y).cuda()
        out = torch.empty((3,), dtype=torch.int32, device="cuda")
        abi.check(abi.lib().nncv_hip_argmax(dy.data_ptr(), 3, F, out.data_ptr(), None))
        assert np.array_equal(out.cpu().numpy(), oracle.top1_scan(y)), F


def test_classify_u8_end_to_end():
    """u8 image -> top-1 in one call: equals oracle(preprocess) -> oracle network -> scan."""
    hb = synth.round_fp16(synth.resnet18_params())
    img = _image(21, (2, 64, 64, 3))
    x = synth.round_fp16(oracle.preprocess_u8(img))
    want = oracle.resnet18_forward(x, hb)
    m = Model(hb, abi.F16)
    d_img = torch.from_numpy(img).cuda()
    logits = torch.empty((2, 1000), dtype=torch.float32, device="cuda")
    top1 = torch.empty((2,), dtype=torch.int32, device="cuda")
    abi.check(abi.lib().nncv_hip_resnet18_classify_u8(m.h, d_img.data_ptr(), 2, 64, 64, 3, logits.data_ptr(), top1.data_ptr(), None))
    got = host(logits)
    assert rel_l2(got, want) < FP16_REL_L2
    assert np.array_equal(top1.cpu().numpy(), oracle.top1_scan(want))
    assert np.array_equal(top1.cpu().numpy(), oracle.top1_scan(got))
