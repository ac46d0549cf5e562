"""The callers the C ABI exists for, run on the GPU as child processes and from several threads.

 * examples/res18_main.cpp (this repository's driver with the flow of the reference's
   examples/Res18/main.cpp:18-23, :79-114, built by nncv_amd/build.py) reads a model.bin, calls
   _mlir_ciface_forward and prints the top-1 index per image: compared with the oracle.
 * oracle/_ref/res18_ref_driver is the reference's own examples/Res18/main.cpp, compiled unchanged
   (with its own DataType.cpp and the stb_image.h it vendors) and linked against libnncv_hip.so in
   place of the compiled model object.  It reads ./model.bin and ./cat_256x256.jpg (the photo of the
   reference's example, kept as tests/golden/cat_256x256.jpg) and prints its top-1 index, which must
   be the oracle's on the pixels the same decoder produces.  Skipped where that build is absent.
 * _mlir_ciface_forward from two threads at once: each result equals the one a serial call gives.
 * the device entry point on two streams: one handle (ordered by the library) and two handles (concurrent, each
   with its own workspace) -- both bit-equal to passes run alone.
"""
import os
import shutil
import subprocess
import threading

import numpy as np
import pytest
import torch  # before the library is loaded: one HIP runtime per process (see nncv_amd/abi.py)

import oracle
from nncv_amd import abi, build, modelbin, synth

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_DRIVER = os.path.join(ROOT, "oracle", "_ref", "res18_ref_driver")
STB_DECODE = os.path.join(ROOT, "oracle", "_ref", "stb_decode")
PHOTO = os.path.join(ROOT, "tests", "golden", "cat_256x256.jpg")


@pytest.fixture(scope="module")
def blob():
    return synth.resnet18_params()


def _run(cmd, cwd):
    print("running", cmd, "in", cwd, flush=True)
    r = subprocess.run(cmd, cwd=cwd, capture_output=True, text=True, timeout=110)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, (r.returncode, r.stderr)
    return r.stdout.split("\n")


def test_example_driver_prints_the_oracles_top1(blob, tmp_path):
    assert os.path.exists(build.DRIVER), "nncv_amd/lib/res18_main is missing: run python -m nncv_amd.build"
    modelbin.write_resnet18(str(tmp_path / "model.bin"), blob)
    B, H, W = 2, 96, 64
    x = synth.uniform(9100, (B, 3, H, W), 0.0, 1.0)
    x.tofile(str(tmp_path / "image.f32"))
    lines = _run([build.DRIVER, "model.bin", "image.f32", str(B), str(H), str(W)], str(tmp_path))
    got = [int(l) for l in lines if l.strip().isdigit()]
    # the driver normalises with the ImageNet mean / std, each step in fp32
    mean = np.array([0.485, 0.456, 0.406], np.float32).reshape(1, 3, 1, 1)
    std = np.array([0.229, 0.224, 0.225], np.float32).reshape(1, 3, 1, 1)
    want = oracle.resnet18_forward(((x - mean) / std).astype(np.float32), blob)
    assert got == [int(i) for i in want.argmax(1)], (got, want.argmax(1))


@pytest.mark.skipif(not (os.path.exists(REF_DRIVER) and os.path.exists(STB_DECODE)),
                    reason="oracle/_ref holds no build of the reference's driver")
def test_the_references_own_driver_runs_on_this_library(blob, tmp_path):
    modelbin.write_resnet18(str(tmp_path / "model.bin"), blob)
    shutil.copy(PHOTO, str(tmp_path / "cat_256x256.jpg"))
    lines = [l for l in _run([REF_DRIVER], str(tmp_path)) if l.strip()]
    assert lines[0].split() == ["256", "256", "3"]
    assert lines[1].startswith("Time: ")
    got = int(lines[2])
    raw = subprocess.run([STB_DECODE, PHOTO], capture_output=True, check=True).stdout
    head, _, pixels = raw.partition(b"\n")
    w, h, c = (int(v) for v in head.split())
    img = np.frombuffer(pixels, np.uint8).reshape(1, h, w, c)
    logits = oracle.resnet18_forward(oracle.preprocess_u8(img), blob)
    want = int(oracle.top1_scan(logits)[0])
    print("reference driver top-1", got, "oracle", want, flush=True)
    assert got == want


def test_forward_from_two_threads_at_once(blob):
    """The reference's object is re-entrant; here calls serialise on the library's mutex and share one
    arena and one weight cache.  Two threads, different inputs and shapes, several rounds: every result
    must be bit-equal to what the same call returns alone."""
    xs = [synth.uniform(9200, (1, 3, 64, 64), 0.0, 1.0), synth.uniform(9201, (3, 3, 96, 64), 0.0, 1.0)]
    serial = [abi.forward(x, blob) for x in xs]
    for x, got in zip(xs, serial):
        want = oracle.resnet18_forward(x, blob)
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-4
    results = [[], []]
    errors = []

    def work(k):
        try:
            for _ in range(6):
                results[k].append(abi.forward(xs[k], blob))
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
        assert not t.is_alive()
    assert not errors, errors
    for k in range(2):
        assert len(results[k]) == 6
        for r in results[k]:
            assert np.array_equal(r.view(np.uint32), serial[k].view(np.uint32))


def test_host_abi_on_a_large_batch_stages_its_upload(blob):
    """_mlir_ciface_forward_f16 on 16 host images (examples/Res18/main.cpp:95-99 with a batch): the input goes to pinned
    staging memory in pieces copied by several host threads, or straight from the caller's buffer when that is pinned.
    Either way the logits are the bits of the device entry point on the same batch, on every one of five calls; they meet
    the fp16 bar and the oracle's top-1 on every image; and a second thread calling with another batch at the same time
    changes nothing."""
    import torch
    from gpu_util import Model, dev, host, rel_l2, FP16_REL_L2
    hb = synth.round_fp16(blob)
    b16 = hb.astype(np.float16)
    x = synth.round_fp16(synth.uniform(9250, (16, 3, 224, 224), 0.0, 1.0))
    x16 = x.astype(np.float16)
    calls = [abi.forward(x16, b16).astype(np.float32) for _ in range(5)]
    for c in calls[1:]:
        assert np.array_equal(c, calls[0])
    m = Model(hb, abi.F16, abi.ALGO_AUTO)
    alone = host(m(dev(x, abi.F16))).astype(np.float16).astype(np.float32)
    assert np.array_equal(calls[0], alone)
    m.close()
    want = oracle.hwp_resnet18_forward(x, hb)
    assert rel_l2(calls[0], want) < FP16_REL_L2 and np.array_equal(calls[0].argmax(1), want.argmax(1))
    pinned = torch.from_numpy(x16).pin_memory()
    assert np.array_equal(abi.forward(pinned.numpy(), b16).astype(np.float32), calls[0])
    other = synth.round_fp16(synth.uniform(9251, (20, 3, 96, 96), 0.0, 1.0)).astype(np.float16)
    other_alone = abi.forward(other, b16)
    results, errors = [[], []], []

    def work(k, arr):
        try:
            for _ in range(4):
                results[k].append(abi.forward(arr, b16))
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(0, x16)), threading.Thread(target=work, args=(1, other))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
        assert not t.is_alive()
    assert not errors, errors
    for r in results[0]:
        assert np.array_equal(r.astype(np.float32), calls[0])
    for r in results[1]:
        assert np.array_equal(r, other_alone)


def test_device_calls_on_two_streams_do_not_overlap_in_the_shared_workspace(blob):
    """The device entry point on two caller streams alternately, without synchronising in between: the
    library orders the second stream behind the first (they share the activation arena), so both
    results equal the serial ones."""
    import torch
    from gpu_util import Model, dev, host
    m = Model(synth.round_fp16(blob), abi.F16, abi.ALGO_AUTO)
    L = abi.lib()
    xa = dev(synth.round_fp16(synth.uniform(9300, (8, 3, 224, 224), 0.0, 1.0)), abi.F16)
    xb = dev(synth.round_fp16(synth.uniform(9301, (8, 3, 224, 224), 0.0, 1.0)), abi.F16)
    want_a, want_b = host(m(xa)), host(m(xb))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    oa = torch.empty((8, 1000), dtype=torch.float32, device="cuda")
    ob = torch.empty((8, 1000), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    for _ in range(5):
        abi.check(L.nncv_hip_resnet18_forward(m.h, xa.data_ptr(), 8, 224, 224, oa.data_ptr(), s1.cuda_stream))
        abi.check(L.nncv_hip_resnet18_forward(m.h, xb.data_ptr(), 8, 224, 224, ob.data_ptr(), s2.cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(oa.cpu().numpy(), want_a)
    assert np.array_equal(ob.cpu().numpy(), want_b)
    m.close()


@pytest.mark.parametrize("dt", [abi.F16, abi.F32])
def test_two_handles_on_two_streams_run_concurrently_and_stay_exact(blob, dt):
    """Every network handle owns its workspace: passes of two handles enqueued alternately on two caller streams, with
    nothing ordering them, overlap on the GPU and must still each give the bits of a pass run alone -- fp16 at the
    measured batch and fp32 at batch 1, where the deep layers split K over workgroups (tickets and partial sums are
    per handle too)."""
    import torch
    from gpu_util import Model, dev, host
    b = synth.round_fp16(blob) if dt == abi.F16 else blob
    N = 16 if dt == abi.F16 else 1
    ma, mb = Model(b, dt, abi.ALGO_AUTO), Model(b, dt, abi.ALGO_AUTO)
    L = abi.lib()
    mk = (lambda seed: synth.round_fp16(synth.uniform(seed, (N, 3, 224, 224), 0.0, 1.0))) if dt == abi.F16 else \
         (lambda seed: synth.uniform(seed, (N, 3, 224, 224), 0.0, 1.0))
    xa, xb = dev(mk(9400), dt), dev(mk(9401), dt)
    want_a, want_b = host(ma(xa)), host(mb(xb))
    assert not np.array_equal(want_a, want_b)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    oa = torch.zeros((N, 1000), dtype=torch.float32, device="cuda")
    ob = torch.zeros((N, 1000), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    for it in range(8):
        abi.check(L.nncv_hip_resnet18_forward(ma.h, xa.data_ptr(), N, 224, 224, oa.data_ptr(), s1.cuda_stream))
        abi.check(L.nncv_hip_resnet18_forward(mb.h, xb.data_ptr(), N, 224, 224, ob.data_ptr(), s2.cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(oa.cpu().numpy(), want_a)
    assert np.array_equal(ob.cpu().numpy(), want_b)
    ma.close()
    mb.close()


def test_overlap_hint_changes_the_launch_shapes_not_the_results(blob):
    """nncv_hip_set_overlap_hint(4): the planners switch to the forms meant for several passes in flight (128-filter stream
    form on layer2 / layer3, layer1 on the form that keeps its weights in registers, average pool and FC as separate launches), the logits stay within
    the fp16 bar of the oracle with its top-1, four handles on four streams each reproduce the bits of a pass run alone,
    and hint 1 brings the usual shapes back."""
    import torch
    import oracle
    from gpu_util import Model, dev, host, rel_l2, FP16_REL_L2
    L = abi.lib()
    hb = synth.round_fp16(blob)
    N = 16
    xs = [synth.round_fp16(synth.uniform(9500 + i, (N, 3, 224, 224), 0.0, 1.0)) for i in range(4)]

    def tags(m, xd):
        m(xd)
        torch.cuda.synchronize()
        abi.profile_enable(True)
        try:
            abi.profile_report()
            got = host(m(xd))
            rep = abi.profile_report()
        finally:
            abi.profile_enable(False)
        return got, {k: v["launches"] for k, v in rep.items()}

    try:
        abi.check(L.nncv_hip_set_overlap_hint(4))
        ms = [Model(hb, abi.F16, abi.ALGO_AUTO)]
        ms += [ms[0].clone() for _ in range(3)]  # three more handles on the same device weights, each with its own workspace
        xd = [dev(x, abi.F16) for x in xs]
        alone, rep = tags(ms[0], xd[0])
        print("hint 4:", rep, flush=True)
        count = lambda r, prefix: sum(v for k, v in r.items() if k.startswith(prefix))
        assert rep.get("conv3x3_stream<f16,1x4x1>", 0) == 6            # layer2 and layer3
        assert rep.get("conv3x3_stream<f16,1x2x2,res>", 0) == 4        # layer1: one channel slab, weights resident in registers
        assert count(rep, "conv3x3_patch") == 3 and count(rep, "conv3x3_stream") == 10  # layer4 stays on the patch kernel
        assert count(rep, "conv3x3s2_patch") == 3 and count(rep, "igemm") == 1  # the FC of the split head
        assert "avgpool_fc" not in rep and rep.get("global_avgpool", 0) == 1
        want = oracle.resnet18_forward(xs[0][:4], hb)
        assert rel_l2(alone[:4], want) < FP16_REL_L2 and (alone[:4].argmax(1) == want.argmax(1)).all()
        # four passes in flight, repeatedly: every handle must reproduce the pass it gives alone
        wants = [alone] + [host(ms[i](xd[i])) for i in range(1, 4)]
        st = [torch.cuda.Stream() for _ in range(4)]
        outs = [torch.zeros((N, 1000), dtype=torch.float32, device="cuda") for _ in range(4)]
        torch.cuda.synchronize()
        for it in range(6):
            for i in range(4):
                abi.check(L.nncv_hip_resnet18_forward(ms[i].h, xd[i].data_ptr(), N, 224, 224, outs[i].data_ptr(), st[i].cuda_stream))
        torch.cuda.synchronize()
        for i in range(4):
            assert np.array_equal(outs[i].cpu().numpy(), wants[i]), i
        # back to one pass at a time: the usual shapes, and (different K order in layer2 / layer3) the same logits
        # to within rounding of the fp16 activations
        abi.check(L.nncv_hip_set_overlap_hint(1))
        again, rep1 = tags(ms[0], xd[0])
        print("hint 1:", rep1, flush=True)
        assert count(rep1, "conv3x3_stream") == 10 and rep1.get("avgpool_fc", 0) == 1
        assert rel_l2(again, alone) < 5e-3
        for m in ms:
            m.close()
    finally:
        abi.check(L.nncv_hip_set_overlap_hint(1))


def test_handles_with_different_passes_in_flight_work_side_by_side(blob):
    """nncv_hip_resnet18_create_ex: the number of passes in flight belongs to the handle.  One handle planned for four
    passes and one planned for one pass, alive together in one process, each launch the shapes of its own setting (also
    when their calls alternate and replay captured graphs), a clone inherits the value, the process-wide default stays
    what it was, and both agree with the oracle."""
    import torch
    import oracle
    from gpu_util import Model, dev, host, rel_l2, FP16_REL_L2
    L = abi.lib()
    hb = synth.round_fp16(blob)
    N = 16
    x = synth.round_fp16(synth.uniform(9800, (N, 3, 224, 224), 0.0, 1.0))
    xd = dev(x, abi.F16)
    wide = Model(hb, abi.F16, abi.ALGO_AUTO, passes=4)
    plain = Model(hb, abi.F16, abi.ALGO_AUTO, passes=1)
    twin = wide.clone()
    assert L.nncv_hip_resnet18_passes_in_flight(wide.h) == 4 and L.nncv_hip_resnet18_passes_in_flight(twin.h) == 4
    assert L.nncv_hip_resnet18_passes_in_flight(plain.h) == 1

    def tags(m):
        abi.profile_enable(True)
        try:
            abi.profile_report()
            got = host(m(xd))
            rep = abi.profile_report()
        finally:
            abi.profile_enable(False)
        return got, {k: v["launches"] for k, v in rep.items()}

    count = lambda r, prefix: sum(v for k, v in r.items() if k.startswith(prefix))
    for _ in range(2):  # alternating: neither handle's setting leaks into the other's plans
        got_w, rep_w = tags(wide)
        got_p, rep_p = tags(plain)
        assert rep_w.get("conv3x3_stream<f16,1x4x1>", 0) == 6 and "avgpool_fc" not in rep_w, rep_w
        assert count(rep_p, "conv3x3_stream") == 10 and rep_p.get("avgpool_fc", 0) == 1, rep_p
    got_t, rep_t = tags(twin)
    assert rep_t == rep_w and np.array_equal(got_t, got_w)
    want = oracle.hwp_resnet18_forward(x, hb)
    for got in (got_w, got_p):
        assert rel_l2(got, want) < FP16_REL_L2 and (got.argmax(1) == want.argmax(1)).all()
    # replayed graphs (third call on): each handle keeps reproducing its own bits while the calls alternate
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    ow = torch.zeros((N, 1000), dtype=torch.float32, device="cuda")
    op = torch.zeros((N, 1000), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    for _ in range(5):
        abi.check(L.nncv_hip_resnet18_forward(wide.h, xd.data_ptr(), N, 224, 224, ow.data_ptr(), s1.cuda_stream))
        abi.check(L.nncv_hip_resnet18_forward(plain.h, xd.data_ptr(), N, 224, 224, op.data_ptr(), s2.cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(ow.cpu().numpy(), got_w) and np.array_equal(op.cpu().numpy(), got_p)
    # destroying one handle leaves the other's captured passes alone
    wide.close()
    abi.check(L.nncv_hip_resnet18_forward(plain.h, xd.data_ptr(), N, 224, 224, op.data_ptr(), s2.cuda_stream))
    abi.check(L.nncv_hip_resnet18_forward(twin.h, xd.data_ptr(), N, 224, 224, ow.data_ptr(), s1.cuda_stream))
    torch.cuda.synchronize()
    assert np.array_equal(ow.cpu().numpy(), got_w) and np.array_equal(op.cpu().numpy(), got_p)
    plain.close()
    twin.close()


def test_pick_streams_returns_usable_streams(blob):
    """nncv_hip_pick_streams: four library-owned streams, at least one of them counted as overlapping, the same list on a
    second call, and passes enqueued on them give the bits of passes run alone."""
    import ctypes
    import torch
    from gpu_util import Model, dev, host
    L = abi.lib()
    st = (ctypes.c_void_p * 4)()
    found = ctypes.c_int(0)
    abi.check(L.nncv_hip_pick_streams(4, st, ctypes.byref(found)))
    print("overlapping streams:", found.value, flush=True)
    assert 1 <= found.value <= 4 and all(st[i] for i in range(4)) and len({st[i] for i in range(4)}) == 4
    st2 = (ctypes.c_void_p * 4)()
    abi.check(L.nncv_hip_pick_streams(4, st2, None))
    assert [st2[i] for i in range(4)] == [st[i] for i in range(4)]
    assert L.nncv_hip_pick_streams(9, st, None) != 0
    hb = synth.round_fp16(blob)
    ms = [Model(hb, abi.F16, abi.ALGO_AUTO, passes=4)]
    ms += [ms[0].clone() for _ in range(3)]
    xs = [dev(synth.round_fp16(synth.uniform(9900 + i, (4, 3, 64, 64), 0.0, 1.0)), abi.F16) for i in range(4)]
    wants = [host(ms[i](xs[i])) for i in range(4)]
    outs = [torch.zeros((4, 1000), dtype=torch.float32, device="cuda") for _ in range(4)]
    torch.cuda.synchronize()
    for _ in range(4):
        for i in range(4):
            abi.check(L.nncv_hip_resnet18_forward(ms[i].h, xs[i].data_ptr(), 4, 64, 64, outs[i].data_ptr(), st[i]))
    torch.cuda.synchronize()
    for i in range(4):
        assert np.array_equal(outs[i].cpu().numpy(), wants[i]), i
    for m in ms:
        m.close()


def test_clones_share_the_weights_and_outlive_the_first_handle(blob):
    """nncv_hip_resnet18_clone: the clone gives the bits of the model it was made from, keeps working after that model's
    handle is destroyed (the weights live until the last handle goes), and is refused for fp32 models, whose K-split
    tickets belong to the layers."""
    import pytest
    from gpu_util import Model, dev, host
    hb = synth.round_fp16(blob)
    x = dev(synth.round_fp16(synth.uniform(9700, (3, 3, 96, 128), 0.0, 1.0)), abi.F16)
    first = Model(hb, abi.F16, abi.ALGO_AUTO)
    want = host(first(x))
    twin = first.clone()
    assert np.array_equal(host(twin(x)), want)
    first.close()
    assert np.array_equal(host(twin(x)), want)
    again = twin.clone()
    twin.close()
    assert np.array_equal(host(again(x)), want)
    again.close()
    m32 = Model(blob, abi.F32, abi.ALGO_AUTO)
    with pytest.raises(abi.NncvHipError, match="fp16 models only"):
        m32.clone()
    m32.close()
