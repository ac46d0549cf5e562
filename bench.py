#!/usr/bin/env python3
"""ResNet-18 inference benchmark of libnncv_hip.so on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 32] [--algo auto|winograd|igemm]

One step = one forward pass of BASELINE config 4 (ResNet-18, fp16 storage / fp32 accumulate,
input [32,3,224,224], seeded synthetic input and random-init weights) with the input already
resident in HBM and the logits left in HBM.  Prints ONE JSON line.

Besides the headline images/s the line carries
  roofline      the dominant kernel (the MFMA kernel instance that takes the most time): algorithmic
                flops per launch / average launch duration, measured live with HIP events on the
                launch stream (the layer of that instance alone, 200 launches back to back), against
                the published dense fp16 MFMA peak;
  kernels       an event-timed breakdown for every kernel tag (ms per step, share);
  batch1        images/s of the same network at batch 1;
  config.passes_in_flight, one_pass_at_a_time
                `value` keeps several forward passes in flight, each on its own model handle and stream (the
                count is the best of 2, 3 and 4 in a short trial, the streams are chosen by measuring which of
                them overlap); the same loop on one handle and one stream is reported next to it;
  host_abi      images/s through the reference's own entry point, _mlir_ciface_forward_f16, with host
                buffers in and out (what examples/Res18/main.cpp:95-99 times): PCIe transfers included;
  configs       BASELINE configs 1-3: the 1024^3 fp32 matmul, the single fp32 3x3 convolution (direct and
                Winograd), the fp32 network on one 256x256 image;
  bandwidth     the bandwidth-bound kernels against the HBM peak: Winograd input / output transforms,
                the stand-alone 3x3 stride-2 max-pool;
  conv3x3_sweep BASELINE config 5: each 3x3 layer shape of the network alone at batch 64, TFLOP/s and
                the fraction of the fp16 matrix peak;
  cpu_baseline  CPU restatements of the convolution schedule (oracle/hostwparallel.cpp, fp32, AVX2) timed
                on this box's host cores on a bounded sample of the same workload: this repository's own
                OpenMP routine on all cores and on 4 threads, and the reference's sequential tile order
                -- reported baselines, not targets.

The GPU's clocks take some 20 ms of continuous work to ramp up from idle; every timed loop below
therefore follows an untimed run of the same work that is at least that long.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
# Hardware queues of this process (the HIP runtime's own setting, read when it initialises; default 4).  Streams that
# share a queue run their work one after the other; where the environment does not fix the number, eight queues make that
# rarer.  Which streams actually overlap is measured by the library (nncv_hip_pick_streams), whatever the number is.
os.environ.setdefault("GPU_MAX_HW_QUEUES", "8")
IN_FLIGHT_CANDIDATES = (2, 3, 4)


def library_streams(L, want):
    """`want` HIP streams from the library (nncv_hip_pick_streams), and what its probe found.

    Two streams overlap only when the runtime gave them different hardware queues AND those queues sit on different
    pipes of the command processor (four pipes; queue q of a process is served by pipe q mod 4): work on two streams
    that share a queue runs one after the other, on two queues of one pipe it gains 14 %.  Which queue a stream gets
    depends on every stream the process created before it, so the library chooses its streams by measurement (chains
    of short kernels on eight candidates, pairwise) and hands out the ones that overlap first."""
    import ctypes
    st = (ctypes.c_void_p * want)()
    found = ctypes.c_int(0)
    if L.nncv_hip_pick_streams(want, st, ctypes.byref(found)) != 0:
        raise RuntimeError(L.nncv_hip_last_error().decode())
    return [st[i] for i in range(want)], {"candidates": 8, "overlapping": int(found.value), "by": "nncv_hip_pick_streams"}


MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 matrix peak
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X fp32 matrix peak
HBM_PEAK_GBS = 8000.0
CLOCK_WARMUP_MS = 60.0          # untimed work ahead of a timed loop (see the module docstring)
# kernel tag -> (C, F, H=W) of the ResNet-18 layer at batch 32 that the tag's instance runs most
DOMINANT_LAYER = {
    "conv3x3_stream<f16,1x2x2>": (128, 128, 28),
    "conv3x3_stream<f16,1x4x1>": (128, 128, 28),
    "conv3x3_stream<f16,1x1x4>": (256, 256, 14),
    "conv3x3_patch<f16,4,1>": (64, 64, 56),
    "conv3x3_patch<f16,2,2>": (128, 128, 28),
    "conv3x3_patch<f16,1,4>": (512, 512, 7),
}
# HBM bytes per launch of those layers from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script, scaled by the same counters' reading for a device copy of known size (factor 2.0 for
# FETCH_SIZE, 1.0 for WRITE_SIZE on this part).
DOMINANT_TRAFFIC = {  # profiles/resnet18_fp16_bs32_hbm_counters.txt, launches without a residual input
    "conv3x3_stream<f16,1x2x2>": (8772 + 6272) * 1024,
    "conv3x3_patch<f16,2,2>": (8746 + 6272) * 1024,
    "conv3x3_patch<f16,4,1>": (13341 + 12544) * 1024,
    "conv3x3_patch<f16,1,4>": (17301 + 1568) * 1024,
}


# the same for the launch plan of three or more passes in flight
IN_FLIGHT_TRAFFIC = {  # profiles/resnet18_fp16_bs32_in_flight_plan_hbm_counters.txt, the layer alone, no residual input
    "conv3x3_stream<f16,1x4x1>": (8835 + 6272) * 1024,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults long enough for the clocks to settle: 50 steps after 10 (15 ms of work) read 7 % low
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--batch", type=int, default=0, help="0 = the workload's default (32; yolov5s 16)")
    ap.add_argument("--algo", default="auto", choices=["auto", "winograd", "igemm"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-batch1", action="store_true", help="skip the batch-1 measurement and the per-layer sweep (for per-kernel profiles)")
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-layer 3x3 sweep at batch 64 (BASELINE config 5)")
    ap.add_argument("--profile-steps", type=int, default=5)
    ap.add_argument("--in-flight", type=int, default=0,
                    help="forward passes kept in flight: step k runs on model handle and HIP stream k mod this number "
                         "(each handle owns its workspace); 1 = one pass after the other; 0 = the best of 2, 3 and 4 in a "
                         "short trial (how many passes overlap depends on the hardware queues the runtime was given)")
    ap.add_argument("--no-overlap-hint", action="store_true",
                    help="do not tell the library how many passes are in flight (nncv_hip_set_overlap_hint): it then plans "
                         "every launch as if it had the chip to itself")
    ap.add_argument("--in-flight-batch1", type=int, default=0,
                    help="the same for the batch-1 measurement (a batch-1 pass is a chain of 18 short launches that leaves "
                         "most of the chip idle)")
    ap.add_argument("--workload", default="resnet18", choices=["resnet18", "mobilenetv3", "yolov5s"],
                    help="resnet18 = the headline configuration; mobilenetv3 / yolov5s = the networks of tests/Nets/MobileNetV3.mlir "
                         "and Yolov5s.mlir through the operator-list executor (same step definition, their own JSON line; "
                         "default batch 32 at 224x224 and 16 at 640x640)")
    ap.add_argument("--image", type=int, default=0, help="image side for the graph workloads (0 = 224 / 640)")
    ap.add_argument("--configs-only", action="store_true",
                    help="run only the `configs` and `bandwidth` legs (BASELINE configs 1-3, Winograd transforms, max-pool) and "
                         "print them: the command behind the fp32 kernel traces in profiles/")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a known-size kernel to scale HBM counters by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py: this build measures ONE GPU only (inference shards over the batch with no "
                         "communication between GPUs, so a second GPU adds nothing to measure). Run with --gpus 1.\n")
        sys.exit(2)

    import numpy as np
    import torch
    from nncv_amd import abi, resnet18_spec as spec, synth

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(1)
    L = abi.lib()  # raises if the HIP library is missing: there is no fallback path
    if args.batch <= 0:
        args.batch = 16 if args.workload == "yolov5s" else 32
    if args.workload != "resnet18":
        return bench_graph(args, L)
    if args.configs_only:
        torch.zeros(1, device="cuda")
        stream0 = torch.cuda.current_stream().cuda_stream
        print(json.dumps({"configs": baseline_configs(L, stream0, synth.resnet18_params()), "bandwidth": bandwidth_kernels(L, stream0),
                          "device": L.nncv_hip_device_arch().decode()}))
        return
    algo = {"auto": abi.ALGO_AUTO, "winograd": abi.ALGO_WINOGRAD, "igemm": abi.ALGO_IGEMM}[args.algo]

    N, H = args.batch, 224
    blob32 = synth.resnet18_params()
    blob = blob32.astype(np.float16)
    x = synth.cfg4_input(N).astype(np.float16)
    torch.zeros(1, device="cuda")  # HIP context up before the clock starts
    torch.cuda.synchronize()
    t_create = time.perf_counter()
    model = L.nncv_hip_resnet18_create(blob.ctypes.data, blob.size, abi.F16, algo)
    if not model:
        raise RuntimeError(L.nncv_hip_last_error().decode())
    # one-time cost of a model: upload of the 23 MB blob, BN fold, filter re-lay (synchronous)
    t_create = time.perf_counter() - t_create
    xd = torch.from_numpy(x).cuda()
    logits = torch.empty((N, 1000), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    # Passes in flight: handle i and stream i serve steps i, i + K, i + 2K ...  A handle owns its workspace, so passes of
    # different handles overlap on the GPU (one pass's launch gaps, prologues and tails fill with the other's work); every
    # pass is still a whole forward over one batch of N images, into its own logits buffer.
    # The number of passes in flight is a property of the handles (nncv_hip_resnet18_create_ex; clones inherit it): the
    # library plans their launches for it.  One set of handles per value tried, each set one model and its clones.
    asked1 = 1 if args.no_batch1 else args.in_flight_batch1
    KMAX = max(args.in_flight, asked1, max(IN_FLIGHT_CANDIDATES) if 0 in (args.in_flight, asked1) else 1)
    outs = [logits] + [torch.empty((N, 1000), dtype=torch.float32, device="cuda") for _ in range(1, KMAX)]
    handle_sets = {1: [model]}
    all_handles = [model]

    def handles_for(k_in_flight):
        passes = 1 if args.no_overlap_hint else k_in_flight
        hs = handle_sets.get(passes)
        if hs is None:
            first = L.nncv_hip_resnet18_create_ex(blob.ctypes.data, blob.size, abi.F16, algo, passes)
            if not first:
                raise RuntimeError(L.nncv_hip_last_error().decode())
            hs = handle_sets[passes] = [first]
            all_handles.append(first)
        while len(hs) < k_in_flight:
            h = L.nncv_hip_resnet18_clone(hs[0])  # its own workspace on the same device weights
            if not h:
                raise RuntimeError(L.nncv_hip_last_error().decode())
            hs.append(h)
            all_handles.append(h)
        return hs

    # every handle reads its own copy of the input (passes in flight must not share one cached tensor)
    xds = [xd] + [xd.clone() for _ in range(1, KMAX)]
    x1s = [t[:1].contiguous() for t in xds]
    x1 = x1s[0]
    l1 = [torch.empty((1, 1000), dtype=torch.float32, device="cuda") for _ in range(KMAX)]
    pool_streams, stream_probe = [], None
    if KMAX > 1:
        pool_streams, stream_probe = library_streams(L, KMAX)

    def step(xt, out, n):
        abi.check(L.nncv_hip_resnet18_forward(model, xt.data_ptr(), n, H, H, out.data_ptr(), stream))

    def timed(xts, out_list, n, warmup, steps, k_in_flight):
        hs = handles_for(k_in_flight)

        def go(i):
            j = i % k_in_flight
            # with several passes in flight every handle gets a stream of its own, measured to overlap with the others
            # (nncv_hip_pick_streams); one pass at a time stays on the default stream, like every other measurement here
            sj = stream if k_in_flight == 1 else pool_streams[j]
            abi.check(L.nncv_hip_resnet18_forward(hs[j], xts[j].data_ptr(), n, H, H, out_list[j].data_ptr(), sj))
        # clock warm-up: untimed steps until CLOCK_WARMUP_MS of wall time have passed, then the W asked for
        t_w = time.perf_counter()
        while (time.perf_counter() - t_w) * 1e3 < CLOCK_WARMUP_MS:
            for i in range(20):
                go(i)
            torch.cuda.synchronize()
        for i in range(warmup):
            go(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            go(i)
        torch.cuda.synchronize()  # every stream
        dt = time.perf_counter() - t0
        return dt / steps

    def pick_in_flight(asked, xts, out_list, n):
        """(passes in flight, {candidate: ms per pass in the trial})"""
        if asked > 0:
            return asked, None
        trial = {k: timed(xts, out_list, n, 20, max(30, args.steps // 2), k) for k in IN_FLIGHT_CANDIDATES}
        return min(trial, key=trial.get), {str(k): round(v * 1e3, 4) for k, v in trial.items()}

    K, k_trial = pick_in_flight(args.in_flight, xds, outs, N)
    sec = timed(xds, outs, N, args.warmup, args.steps, K)
    sec_serial = sec if K == 1 else timed(xds, outs, N, args.warmup, args.steps, 1)
    ips = N / sec
    flops_step = spec.flops_per_image(H) * N

    # batch 1 (the other half of the headline metric)
    K1, k1_trial = (1, None) if args.no_batch1 else pick_in_flight(args.in_flight_batch1, x1s, l1, 1)
    sec1 = None if args.no_batch1 else timed(x1s, l1, 1, args.warmup, max(args.steps, 50), K1)
    sec1_serial = None if args.no_batch1 else (sec1 if K1 == 1 else timed(x1s, l1, 1, args.warmup, max(args.steps, 50), 1))

    # event-timed per-kernel pass (separate from the timed region above: the events serialise launches)
    abi.profile_enable(True)
    abi.profile_report()
    for _ in range(args.profile_steps):
        step(xd, logits, N)
    torch.cuda.synchronize()
    prof = abi.profile_report()
    abi.profile_enable(False)
    total_ms = sum(v["ms"] for v in prof.values()) or 1.0
    kernels = {}
    for tag, v in sorted(prof.items(), key=lambda kv: -kv[1]["ms"]):
        per_launch_ms = v["ms"] / v["launches"]
        kernels[tag] = {
            "launches_per_step": v["launches"] / args.profile_steps,
            "ms_per_step": round(v["ms"] / args.profile_steps, 5),
            "share": round(v["ms"] / total_ms, 4),
            "avg_launch_us": round(per_launch_ms * 1e3, 3),
            "tflops": round(v["flops"] / (v["ms"] * 1e-3) / 1e12, 3) if v["flops"] else None,
            "gbs": round(v["bytes"] / (v["ms"] * 1e-3) / 1e9, 2),
        }
    # dominant kernel: the MFMA kernel instance (direct 3x3 or implicit GEMM) with the most time
    dom = max((t for t in prof if prof[t]["flops"] > 0), key=lambda t: prof[t]["ms"])
    d = prof[dom]
    flops_per_launch = d["flops"] / d["launches"]
    roofline = {"kernel": dom, "bound": "mfma", "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "flops_per_launch": flops_per_launch, "launches_per_step": d["launches"] / args.profile_steps,
                "traffic": DOMINANT_TRAFFIC.get(dom)}
    # Its launch duration: an event pair around ONE launch carries ~4 us of event/dispatch
    # latency on top of the kernel (the per-tag table above is good for shares, not for a
    # roofline).  So the dominant instance is re-run alone: the layer of that instance with the
    # network's own shape, BN + ReLU epilogue, `reps` launches back to back on the launch stream
    # between one pair of events.  The quotient still contains the ~1 us gap between consecutive
    # dispatches, i.e. it errs on the slow side of the profiler's pure kernel time.
    shape = DOMINANT_LAYER.get(dom)
    if shape is not None and N == 32:
        C, F, HW = shape
        w = synth.normal(77, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9)))).astype(np.float16)
        bn = [synth.uniform(78 + i, (F,), 0.5, 1.5).astype(np.float16) for i in range(4)]
        conv = L.nncv_hip_conv_create(abi.F16, w.ctypes.data, F, C, 3, 3, 1, 1, *[b.ctypes.data for b in bn], 1, abi.ALGO_IGEMM)
        if not conv:
            raise RuntimeError(L.nncv_hip_last_error().decode())
        xin = torch.randn((N, HW, HW, C), device="cuda", dtype=torch.float16)
        yout = torch.empty((N, HW, HW, F), device="cuda", dtype=torch.float16)
        reps = 200
        import ctypes
        avg = ctypes.c_float(0.0)
        abi.check(L.nncv_hip_conv_time(conv, xin.data_ptr(), N, HW, HW, None, yout.data_ptr(), 4000, stream, ctypes.byref(avg)))  # clocks
        abi.check(L.nncv_hip_conv_time(conv, xin.data_ptr(), N, HW, HW, None, yout.data_ptr(), reps, stream, ctypes.byref(avg)))
        us = float(avg.value)
        L.nncv_hip_conv_destroy(conv)
        layer_flops = 2.0 * N * HW * HW * F * C * 9
        achieved = layer_flops / (us * 1e-6) / 1e12
        roofline.update({"achieved": round(achieved, 3), "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 5),
                         "avg_launch_us": round(us, 3), "launches": reps, "flops_per_launch": layer_flops,
                         "timing": "layer [%d,%d,%d,%d]->%d alone, %d back-to-back launches between one HIP event pair"
                                   % (N, HW, HW, C, F, reps)})
    else:
        achieved = d["flops"] / (d["ms"] * 1e-3) / 1e12
        roofline.update({"achieved": round(achieved, 3), "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 5),
                         "avg_launch_us": round(d["ms"] / d["launches"] * 1e3, 3), "launches": d["launches"],
                         "timing": "one HIP event pair per launch (includes ~4 us of event latency)"})
    # The same leg for what `value` runs: with three or more passes in flight the handles launch the 128-filter form of the
    # stream kernel on layer2 / layer3 (six launches per pass: the instance with the most time in that mode).  Its layer
    # alone, planned for K passes in flight (single layers plan with the process-wide default), back to back as above.
    roofline_in_flight = None
    if K >= 3 and not args.no_overlap_hint and N == 32:
        roofline_in_flight = layer_roofline(L, stream, N, 128, 128, 28, K)
        roofline_in_flight["traffic"] = IN_FLIGHT_TRAFFIC.get(roofline_in_flight["kernel"])
        roofline_in_flight["launches_per_step"] = 6
        roofline_in_flight["note"] = ("the dominant kernel instance of the launch plan `value` runs (passes_in_flight >= 3), timed "
                                      "alone; in the timed region its launches share the chip with those of the other passes "
                                      "and have no duration of their own")
    roofline["launch_shapes"] = ("those of one pass at a time (overlap hint 1), which the summaries under profiles/ hold; with "
                                 "three or more passes in flight layer2 / layer3 run the same kernel's 128-filter form and "
                                 "layer1 its resident-weight form on half the places (see config.passes_in_flight), where a launch of one pass has no "
                                 "duration of its own")
    conv3x3_flops = 13 * 2 * 56 * 56 * 64 * 64 * 9 * N  # the 13 stride-1 3x3 layers all cost the same per image
    out = {
        "metric": "resnet18_fp16_bs%d_images_per_s" % N, "value": round(ips, 2), "unit": "images/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 4: ResNet-18 forward, fp16, input [%d,3,224,224], seeded U[0,1] input, "
                               "random-init Kaiming/BN-folded weights from a model.bin-order blob" % N,
                   "batch": N, "image": H, "algo3x3": args.algo, "input_resident_in_hbm": True,
                   "passes_in_flight": K, "passes_in_flight_trial_ms": k_trial, "stream_probe": stream_probe,
                   "passes_in_flight_note": "step k runs on model handle and HIP stream k mod %d, each handle with its own "
                                            "workspace, input copy and logits buffer; every step is one whole forward pass over "
                                            "one batch of %d images; ms_per_step is elapsed time / steps, i.e. the reciprocal "
                                            "of the pass rate, not the latency of a pass; `one_pass_at_a_time` is the same loop "
                                            "on one handle and one stream, where the two coincide" % (K, N)},
        "tflops_effective": round(flops_step / sec / 1e12, 3),
        "frac_of_fp16_mfma_peak": round(flops_step / sec / 1e12 / MFMA_F16_PEAK_TFLOPS, 5),
        "conv3x3s1_gflop_per_step": round(conv3x3_flops / 1e9, 2),
        "one_pass_at_a_time": {"images_per_s": round(N / sec_serial, 2), "ms_per_step": round(sec_serial * 1e3, 4),
                               "tflops_effective": round(flops_step / sec_serial / 1e12, 3)},
        "batch1": None if sec1 is None else {"images_per_s": round(1.0 / sec1, 2), "ms_per_image": round(sec1 * 1e3, 4),
                                             "passes_in_flight": K1, "passes_in_flight_trial_ms": k1_trial,
                                             "one_pass_at_a_time": {"images_per_s": round(1.0 / sec1_serial, 2),
                                                                    "ms_per_image": round(sec1_serial * 1e3, 4)}},
        "model_create_ms": round(t_create * 1e3, 2),
        "roofline": roofline,
        "roofline_in_flight": roofline_in_flight,
        "kernels": kernels,
        "device": L.nncv_hip_device_arch().decode(),
    }

    if not (args.no_sweep or args.no_batch1):
        out["host_abi"] = host_abi(blob, x)
        out["configs"] = baseline_configs(L, stream, blob32)
        out["bandwidth"] = bandwidth_kernels(L, stream)
        out["conv3x3_sweep"] = conv3x3_sweep(L, stream)
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(blob32, x)
    for h in all_handles:
        L.nncv_hip_resnet18_destroy(h)
    print(json.dumps(out))


def layer_roofline(L, stream, N, C, F, HW, passes, reps=200):
    """One fp16 3x3 stride-1 layer [N,HW,HW,C] -> F with BN + ReLU alone, planned for `passes` passes in flight: `reps`
    launches back to back between one HIP event pair on the launch stream, after a clock warm-up of the same launches."""
    import ctypes
    import numpy as np
    import torch
    from nncv_amd import abi, synth
    w = synth.normal(77, (F, C, 3, 3), std=float(np.sqrt(2.0 / (C * 9)))).astype(np.float16)
    bn = [synth.uniform(78 + i, (F,), 0.5, 1.5).astype(np.float16) for i in range(4)]
    conv = L.nncv_hip_conv_create(abi.F16, w.ctypes.data, F, C, 3, 3, 1, 1, *[b.ctypes.data for b in bn], 1, abi.ALGO_IGEMM)
    if not conv:
        raise RuntimeError(L.nncv_hip_last_error().decode())
    xin = torch.randn((N, HW, HW, C), device="cuda", dtype=torch.float16)
    yout = torch.empty((N, HW, HW, F), device="cuda", dtype=torch.float16)
    avg = ctypes.c_float(0.0)
    abi.check(L.nncv_hip_set_overlap_hint(passes))
    try:
        abi.profile_enable(True)
        abi.profile_report()
        abi.check(L.nncv_hip_conv_forward(conv, xin.data_ptr(), N, HW, HW, abi.NHWC, None, yout.data_ptr(), stream))
        tags = list(abi.profile_report())
        abi.profile_enable(False)
        abi.check(L.nncv_hip_conv_time(conv, xin.data_ptr(), N, HW, HW, None, yout.data_ptr(), 4000, stream, ctypes.byref(avg)))  # clocks
        abi.check(L.nncv_hip_conv_time(conv, xin.data_ptr(), N, HW, HW, None, yout.data_ptr(), reps, stream, ctypes.byref(avg)))
    finally:
        abi.profile_enable(False)
        abi.check(L.nncv_hip_set_overlap_hint(1))
        L.nncv_hip_conv_destroy(conv)
    us = float(avg.value)
    flops = 2.0 * N * HW * HW * F * C * 9
    achieved = flops / (us * 1e-6) / 1e12
    return {"kernel": tags[0] if tags else None, "bound": "mfma", "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "achieved": round(achieved, 3), "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 5), "avg_launch_us": round(us, 3),
            "launches": reps, "flops_per_launch": flops, "planned_for_passes_in_flight": passes,
            "timing": "layer [%d,%d,%d,%d]->%d alone, %d back-to-back launches between one HIP event pair" % (N, HW, HW, C, F, reps)}


def host_abi(blob16, x16, calls=60):
    """images/s through _mlir_ciface_forward_f16 with HOST buffers in and out, as the reference's driver calls and
    times its compiled model (examples/Res18/main.cpp:95-99): input upload, forward pass, logits download and the
    callee-allocated result are all inside.  The first call (blob upload, BN fold, filter re-lay) is reported alone."""
    import numpy as np
    from nncv_amd import abi
    res = {}
    for name, n in (("bs32", x16.shape[0]), ("bs1", 1)):
        xs = np.ascontiguousarray(x16[:n])
        t0 = time.perf_counter()
        abi.forward(xs, blob16)
        first = time.perf_counter() - t0
        for _ in range(10):
            abi.forward(xs, blob16)
        t0 = time.perf_counter()
        for _ in range(calls):
            abi.forward(xs, blob16)
        dt = (time.perf_counter() - t0) / calls
        res[name] = {"images_per_s": round(n / dt, 1), "ms_per_call": round(dt * 1e3, 4), "calls": calls,
                     "first_call_ms": round(first * 1e3, 2)}
    res["what"] = ("_mlir_ciface_forward_f16(dst, src, params) on pageable host arrays, PCIe transfers and the result's "
                   "posix_memalign included; the first call of the process builds the device model")
    return res


def baseline_configs(L, stream, blob32):
    """BASELINE configs 1-3, device-resident, each after a clock warm-up of the same work.
    cfg1: C[1024,1024] += A.B fp32 (tests/MatMulOptimization/MatMulDeafult.mlir:6-9), 200 launches back to back.
    cfg2: the single fp32 3x3 convolution [1,64,56,56] x [64,64,3,3], direct form and Winograd F(4x4,3x3) route.
    cfg3: the fp32 network on one 256x256 image."""
    import ctypes
    import numpy as np
    import torch
    from nncv_amd import abi, synth
    out = {}
    avg = ctypes.c_float(0.0)
    a, b = synth.cfg1_matmul()
    ad, bd = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    cd = torch.zeros((1024, 1024), dtype=torch.float32, device="cuda")
    for reps in (3000, 200):
        abi.check(L.nncv_hip_matmul_time(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), 1024, 1024, 1024, reps, stream, ctypes.byref(avg)))
    tf = 2.0 * 1024 ** 3 / (avg.value * 1e-6) / 1e12
    out["cfg1_matmul_1024"] = {"avg_launch_us": round(float(avg.value), 2), "tflops": round(tf, 2), "launches": 200,
                               "frac_of_fp32_mfma_peak": round(tf / MFMA_F32_PEAK_TFLOPS, 4)}
    x, w = synth.cfg2_conv()
    xin = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 2, 3, 1))).cuda()
    yout = torch.empty((1, 56, 56, 64), dtype=torch.float32, device="cuda")
    cfg2 = {}
    for name, algo in (("direct", abi.ALGO_IGEMM), ("winograd", abi.ALGO_WINOGRAD)):
        conv = L.nncv_hip_conv_create(abi.F32, w.ctypes.data, 64, 64, 3, 3, 1, 1, None, None, None, None, 0, algo)
        if not conv:
            raise RuntimeError(L.nncv_hip_last_error().decode())
        for reps in (3000, 200):
            abi.check(L.nncv_hip_conv_time(conv, xin.data_ptr(), 1, 56, 56, None, yout.data_ptr(), reps, stream, ctypes.byref(avg)))
        L.nncv_hip_conv_destroy(conv)
        cfg2[name + "_us"] = round(float(avg.value), 2)
    cfg2["gflop"] = round(2.0 * 56 * 56 * 64 * 64 * 9 / 1e9, 4)
    cfg2["note"] = "per forward call of the layer, all its launches (Winograd: input transform, 36-batched GEMM, output transform)"
    out["cfg2_conv3x3_fp32"] = cfg2
    model = L.nncv_hip_resnet18_create(blob32.ctypes.data, blob32.size, abi.F32, abi.ALGO_AUTO)
    if not model:
        raise RuntimeError(L.nncv_hip_last_error().decode())
    x3 = torch.from_numpy(synth.cfg3_input()).cuda()
    l3 = torch.empty((1, 1000), dtype=torch.float32, device="cuda")

    def step3():
        abi.check(L.nncv_hip_resnet18_forward(model, x3.data_ptr(), 1, 256, 256, l3.data_ptr(), stream))

    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < CLOCK_WARMUP_MS:
        for _ in range(20):
            step3()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(200):
        step3()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / 200 * 1e3
    L.nncv_hip_resnet18_destroy(model)
    out["cfg3_resnet18_fp32_bs1_256"] = {"ms_per_image": round(ms, 4), "images_per_s": round(1e3 / ms, 1), "steps": 200,
                                         "tflops_effective": round(4.738e9 / (ms * 1e-3) / 1e12, 3)}
    return out


def bandwidth_kernels(L, stream, batch=256, reps=50):
    """The bandwidth-bound kernels against the HBM peak, algorithmic bytes / average launch time: Winograd F(4x4,3x3)
    input and output transforms on layer1's shape (fp16 NHWC [batch,56,56,64]: read the tensor, write the 36 x tiles x
    C transformed one, and back) and the stand-alone 3x3 stride-2 max-pool ([batch,112,112,64] -> [batch,56,56,64]).
    `reps` calls between two events after a clock warm-up; the batch is large so that the host's call rate is not what
    is measured."""
    import torch
    from nncv_amd import abi
    C, H = 64, 56
    tiles = batch * (H // 4) * (H // 4)
    x = torch.randn((batch, H, H, C), device="cuda", dtype=torch.float16)
    V = torch.empty((36, tiles, C), device="cuda", dtype=torch.float16)
    y = torch.empty((batch, H, H, C), device="cuda", dtype=torch.float16)
    big = torch.randn((batch, 112, 112, C), device="cuda", dtype=torch.float16)

    def t_input():
        abi.check(L.nncv_hip_wino43_input(abi.F16, x.data_ptr(), abi.NHWC, V.data_ptr(), batch, C, H, H, 1, stream))

    def t_output():
        abi.check(L.nncv_hip_wino43_output(abi.F16, V.data_ptr(), y.data_ptr(), abi.NHWC, batch, C, H, H, None, None, None, 0, stream))

    def t_pool():
        abi.check(L.nncv_hip_maxpool3x3s2(abi.F16, big.data_ptr(), y.data_ptr(), batch, 112, 112, C, stream))

    def timed(fn):
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < CLOCK_WARMUP_MS:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    out = {}
    es = 2
    for name, fn, nbytes in (("wino43_input_transform", t_input, es * (batch * H * H * C + 36 * tiles * C)),
                             ("wino43_output_transform", t_output, es * (36 * tiles * C + batch * H * H * C)),
                             ("maxpool3x3s2", t_pool, es * batch * C * (112 * 112 + 56 * 56))):
        us = timed(fn)
        gbs = nbytes / (us * 1e-6) / 1e9
        out[name] = {"avg_launch_us": round(us, 2), "algorithmic_mb": round(nbytes / 1e6, 2), "gbs": round(gbs, 1),
                     "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    out["shape"] = "fp16 NHWC, batch %d: transforms on [N,56,56,64] (layer1), pool [N,112,112,64] -> [N,56,56,64]" % batch
    return out


def conv3x3_sweep(L, stream, batch=64, reps=200):
    """BASELINE config 5: the seven 3x3 layer shapes of ResNet-18 at batch 64, fp16, each fused with
    BN + ReLU (+ the residual add on the stride-1 rows), one layer at a time: `reps` launches back to
    back between one HIP event pair.  Weights and BN are the seeded ones of the parity tests; the
    activations are device-side normals (the time does not depend on their values)."""
    import ctypes
    import numpy as np
    import torch
    from nncv_amd import abi, synth
    rows = []
    for i, (c, k, h, st) in enumerate(synth.CFG5_LAYERS):
        seed = 5000 + 10 * i
        w = synth.normal(seed + 1, (k, c, 3, 3), std=float(np.sqrt(2.0 / (c * 9)))).astype(np.float16)
        bn = [synth.uniform(seed + 2, (k,), 0.5, 1.5), synth.normal(seed + 3, (k,), std=0.1),
              synth.normal(seed + 4, (k,), std=0.1), synth.uniform(seed + 5, (k,), 0.5, 1.5)]
        bn = [b.astype(np.float16) for b in bn]
        conv = L.nncv_hip_conv_create(abi.F16, w.ctypes.data, k, c, 3, 3, st, 1, *[b.ctypes.data for b in bn], 1, abi.ALGO_AUTO)
        if not conv:
            raise RuntimeError(L.nncv_hip_last_error().decode())
        oh = (h + 2 - 3) // st + 1
        xin = torch.randn((batch, h, h, c), device="cuda", dtype=torch.float16)
        res = torch.randn((batch, oh, oh, k), device="cuda", dtype=torch.float16) if st == 1 else None
        yout = torch.empty((batch, oh, oh, k), device="cuda", dtype=torch.float16)
        avg = ctypes.c_float(0.0)
        for r in (3000, reps):  # the first pass is the clock warm-up
            abi.check(L.nncv_hip_conv_time(conv, xin.data_ptr(), batch, h, h, res.data_ptr() if res is not None else None,
                                           yout.data_ptr(), r, stream, ctypes.byref(avg)))
        L.nncv_hip_conv_destroy(conv)
        flops = 2.0 * batch * oh * oh * k * c * 9
        tf = flops / (avg.value * 1e-6) / 1e12
        rows.append({"layer": "%d->%d %dx%d s%d" % (c, k, h, h, st), "gflop": round(flops / 1e9, 2),
                     "avg_launch_us": round(float(avg.value), 2), "tflops": round(tf, 1),
                     "frac_of_fp16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4)})
    return {"batch": batch, "dtype": "f16", "epilogue": "BN + ReLU (+ residual on stride-1 rows)", "launches": reps, "rows": rows}


def bench_graph(args, L):
    """MobileNetV3-small ([batch,3,224,224] -> [batch,1000]) or YOLOv5s ([batch,3,640,640] -> [batch,25200,85]) forward, fp16
    storage / fp32 accumulate, input resident in HBM, through nncv_hip_graph_forward; same timing protocol as the
    headline workload."""
    import numpy as np
    import torch
    from nncv_amd import abi, synth
    import oracle

    yolo = args.workload == "yolov5s"
    N, H = args.batch, args.image or (640 if yolo else 224)
    if yolo:
        from nncv_amd import yolov5s_spec as mspec
        blob32, ops = synth.yolov5s_params(), mspec.graph_ops()
        name, fixture = "YOLOv5s", "tests/Nets/Yolov5s.mlir"
    else:
        from nncv_amd import mobilenetv3_spec as mspec
        blob32, ops = synth.mobilenetv3_params(), abi.mobilenetv3_small_ops()[0]
        name, fixture = "MobileNetV3-small", "tests/Nets/MobileNetV3.mlir"
    # passes in flight: graph handle i and stream i serve steps i, i + K ... (see main)
    asked1 = 1 if args.no_batch1 else args.in_flight_batch1
    KMAX = max(args.in_flight, asked1, max(IN_FLIGHT_CANDIDATES) if 0 in (args.in_flight, asked1) else 1)
    gs = [abi.graph_create(ops, 3, blob32.astype(np.float16)) for _ in range(KMAX)]
    g = gs[0]
    oc, oh, ow = abi.graph_output_shape(g, H, H)
    per_image = oc * oh * ow
    x = synth.uniform(4000, (N, 3, H, H), 0.0, 1.0).astype(np.float16)
    xd = torch.from_numpy(x).cuda()
    results = [torch.empty((N, per_image), dtype=torch.float32, device="cuda") for _ in range(KMAX)]
    result = results[0]
    stream = torch.cuda.current_stream().cuda_stream
    x1 = xd[:1].contiguous()
    r1 = [torch.empty((1, per_image), dtype=torch.float32, device="cuda") for _ in range(KMAX)]
    pool_streams, stream_probe = [], None
    if KMAX > 1:
        pool_streams, stream_probe = library_streams(L, KMAX)

    def step(xt, out, n):
        abi.check(L.nncv_hip_graph_forward(g, xt.data_ptr(), n, H, H, out.data_ptr(), n * per_image, stream))

    def timed(xt, out_list, n, warmup, steps, k_in_flight):
        def go(i):
            j = i % k_in_flight
            sj = stream if k_in_flight == 1 else pool_streams[j]  # see main: pool streams when passes overlap
            abi.check(L.nncv_hip_graph_forward(gs[j], xt.data_ptr(), n, H, H, out_list[j].data_ptr(), n * per_image, sj))
        # the operator-list executor plans with the process-wide default of passes in flight
        abi.check(L.nncv_hip_set_overlap_hint(1 if args.no_overlap_hint else k_in_flight))
        # clock warm-up: untimed steps until CLOCK_WARMUP_MS of wall time have passed, then the W asked for
        t_w = time.perf_counter()
        while (time.perf_counter() - t_w) * 1e3 < CLOCK_WARMUP_MS:
            for i in range(20):
                go(i)
            torch.cuda.synchronize()
        for i in range(warmup):
            go(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            go(i)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        abi.check(L.nncv_hip_set_overlap_hint(1))
        return dt / steps

    def pick_in_flight(asked, xt, out_list, n):
        if asked > 0:
            return asked, None
        trial = {k: timed(xt, out_list, n, 20, max(30, args.steps // 2), k) for k in IN_FLIGHT_CANDIDATES}
        return min(trial, key=trial.get), {str(k): round(v * 1e3, 4) for k, v in trial.items()}

    K, k_trial = pick_in_flight(args.in_flight, xd, results, N)
    sec = timed(xd, results, N, args.warmup, args.steps, K)
    sec_serial = sec if K == 1 else timed(xd, results, N, args.warmup, args.steps, 1)
    K1, k1_trial = (1, None) if args.no_batch1 else pick_in_flight(args.in_flight_batch1, x1, r1, 1)
    sec1 = None if args.no_batch1 else timed(x1, r1, 1, args.warmup, max(args.steps, 50), K1)
    sec1_serial = None if args.no_batch1 else (sec1 if K1 == 1 else timed(x1, r1, 1, args.warmup, max(args.steps, 50), 1))
    abi.profile_enable(True)
    abi.profile_report()
    for _ in range(args.profile_steps):
        step(xd, result, N)
    torch.cuda.synchronize()
    prof = abi.profile_report()
    abi.profile_enable(False)
    total_ms = sum(v["ms"] for v in prof.values()) or 1.0
    kernels = {}
    for tag, v in sorted(prof.items(), key=lambda kv: -kv[1]["ms"]):
        kernels[tag] = {"launches_per_step": v["launches"] / args.profile_steps, "ms_per_step": round(v["ms"] / args.profile_steps, 5),
                        "share": round(v["ms"] / total_ms, 4), "avg_launch_us": round(v["ms"] / v["launches"] * 1e3, 3),
                        "tflops": round(v["flops"] / (v["ms"] * 1e-3) / 1e12, 3) if v["flops"] else None,
                        "gbs": round(v["bytes"] / (v["ms"] * 1e-3) / 1e9, 2)}
    # Dominant tag, one HIP event pair per launch (~4 us of event latency included).  MobileNetV3's launches move a
    # few MB each: priced in algorithmic bytes against HBM.  YOLOv5s' dominant tag is an MFMA convolution instance.
    dom = max(prof, key=lambda t: prof[t]["ms"])
    d = prof[dom]
    if yolo and d["flops"] > 0:
        achieved = d["flops"] / (d["ms"] * 1e-3) / 1e12
        roofline = {"kernel": dom, "bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 5)}
    else:
        achieved = d["bytes"] / (d["ms"] * 1e-3) / 1e9
        roofline = {"kernel": dom, "bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 5)}
    roofline.update({"traffic": None, "avg_launch_us": round(d["ms"] / d["launches"] * 1e3, 3), "launches": d["launches"],
                     "timing": "one HIP event pair per launch, all launches of the tag in %d passes" % args.profile_steps})
    flops_step = mspec.flops_per_image(H) * N
    out = {
        "metric": "%s_fp16_bs%d_images_per_s" % ("yolov5s" if yolo else "mobilenetv3_small", N), "value": round(N / sec, 2),
        "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "%s forward (the network of %s), fp16, input [%d,3,%d,%d], seeded U[0,1] input, random-init weights "
                               "from a model.bin-order blob" % (name, fixture, N, H, H),
                   "batch": N, "image": H, "input_resident_in_hbm": True, "passes_in_flight": K,
                   "passes_in_flight_trial_ms": k_trial, "stream_probe": stream_probe},
        "tflops_effective": round(flops_step / sec / 1e12, 3),
        "one_pass_at_a_time": {"images_per_s": round(N / sec_serial, 2), "ms_per_step": round(sec_serial * 1e3, 4)},
        "batch1": None if sec1 is None else {"images_per_s": round(1.0 / sec1, 2), "ms_per_image": round(sec1 * 1e3, 4),
                                             "passes_in_flight": K1, "passes_in_flight_trial_ms": k1_trial,
                                             "one_pass_at_a_time": {"images_per_s": round(1.0 / sec1_serial, 2),
                                                                    "ms_per_image": round(sec1_serial * 1e3, 4)}},
        "roofline": roofline, "kernels": kernels, "device": L.nncv_hip_device_arch().decode(),
    }
    if not args.no_cpu_baseline:
        hb = synth.round_fp16(blob32)
        xf = x.astype(np.float32)
        nb = min(2 if yolo else 8, N)
        if yolo:
            run = lambda xs: oracle.run_graph(ops, xs, hb, 3, conv=oracle.hwp_conv2d)
            what = "operator-list evaluator of oracle/ with the OpenMP x AVX2 convolution (oracle/hostwparallel.cpp), numpy for the rest"
            cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", 1 << 10)))
        else:
            T = {n_: hb[o:o + mspec.numel(shape)].reshape(shape) for n_, (o, shape) in mspec.offsets().items()}
            run = lambda xs: oracle.mobilenetv3_forward(xs, T)
            what = "scalar C / numpy restatement of the fixture's operators (oracle/)"
            cores = 1
        run(xf[:1])
        done, t0 = 0, time.perf_counter()
        while True:
            run(xf[:nb])
            done += nb
            dt = time.perf_counter() - t0
            if dt > 10.0 or done >= 4096:
                break
        out["cpu_baseline"] = {"value": round(done / dt, 3), "unit": "images/s", "cores": cores, "kind": "port",
                               "sample": "%d images (batches of %d) in %.1f s; fp32, %s" % (done, nb, dt, what)}
    for h in gs:
        L.nncv_hip_graph_destroy(h)
    print(json.dumps(out))


def cpu_baseline(blob32, x16):
    """CPU baselines timed on this host: fp32 ResNet-18 forward of the first images of the same batch (half-rounded
    weights and input, like the parity tests), convolutions in oracle/hostwparallel.cpp, the other ops in the scalar
    oracle.  `value` / `value_4_threads`: this repository's own OpenMP x AVX2 convolution ((image, filter) pairs across
    threads) on all cores / on the reference's default of 4 threads; `value_ref_schedule`: the reference's tile order,
    which is sequential.  Bounded: one warm-up call each, then 12 + 6 + 6 s of forward passes."""
    import numpy as np
    import oracle
    from nncv_amd import synth
    hb = synth.round_fp16(blob32)
    x = x16.astype(np.float32)
    cores = len(os.sched_getaffinity(0))
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    nb = min(8, x.shape[0])
    def cpu_model():
        try:
            for line in open("/proc/cpuinfo"):
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
        except OSError:
            pass
        return "unknown"

    def rate(threads, budget_s, schedule="omp", batch=nb):
        oracle.hwp_threads(threads)
        oracle.hwp_resnet18_forward(x[:1], hb, schedule=schedule)
        done, t0 = 0, time.perf_counter()
        while True:
            oracle.hwp_resnet18_forward(x[:batch], hb, schedule=schedule)
            done += batch
            dt = time.perf_counter() - t0
            if dt > budget_s or done >= 4096:
                return done, dt

    done, dt = rate(cores, 12.0)
    # the reference's own default is `-num-threads 4` (src/nncv/compiler/main.cpp:231)
    done4, dt4 = rate(min(4, cores), 6.0)
    # the reference's schedule: convolutions tiled with sequential scf.for (ModernTile.cpp:330-331), i.e. on one thread
    doner, dtr = rate(1, 6.0, schedule="ref", batch=1)
    oracle.hwp_threads(cores)
    return {"value": round(done / dt, 3), "unit": "images/s", "cores": cores, "kind": "port",
            "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
            "value_4_threads": round(done4 / dt4, 3),
            "value_ref_schedule": round(doner / dtr, 3),
            "sample": "value: %d images (batches of %d from the same input) in %.1f s on %d threads; value_4_threads: %d images in "
                      "%.1f s on 4 threads (the reference's default -num-threads) -- both with this repository's own OpenMP x AVX2 "
                      "convolution, (image, filter) pairs across threads, which is faster than the reference's schedule; "
                      "value_ref_schedule: %d images in %.1f s with the convolutions in the reference's tile order, which is "
                      "sequential (ModernTile.cpp:184-199, :330-331), AVX2 8x8 blocks, one thread; fp32; every other operator "
                      "on the scalar oracle (oracle/hostwparallel.cpp, oracle/nncv_oracle.c)" % (done, nb, dt, cores, done4, dt4, doner, dtr)}


if __name__ == "__main__":
    main()
