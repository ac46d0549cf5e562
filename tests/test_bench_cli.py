"""bench.py's host logic, without a GPU: the refusal of more than one GPU and the stream probe."""
import importlib.util
import os
import subprocess
import sys
import time
import types

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    for extra_env, argv in (({}, ["--gpus", "2"]), ({"WORLD_SIZE": "2"}, [])):
        env = dict(os.environ, **extra_env)
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + argv, env=env, capture_output=True, text=True, timeout=120)
        assert r.returncode != 0
        assert "--gpus 1" in r.stderr and r.stdout.strip() == ""


class FakeGpu:
    """Eight streams dealt to hardware queues the way a runtime with four queues was seen to deal them (two streams on one
    queue run one after the other, two queues on one pipe gain 14 %); synchronize() sleeps for what the enqueued passes cost."""

    def __init__(self, queue_of_stream, pass_s=2e-4):
        self.queue_of_stream, self.pass_s, self.pending, self.made = queue_of_stream, pass_s, [], 0
        self.cuda = types.SimpleNamespace(Stream=self.stream, synchronize=self.synchronize)

    def stream(self):
        s = types.SimpleNamespace(cuda_stream=1000 + self.made)
        self.made += 1
        return s

    def run_pass(self, handle, stream):
        self.pending.append(stream - 1000)

    def synchronize(self):
        per_stream = {}
        for s in self.pending:
            per_stream[s] = per_stream.get(s, 0) + 1
        self.pending = []
        if not per_stream:
            return
        # passes on one queue add up; queues on one pipe (queue mod 4) slow each other to 1.75x of one; pipes run side by side
        per_queue = {}
        for s, n in per_stream.items():
            q = self.queue_of_stream[s]
            per_queue[q] = per_queue.get(q, 0) + n
        per_pipe = {}
        for q, n in per_queue.items():
            per_pipe.setdefault(q % 4, []).append(n)
        cost = max(sum(v) * (1.0 if len(v) == 1 else 0.875) for v in per_pipe.values())
        time.sleep(cost * self.pass_s)


def test_stream_probe_takes_streams_that_overlap():
    bench = load_bench()
    # streams 2 and 3 share queue 2, 4 shares queue 1, 5 shares queue 0, 6 is alone on queue 3, 7 joins queue 2
    gpu = FakeGpu([0, 1, 2, 2, 1, 0, 3, 2])
    taken, report = bench.concurrent_streams(gpu, gpu.run_pass, 4)
    assert [t.cuda_stream - 1000 for t in taken] == [0, 1, 2, 6]
    assert report == {"candidates": 8, "overlapping": 4}
    # eight queues on four pipes: stream 4 sits on the pipe of stream 0 and is passed over
    gpu = FakeGpu([0, 1, 2, 3, 4, 5, 6, 7])
    taken, report = bench.concurrent_streams(gpu, gpu.run_pass, 4)
    assert [t.cuda_stream - 1000 for t in taken] == [0, 1, 2, 3] and report["overlapping"] == 4
    # every stream on one queue: nothing overlaps, the probe says so and still hands back the number asked for
    gpu = FakeGpu([0] * 8)
    taken, report = bench.concurrent_streams(gpu, gpu.run_pass, 3)
    assert len(taken) == 3 and report["overlapping"] == 1
