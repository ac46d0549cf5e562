"""bench.py's host logic, without a GPU: the refusal of more than one GPU (the stream probe lives in the library:
nncv_hip_pick_streams, tests/test_gpu_driver.py)."""
import importlib.util
import os
import subprocess
import sys

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
