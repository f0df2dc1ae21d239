"""What of bench.py's contract can be held without a GPU: one GPU only (a request for more says so and exits),
no GPU says so and exits, and the defaults of the flags the driver passes."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, env=None):
    e = dict(os.environ)
    e.pop("WORLD_SIZE", None)
    e.update(env or {})
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, env=e, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode == 2 and "one GPU" in r.stderr and not r.stdout.strip(), (r.returncode, r.stderr)
    r = _run(env={"WORLD_SIZE": "2"})
    assert r.returncode == 2 and "one GPU" in r.stderr, (r.returncode, r.stderr)


def test_flags_and_defaults():
    sys.path.insert(0, ROOT)
    import bench
    old = sys.argv
    try:
        sys.argv = ["bench.py"]
        a = bench.parse()
        assert (a.gpus, a.steps, a.warmup) == (1, 200, 20) and a.settle_ms == 40.0 and not a.no_extra and not a.no_cpu
        sys.argv = ["bench.py", "--gpus", "1", "--steps", "7", "--warmup", "3", "--settle-ms", "0"]
        a = bench.parse()
        assert (a.gpus, a.steps, a.warmup, a.settle_ms) == (1, 7, 3, 0.0)
    finally:
        sys.argv = old
    assert set(bench.EXTRAS) >= {"tbq", "terngrad_resnet50", "terngrad_sizes", "dgc", "powersgd", "scheduler"}
