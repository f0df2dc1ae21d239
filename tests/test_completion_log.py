"""Host logic of the log of barrier-launch encodes (csrc/hpx_completion_log.h): records of calls that have finished
well are dropped at the next call, records are never dropped while the expiry flag is up, and what is left is what
a repair has to repeat.  The header has no GPU dependency; the test compiles tests/host_completion_log.cpp with the
host compiler and runs it."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_completion_log_pruning(tmp_path):
    exe = str(tmp_path / "host_completion_log")
    src = os.path.join(ROOT, "tests", "host_completion_log.cpp")
    inc = os.path.join(ROOT, "torch-hipress-extension_amd", "csrc")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-fsanitize=address,undefined",
                           "-I" + inc, src, "-o", exe])
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip() == "OK", (r.stdout, r.stderr)
