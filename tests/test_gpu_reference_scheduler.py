"""The reference's own scheduler and Python module (hp_cuda.cpp, unmodified but for the swap of its nine driver
declarations for this library's two headers; built by oracle/ref_host.py into oracle/_ref/) running on this
library's drivers on the GPU: COMP, DECOMP and ROOT tasks of every algorithm, bit-exact against the CPU oracle.

It is the drop-in claim tested end to end: the drivers are called by the reference's code, on the reference's
streams and threads, and their results are consumed the way the reference consumes them — the copy of B on a
different stream right after the driver returns.  One process per algorithm (tests/ref_sched_worker.py), since the
reference's module fixes its algorithm and its threads at the first init.  Skipped where the module has not been
built (it can only be built where the reference's sources are).
"""
import os
import subprocess
import sys

import pytest

from oracle import ref_host

pytestmark = pytest.mark.gpu

WORKER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_sched_worker.py")


@pytest.mark.skipif(not os.path.exists(ref_host.module_path()), reason="oracle/_ref/hp_cuda module not built")
@pytest.mark.parametrize("alg", ["tbq", "terngrad", "graddrop", "powersgd"])
def test_reference_scheduler_over_this_librarys_drivers(alg, pkg):
    env = dict(os.environ, HPX_CLOCK_SEED="77")
    print(f"worker {alg}", flush=True)
    r = subprocess.run([sys.executable, "-u", WORKER, alg], env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and f"OK {alg}" in r.stdout, (r.returncode, r.stdout[-3000:], r.stderr[-5000:])
