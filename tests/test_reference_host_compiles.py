"""The reference's own host translation unit against this library's two driver headers.

The reference's `hp_cuda.cpp` declares the nine kernel drivers by hand (hp_cuda.cpp:18-102) and calls them from its
scheduler loops (hp_cuda.cpp:284-301, :464-477, :610-611, :729-752).  A maintainer swaps that block of declarations
for `#include "hp_cuda_shim.h"` and `#include "hp_cuda_shim_torch.h"` and links `libhpx.so` in place of
`hp_cuda_kernel.cu`.  `oracle/ref_host.py` does exactly that to the reference's file, read where it lies at test
time (nothing of it is kept; the test skips where the reference is absent), runs the source renames that
PyTorch-ROCm's extension build applies (`torch.utils.hipify`), compiles the result with the host compiler and links
it against `libhpx.so` and libtorch with `--no-undefined`.  The test holds that build to: no edit beyond the swap,
every driver bound to this library, and a module that imports and shows the reference's Python interface.
"""
import os
import subprocess
import sys

import pytest

from oracle import ref_host

pytestmark = pytest.mark.skipif(not ref_host.available(), reason="the reference's sources are not on this machine")


def test_reference_host_file_compiles_and_links_against_the_driver_headers(tmp_path):
    if not os.path.exists(os.path.join(ref_host.PKG, "libhpx.so")):
        import __graft_entry__
        __graft_entry__.ensure_built()
    so, extra_edits = ref_host.build(out_dir=str(tmp_path))
    assert extra_edits == [], extra_edits                    # "nothing else in hp_cuda.cpp changes"
    # the six vector-based drivers come from libhpx.so; the PowerSGD templates were instantiated for the stream
    # type the renamed source passes and call the C ABI
    nm = subprocess.run(["nm", "-D", "--undefined-only", "-C", so], capture_output=True, text=True).stdout
    for name in ("hp_cuda_terngrad(", "hp_cuda_terngradr(", "hp_cuda_tbq(", "hp_cuda_tbqr(", "hp_cuda_gd(", "hp_cuda_gdr(",
                 "hpx_powersgd_encode1", "hpx_powersgd_encode2", "hpx_powersgd_decode"):
        assert name in nm, name
    # it imports (in a process of its own: the module starts threads and keeps static state) and carries the
    # reference's interface, hp_cuda.cpp:1073-1080
    code = ("import sys, torch; sys.path.insert(0, %r); import hp_cuda; "
            "print(sorted(n for n in dir(hp_cuda) if not n.startswith('_'))); print(hp_cuda.getResults(10))" % str(tmp_path))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    assert "['end', 'getResults', 'init', 'submit_task']" in r.stdout and r.stdout.strip().endswith("[]"), r.stdout
