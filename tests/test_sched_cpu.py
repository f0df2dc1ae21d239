"""CPU-side checks of the scheduler boundary (include/hpx_sched.h): exports, argument checks, the
reference's messages.  Nothing here touches a GPU."""
import ctypes as C
import os
import re

import pytest


def test_library_exports_every_declared_scheduler_symbol(capi):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "include", "hpx_sched.h")).read()
    declared = set(re.findall(r"\b(hpx_sched_[a-z0-9_]+)\s*\(", text))
    assert declared == set(capi.SCHED_SYMBOLS)
    L = capi.load()
    for name in declared:
        assert hasattr(L, name)


def test_task_struct_layout_matches_the_header(capi):
    # hpx_task_t: pointer, 2 x int32, then (pointer, int64) x 4, 3 pointers, 3 x int32 (+ padding)
    assert C.sizeof(capi.Task) == 8 + 8 + 4 * 16 + 3 * 8 + 16
    assert capi.Task.tensor.offset == 16 and capi.Task.C_bytes.offset == 72 and capi.Task.n.offset == 104


def test_unknown_algorithm_and_bad_ids(pkg, capsys):
    hp = pkg.hp_cuda
    assert hp.init("ecq", {}, 0, 0, 1) is False                 # hp_cuda.cpp:846-849
    assert "only support terngrad, tbq, graddrop and powersgd now" in hp.last_error()
    assert hp.getResults(10) == [] and hp.getResults(40) == []
    assert hp.getResults(15) == []                              # hp_cuda.cpp:1062-1063
    assert "not invalid task_id in getResults: 15" in hp.last_error()
    assert hp.wait(20, 1) is False
    assert hp.end() is True                                     # end without init is harmless


def test_submit_without_running_threads_raises(pkg):
    import torch
    hp = pkg.hp_cuda
    t = torch.zeros(8)
    with pytest.raises(RuntimeError, match="CUDA tensor"):      # CHECK_CUDA_INPUT, hp_cuda.cpp:107-111
        hp.submit_task("x", t, t, t, 0, 10)
