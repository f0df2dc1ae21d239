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


@pytest.fixture(params=["compiled", "ctypes"])
def hp(request, pkg, hp_cuda_compiled):
    return hp_cuda_compiled if request.param == "compiled" else pkg.hp_cuda


def test_compiled_module_has_the_reference_interface(hp_cuda_compiled):
    # PYBIND11_MODULE(hp_cuda), hp_cuda.cpp:1073-1080: init, end, getResults and three submit_task overloads
    for name in ("init", "end", "getResults", "submit_task"):
        assert callable(getattr(hp_cuda_compiled, name))
    doc = hp_cuda_compiled.submit_task.__doc__
    assert doc.count("torch.Tensor") == 3 + 4 + 5 and "Overloaded function" in doc
    assert (hp_cuda_compiled.COMP_TASK, hp_cuda_compiled.DECOMP_TASK, hp_cuda_compiled.ROOT_DECOMP_COMP_TASK,
            hp_cuda_compiled.POWERSGD_ENCODE1, hp_cuda_compiled.POWERSGD_ENCODE2,
            hp_cuda_compiled.POWERSGD_DECODE) == (10, 20, 30, 40, 50, 60)          # hp_cuda.h:21-26


def test_unknown_algorithm_and_bad_ids(hp, capsys):
    assert hp.init("ecq", {}, 0, 0, 1) is False                 # hp_cuda.cpp:846-849
    assert "only support terngrad, tbq, graddrop and powersgd now" in hp.last_error()
    assert hp.getResults(10) == [] and hp.getResults(40) == []
    assert hp.getResults(15) == []                              # hp_cuda.cpp:1062-1063
    assert "not invalid task_id in getResults: 15" in hp.last_error()
    assert hp.wait(20, 1) is False
    assert hp.end() is True                                     # end without init is harmless


def test_submit_without_running_threads_raises(hp):
    import torch
    t = torch.zeros(8)
    with pytest.raises(RuntimeError, match="CUDA tensor"):      # CHECK_CUDA_INPUT, hp_cuda.cpp:107-111
        hp.submit_task("x", t, t, t, 0, 10)
