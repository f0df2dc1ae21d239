"""The reference's Python-visible module, `hp_cuda` (PYBIND11_MODULE, hp_cuda.cpp:1073-1080):

    init(alg_name, alg_paras, device_id, rank_id, size) -> bool        hp_cuda.cpp:824-874
    end() -> bool                                                      hp_cuda.cpp:883-890
    submit_task(name, tensor, B, C, is_root, task_id) -> bool          hp_cuda.cpp:984-1013
    submit_task(name, tensor, residual, B, C, is_root, task_id)        hp_cuda.cpp:936-981
    submit_task(name, tensor, residual, M, P, Q, task_id)              hp_cuda.cpp:1015-1041
    getResults(task_id) -> list[str]                                   hp_cuda.cpp:1043-1066

over the scheduler of libhpx.so (include/hpx_sched.h).  Same names, argument
order, checks and printed messages; task ids 10/20/30 (comp, decomp, root
decomp+comp) and 40/50/60 (PowerSGD encode1, encode2, decode).

Like the reference's Task (hp_cuda.h:28-51), a submitted task keeps its tensors
alive until the scheduler is done with them.  `wait(task_id, timeout_ms)` is an
addition: the reference's callers poll getResults.
"""
import ctypes as C

import torch

from . import _capi

COMP_TASK = 10
DECOMP_TASK = 20
ROOT_DECOMP_COMP_TASK = 30
POWERSGD_ENCODE1 = 40
POWERSGD_ENCODE2 = 50
POWERSGD_DECODE = 60

_alive = {}   # serial -> tensors of a task in flight


def _check_cuda_input(x, what):
    # CHECK_CUDA_INPUT, hp_cuda.cpp:107-111 (TORCH_CHECK throws)
    if not x.is_cuda:
        raise RuntimeError(f"{what} must be a CUDA tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{what} must be contiguous")


def _check_cpu_input(x, what):
    if x.is_cuda:
        raise RuntimeError(f"{what} must be a CPU tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{what} must be contiguous")


def _release_done():
    L = _capi.load()
    buf = (C.c_uint64 * 256)()
    while True:
        n = L.hpx_sched_take_done(buf, 256)
        for i in range(n):
            _alive.pop(buf[i], None)
        if n < 256:
            break


def init(alg_name, alg_paras, device_id, rank_id, size):
    """Starts the scheduler for one algorithm: "terngrad" {enable_random, bitwidth}, "tbq" {threshold},
    "graddrop" {drop_ratio, sample_rate} or "powersgd" {matrix_approximation_rank}.  The optional key
    "seed" fixes the RNG seed of every encode (the reference reads the clock)."""
    L = _capi.load()
    keys = [k.encode() for k in alg_paras]
    vals = [float(alg_paras[k]) for k in alg_paras]
    rc = L.hpx_sched_init(alg_name.encode(), (C.c_char_p * len(keys))(*keys), (C.c_double * len(vals))(*vals),
                          len(keys), int(device_id), int(rank_id), int(size))
    return rc == 0


def end():
    L = _capi.load()
    L.hpx_sched_end()
    _release_done()
    return True


def _submit(name, tensors, task):
    L = _capi.load()
    _release_done()
    serial = C.c_uint64()
    task.name = name.encode()
    rc = L.hpx_sched_submit(C.byref(task), C.byref(serial))
    if rc != 0:
        text = L.hpx_sched_error().decode()
        if "not running" in text:
            raise RuntimeError(text)      # check_thread(), hp_cuda.cpp:892-900 (CHECK aborts)
        return False                      # the reference prints the reason and returns false
    _alive[serial.value] = tensors
    return True


def submit_task(tensor_name, tensor, *args):
    """The three overloads of the reference, told apart by their argument count:
    (B, C, is_root, task_id), (residual, B, C, is_root, task_id), (residual, M, P, Q, task_id)."""
    t = _capi.Task()
    if len(args) == 4:
        B, Cc, is_root, task_id = args
        _check_cuda_input(tensor, "tensor"); _check_cuda_input(B, "B"); _check_cpu_input(Cc, "C")
        residual = None
    elif len(args) == 5 and isinstance(args[3], int):
        residual, B, Cc, is_root, task_id = args
        _check_cuda_input(tensor, "tensor"); _check_cuda_input(residual, "residual")
        _check_cuda_input(B, "B"); _check_cpu_input(Cc, "C")
    elif len(args) == 5:
        residual, M, P, Q, task_id = args
        for x, what in ((tensor, "tensor"), (residual, "residual"), (M, "M"), (P, "P"), (Q, "Q")):
            _check_cuda_input(x, what)
        t.task_id, t.is_root = int(task_id), 0
        t.tensor, t.tensor_numel = tensor.data_ptr(), tensor.numel()
        t.residual, t.residual_numel = residual.data_ptr(), residual.numel()
        t.M, t.P, t.Q = M.data_ptr(), P.data_ptr(), Q.data_ptr()
        t.n, t.m, t.r = int(M.shape[0]), int(M.shape[1]), int(P.shape[1])
        return _submit(tensor_name, (tensor, residual, M, P, Q), t)
    else:
        raise TypeError("submit_task(): incompatible function arguments")
    t.task_id, t.is_root = int(task_id), int(is_root)
    t.tensor, t.tensor_numel = tensor.data_ptr(), tensor.numel()
    if residual is not None:
        t.residual, t.residual_numel = residual.data_ptr(), residual.numel()
    t.B, t.B_bytes = B.data_ptr(), B.numel() * B.element_size()
    t.C, t.C_bytes = Cc.data_ptr(), Cc.numel() * Cc.element_size()
    return _submit(tensor_name, (tensor, residual, B, Cc), t)


def getResults(task_id):
    L = _capi.load()
    out = []
    buf = C.create_string_buffer(1 << 16)
    while True:
        n = L.hpx_sched_get_results(int(task_id), buf, len(buf))
        if n < 0:     # the library has printed the reference's message
            break
        raw = buf.raw
        off = 0
        for _ in range(n):
            end_ = raw.index(b"\0", off)
            out.append(raw[off:end_].decode())
            off = end_ + 1
        if n == 0:
            break
    _release_done()
    return out


def wait(task_id, timeout_ms=1000):
    """Blocks until getResults(task_id) would return something (True) or the time is up (False)."""
    return _capi.load().hpx_sched_wait(int(task_id), int(timeout_ms)) == 1


def error_count():
    return int(_capi.load().hpx_sched_error_count())


def last_error():
    return _capi.load().hpx_sched_error().decode()
