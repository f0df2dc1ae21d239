"""MI355X-native gradient-compression hot path (TBQ, TernGrad, GradDrop/DGC,
PowerSGD) behind the reference extension's kernel-driver interface.

  _capi        ctypes binding of libhpx.so (C ABI, include/hpx.h)
  hp_cuda_ops  the nine hp_cuda_* driver functions of the reference, as Python
               callables over torch device tensors
  hp_cuda      the reference's Python module (init / end / submit_task /
               getResults) over the task scheduler of libhpx.so
"""
from . import _capi
from . import hp_cuda
from .hp_cuda_ops import (hp_cuda_gd, hp_cuda_gdr, hp_cuda_powersgd_decode, hp_cuda_powersgd_encode1,
                          hp_cuda_powersgd_encode2, hp_cuda_tbq, hp_cuda_tbqr, hp_cuda_terngrad,
                          hp_cuda_terngradr)

__all__ = [
    "_capi", "hp_cuda", "hp_cuda_tbq", "hp_cuda_tbqr", "hp_cuda_terngrad", "hp_cuda_terngradr", "hp_cuda_gd",
    "hp_cuda_gdr", "hp_cuda_powersgd_encode1", "hp_cuda_powersgd_encode2", "hp_cuda_powersgd_decode",
]
