"""CPU-side checks of the drop-in boundary: the library loads and exports every
entry point include/hpx.h declares (no GPU work is issued)."""
import os
import re


def test_library_exports_every_declared_symbol(capi):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "include", "hpx.h")).read()
    declared = set(re.findall(r"\b(hpx_[a-z0-9_]+)\s*\(", text))
    assert declared, "no declarations parsed"
    L = capi.load()
    for name in sorted(declared):
        assert hasattr(L, name), f"libhpx.so lacks {name}"
    assert declared == set(capi.SYMBOLS)


def test_version_and_error_text(capi):
    L = capi.load()
    assert L.hpx_version() >= 100
    assert isinstance(capi.last_error(), str)


def test_argument_validation_needs_no_gpu(capi):
    L = capi.load()
    # negative count is rejected before any HIP call
    assert L.hpx_tbq_encode(-1, None, None, None, None, None, None) == -3
    assert "negative count" in capi.last_error()
    assert L.hpx_tbq_encode(0, None, None, None, None, None, None) == 0
    # the reference's bitwidth check (terngrad_body.h:207-212) runs on the host
    rc = L.hpx_terngrad_encode(1, capi.ptr_array([16]), capi.i32_array([8]), capi.ptr_array([16]),
                               capi.i32_array([12]), capi.u8_array([3]), capi.i32_array([0]), None, None)
    assert rc == -1 and "bitwidth" in capi.last_error()


def test_ops_mirror_reference_names(pkg):
    for name in ("hp_cuda_terngrad", "hp_cuda_terngradr", "hp_cuda_tbq", "hp_cuda_tbqr", "hp_cuda_gd", "hp_cuda_gdr",
                 "hp_cuda_powersgd_encode1", "hp_cuda_powersgd_encode2", "hp_cuda_powersgd_decode"):
        assert callable(getattr(pkg, name))


def test_driver_module_exposes_the_nine_reference_drivers(hp_cuda_compiled):
    import importlib
    drv = importlib.import_module("hp_cuda_drivers")
    for name in ("hp_cuda_terngrad", "hp_cuda_terngradr", "hp_cuda_tbq", "hp_cuda_tbqr", "hp_cuda_gd", "hp_cuda_gdr",
                 "hp_cuda_powersgd_encode1", "hp_cuda_powersgd_encode2", "hp_cuda_powersgd_decode"):
        assert callable(getattr(drv, name))
