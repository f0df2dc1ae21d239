"""ctypes binding of libhpx.so, the C-ABI kernel library (include/hpx.h).

The library is the product: if it has not been built this module raises, it
never falls back to another implementation.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhpx.so")

# every symbol include/hpx.h declares
SYMBOLS = (
    "hpx_version",
    "hpx_last_error",
    "hpx_release_workspaces",
    "hpx_release_stream",
    "hpx_set_option",
    "hpx_get_option",
    "hpx_profile_enable",
    "hpx_profile_reset",
    "hpx_profile_query",
    "hpx_tbq_encode",
    "hpx_tbq_decode",
    "hpx_terngrad_encode",
    "hpx_terngrad_encode_status",
    "hpx_terngrad_repaired",
    "hpx_terngrad_phase_stamps",
    "hpx_terngrad_encode_noalloc",
    "hpx_terngrad_decode",
    "hpx_terngrad_decode_status",
    "hpx_gd_encode",
    "hpx_gd_decode",
    "hpx_gd_fallbacks",
    "hpx_dgc_encode",
    "hpx_dgc_decode",
    "hpx_ecq_encode",
    "hpx_ecq_decode",
    "hpx_powersgd_encode1",
    "hpx_powersgd_encode2",
    "hpx_powersgd_decode",
)

# include/hpx_sched.h
SCHED_SYMBOLS = (
    "hpx_sched_init",
    "hpx_sched_end",
    "hpx_sched_submit",
    "hpx_sched_get_results",
    "hpx_sched_wait",
    "hpx_sched_take_done",
    "hpx_sched_error_count",
    "hpx_sched_error",
)


class Task(C.Structure):
    """hpx_task_t of include/hpx_sched.h."""
    _fields_ = [("name", C.c_char_p), ("task_id", C.c_int32), ("is_root", C.c_int32),
                ("tensor", C.c_void_p), ("tensor_numel", C.c_int64),
                ("residual", C.c_void_p), ("residual_numel", C.c_int64),
                ("B", C.c_void_p), ("B_bytes", C.c_int64),
                ("C", C.c_void_p), ("C_bytes", C.c_int64),
                ("M", C.c_void_p), ("P", C.c_void_p), ("Q", C.c_void_p),
                ("n", C.c_int32), ("m", C.c_int32), ("r", C.c_int32)]


_lib = None


class HpxError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"hpx call failed with code {code}: {text}")
        self.code = code
        self.text = text


def load():
    """Load libhpx.so (built by `make -C csrc`); raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP kernel library first "
            "(python -c 'import __graft_entry__ as g; g.build()' or make -C csrc)")
    L = C.CDLL(LIB_PATH)
    pp, p, i32 = C.c_void_p, C.c_void_p, C.c_int
    L.hpx_version.restype = C.c_int
    L.hpx_last_error.restype = C.c_char_p
    L.hpx_release_workspaces.restype = C.c_int
    L.hpx_profile_enable.argtypes = [C.c_int]
    L.hpx_profile_query.argtypes = [C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_int64)]
    L.hpx_set_option.argtypes = [C.c_char_p, C.c_int64]
    L.hpx_get_option.argtypes = [C.c_char_p, C.POINTER(C.c_int64)]
    L.hpx_tbq_encode.argtypes = [i32, pp, p, pp, pp, p, p]
    L.hpx_tbq_decode.argtypes = [i32, pp, p, pp, p, p, p]
    L.hpx_terngrad_encode.argtypes = [i32, pp, p, pp, p, p, p, p, p]
    L.hpx_terngrad_encode_noalloc.argtypes = [i32, pp, p, pp, p, p, p, p, p]
    L.hpx_terngrad_encode_status.argtypes = [p]
    L.hpx_terngrad_repaired.argtypes = [p]
    L.hpx_terngrad_repaired.restype = C.c_int64
    L.hpx_terngrad_phase_stamps.argtypes = [p, i32]
    L.hpx_gd_fallbacks.argtypes = [p]
    L.hpx_gd_fallbacks.restype = C.c_int64
    L.hpx_release_stream.argtypes = [p]
    L.hpx_terngrad_decode.argtypes = [i32, pp, p, pp, p, p, p]
    L.hpx_terngrad_decode_status.argtypes = [p]
    L.hpx_gd_encode.argtypes = [i32, pp, p, pp, pp, p, p, p, p]
    L.hpx_gd_decode.argtypes = [i32, pp, p, pp, p, p, p]
    L.hpx_dgc_encode.argtypes = [i32, pp, p, pp, p, p, p, p]
    L.hpx_dgc_decode.argtypes = [i32, pp, p, pp, p, p, p]
    L.hpx_ecq_encode.argtypes = [i32, pp, p, pp, pp, p, p, p, p, p, p]
    L.hpx_ecq_decode.argtypes = [i32, pp, p, pp, p, p, p]
    L.hpx_powersgd_encode1.argtypes = [i32, pp, p, pp, pp, pp, pp, p, p, p, p]
    L.hpx_powersgd_encode2.argtypes = [i32, pp, pp, pp, p, p, p, p]
    L.hpx_powersgd_decode.argtypes = [i32, pp, pp, pp, pp, pp, p, p, p, p, p]
    L.hpx_sched_init.argtypes = [C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(C.c_double), C.c_int, C.c_int, C.c_int, C.c_int]
    L.hpx_sched_submit.argtypes = [C.POINTER(Task), C.POINTER(C.c_uint64)]
    L.hpx_sched_get_results.argtypes = [C.c_int, C.c_char_p, C.c_int64]
    L.hpx_sched_get_results.restype = C.c_int64
    L.hpx_sched_wait.argtypes = [C.c_int, C.c_int]
    L.hpx_sched_take_done.argtypes = [C.POINTER(C.c_uint64), C.c_int64]
    L.hpx_sched_take_done.restype = C.c_int64
    L.hpx_sched_error_count.restype = C.c_int64
    L.hpx_sched_error.restype = C.c_char_p
    for name in SYMBOLS + SCHED_SYMBOLS:
        getattr(L, name)  # AttributeError if the build lost an entry point
    _lib = L
    return L


def last_error():
    return load().hpx_last_error().decode()


# ---- marshalling helpers: host arrays of pointers / scalars -----------------
def ptr_array(ptrs):
    return (C.c_void_p * len(ptrs))(*[C.c_void_p(int(x)) for x in ptrs])


def i32_array(vals):
    return (C.c_int32 * len(vals))(*[int(v) for v in vals])


def i64_array(vals):
    return (C.c_int64 * len(vals))(*[int(v) for v in vals])


def u8_array(vals):
    return (C.c_uint8 * len(vals))(*[int(v) & 0xFF for v in vals])


def u64_array(vals):
    return (C.c_uint64 * len(vals))(*[int(v) & 0xFFFFFFFFFFFFFFFF for v in vals])


def f32_array(vals):
    return (C.c_float * len(vals))(*[float(v) for v in vals])


def f64_array(vals):
    return (C.c_double * len(vals))(*[float(v) for v in vals])


def set_option(name, value):
    """Sets a tuning option of the library (see include/hpx.h); returns the previous value."""
    old = C.c_int64()
    rc = load().hpx_get_option(name.encode(), C.byref(old))
    if rc == 0:
        rc = load().hpx_set_option(name.encode(), int(value))
    if rc:
        raise HpxError(rc, last_error())
    return old.value


def profile_query(kernel):
    """(total milliseconds, launches) recorded for `kernel` since the last reset."""
    ms, n = C.c_double(), C.c_int64()
    rc = load().hpx_profile_query(kernel.encode(), C.byref(ms), C.byref(n))
    if rc:
        raise HpxError(rc, last_error())
    return ms.value, n.value
