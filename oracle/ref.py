"""ctypes binding of _ref/libhpref.so: the reference's own header bodies
compiled for the host (ref_harness.cpp).  Optional test infrastructure: it
exists only where `make -C oracle ref` ran against a reference checkout.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_ref", "libhpref.so")
REFERENCE_DIR = "/root/reference"


def available():
    return os.path.exists(_SO)


def build():
    """Build from the reference checkout if it is present; returns availability."""
    if os.path.isdir(REFERENCE_DIR):
        subprocess.check_call(["make", "-C", _HERE, "-B", "ref"])
    return available()


_lib = None


def lib():
    global _lib
    if _lib is None:
        L = C.CDLL(_SO)
        f32p, u8p, i32p = C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_int32)
        L.ref_tbq_encode.argtypes = [f32p, C.c_int32, f32p, u8p, C.c_float, C.c_int]
        L.ref_tbq_decode.argtypes = [f32p, C.c_int32, u8p, C.c_float, C.c_int, C.c_int]
        L.ref_terngrad_encode.argtypes = [f32p, C.c_int32, u8p, C.c_int32, C.c_uint8, C.c_int32, C.c_int]
        L.ref_terngrad_payload_random.argtypes = [f32p, C.c_int32, u8p, C.c_uint8, C.c_uint8, C.c_float, C.c_float, C.c_ulonglong, C.c_int]
        L.ref_terngrad_decode.argtypes = [f32p, C.c_int32, u8p, C.c_int32, C.c_int, C.c_int]
        L.ref_gd_encode.argtypes = [f32p, C.c_int32, f32p, u8p, C.c_double, C.c_double, C.c_int]
        L.ref_gd_sample.argtypes = [f32p, f32p, C.c_int32, C.c_int32, C.c_ulonglong]
        L.ref_gd_encode_seeded.argtypes = [f32p, C.c_int32, f32p, u8p, C.c_double, C.c_double, C.c_ulonglong, i32p, C.c_int]
        L.ref_gd_decode.argtypes = [u8p, C.c_int32, f32p, C.c_int32, C.c_int, C.c_int]
        L.ref_lcg_kth.restype = C.c_uint32
        L.ref_lcg_kth.argtypes = [C.c_uint32, C.c_int]
        L.ref_real01.restype = C.c_float
        L.ref_real01.argtypes = [C.c_uint32, C.c_int]
        _lib = L
    return _lib


def _f32(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u8(a):
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def tbq_encode(g, r, thr, policy=0):
    out = np.full((g.size + 3) // 4, 0xAA, np.uint8)
    assert lib().ref_tbq_encode(_f32(g), g.size, _f32(r), _u8(out), np.float32(thr), policy) == 0
    return out


def tbq_decode(packed, n, thr, out=None, is_add_to=0, policy=0):
    if out is None:
        out = np.zeros(n, np.float32)
    assert lib().ref_tbq_decode(_f32(out), n, _u8(packed), np.float32(thr), int(is_add_to), policy) == 0
    return out


def terngrad_encode_det(x, bitwidth=2, policy=0, out_size=None):
    dpb = 8 // bitwidth
    if out_size is None:
        out_size = 10 + (x.size + dpb - 1) // dpb
    out = np.zeros(out_size, np.uint8)
    rc = lib().ref_terngrad_encode(_f32(x), x.size, _u8(out), out_size, bitwidth, 0, policy)
    return rc, out


def terngrad_payload_random(x, nbytes, bitwidth, mn, gi, seed, policy=0):
    lg2 = {1: 3, 2: 2, 4: 1, 8: 0}[bitwidth]
    pay = np.zeros(nbytes, np.uint8)
    lib().ref_terngrad_payload_random(_f32(x), nbytes, _u8(pay), bitwidth, lg2, np.float32(mn), np.float32(gi), seed, policy)
    return pay


def terngrad_decode(packed, n, out=None, is_add_to=0, policy=0):
    if out is None:
        out = np.zeros(n, np.float32)
    rc = lib().ref_terngrad_decode(_f32(out), n, _u8(packed), packed.size, int(is_add_to), policy)
    return rc, out


def gd_encode_seeded(g, r, sample_rate, drop_ratio, seed, policy=0):
    n = g.size
    sample_cnt = int(np.ceil(n * sample_rate))
    out = np.zeros(max(4 * sample_cnt, 4 + 8 * n) + 16, np.uint8)
    info = (C.c_int32 * 3)()
    rc = lib().ref_gd_encode_seeded(_f32(g), n, _f32(r), _u8(out), sample_rate, drop_ratio, seed, info, policy)
    assert rc == 0
    m = int(out[:4].view(np.int32)[0])
    thr = np.array([info[2]], np.int32).view(np.float32)[0]
    return out[:m].copy(), {"candidates": info[0], "kept": info[1], "threshold": thr}


def gd_encode_clock(g, r, sample_rate, drop_ratio, policy=0):
    n = g.size
    sample_cnt = int(np.ceil(n * sample_rate))
    out = np.zeros(max(4 * sample_cnt, 4 + 8 * n) + 16, np.uint8)
    rc = lib().ref_gd_encode(_f32(g), n, _f32(r), _u8(out), sample_rate, drop_ratio, policy)
    assert rc == 0
    m = int(out[:4].view(np.int32)[0])
    return out[:m].copy()


def gd_sample(r, sample_cnt, seed):
    s = np.zeros(sample_cnt, np.float32)
    lib().ref_gd_sample(_f32(s), _f32(r), r.size, sample_cnt, seed)
    return s


def gd_decode(msg, out, is_add_to=0, in_size=None, policy=0):
    return lib().ref_gd_decode(_u8(msg), msg.size if in_size is None else in_size, _f32(out), out.size, int(is_add_to), policy)


def lcg_kth(seed, k):
    return lib().ref_lcg_kth(seed & 0xFFFFFFFF, k)


def real01(seed, k):
    return np.float32(lib().ref_real01(seed & 0xFFFFFFFF, k))
