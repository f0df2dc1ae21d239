"""ctypes binding of liboracle.so, the plain-C oracle (hpx_oracle.c).

Test infrastructure: numpy arrays in, numpy arrays out, one tensor per call.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with gcc (no GPU toolchain involved)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        f32p, u8p, i32p = C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_int32)
        L.orc_lcg_kth.restype = C.c_uint32
        L.orc_lcg_kth.argtypes = [C.c_uint32, C.c_int]
        L.orc_u01_from_u32.restype = C.c_float
        L.orc_u01_from_u32.argtypes = [C.c_uint32]
        L.orc_u01_shortcut_mismatches.restype = C.c_uint64
        L.orc_u01_shortcut_mismatches.argtypes = [C.c_uint32, C.c_uint32]
        L.orc_u01_fp32_mismatches.restype = C.c_uint64
        L.orc_u01_fp32_mismatches.argtypes = [C.c_uint32, C.c_uint32]
        L.orc_tbq_encode.argtypes = [f32p, C.c_int32, f32p, u8p, C.c_float]
        L.orc_tbq_decode.argtypes = [f32p, C.c_int32, u8p, C.c_float, C.c_int]
        L.orc_terngrad_encode.argtypes = [f32p, C.c_int32, u8p, C.c_int32, C.c_uint8, C.c_int32, C.c_uint64]
        L.orc_terngrad_decode.argtypes = [f32p, u8p, C.c_int32, C.c_int]
        L.orc_gd_sizes.argtypes = [C.c_int32, C.c_double, C.c_double, i32p, i32p, i32p]
        L.orc_gd_sizes.restype = None
        L.orc_gd_sample_index.restype = C.c_uint32
        L.orc_gd_sample_index.argtypes = [C.c_uint64, C.c_int32, C.c_int32]
        L.orc_gd_encode.argtypes = [f32p, C.c_int32, f32p, u8p, C.c_double, C.c_double, C.c_uint64, i32p]
        L.orc_gd_decode.argtypes = [u8p, C.c_int32, f32p, C.c_int32, C.c_int]
        L.orc_dgc_encode.argtypes = [f32p, C.c_int32, u8p, C.c_double, C.c_double, C.c_uint64, i32p]
        L.orc_dgc_decode.argtypes = [u8p, C.c_int32, f32p, C.c_int]
        L.orc_ecq_encode.argtypes = [f32p, C.c_int32, f32p, u8p, C.c_double, C.c_double, C.c_int32, C.c_uint64, i32p]
        L.orc_ecq_decode.argtypes = [u8p, f32p, C.c_int32, C.c_int]
        L.orc_set_fused_multiply_add.argtypes = [C.c_int]
        L.orc_set_fused_multiply_add.restype = None
        L.orc_max_threads.restype = C.c_int
        L.orc_set_threads.argtypes = [C.c_int]
        L.orc_set_threads.restype = None
        _lib = L
    return _lib


def _f32(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u8(a):
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def set_fused_multiply_add(on):
    """Lets the TernGrad oracle fuse `(x - min) * gi + u` and `q * gap + min` as a CUDA build of the reference
    may (for measuring that difference only; parity is held to the unfused CPU arithmetic)."""
    lib().orc_set_fused_multiply_add(int(bool(on)))


def set_threads(n):
    lib().orc_set_threads(int(n))


def max_threads():
    return lib().orc_max_threads()


# ---- LCG -------------------------------------------------------------------
def lcg_kth(seed, k):
    return lib().orc_lcg_kth(seed & 0xFFFFFFFF, k)


def u01_from_u32(x):
    return np.float32(lib().orc_u01_from_u32(x & 0xFFFFFFFF))


def u01_shortcut_mismatches(lo, hi):
    return int(lib().orc_u01_shortcut_mismatches(lo, hi))


def u01_fp32_mismatches(lo, hi):
    return int(lib().orc_u01_fp32_mismatches(lo, hi))


# ---- TBQ -------------------------------------------------------------------
def tbq_packed_size(n):
    return (n + 3) // 4


def tbq_encode(g, r, thr):
    """Returns packed bytes; `r` (residual) is updated in place, `g` untouched."""
    n = g.size
    out = np.full(tbq_packed_size(n), 0xAA, np.uint8)
    rc = lib().orc_tbq_encode(_f32(g), n, _f32(r), _u8(out), np.float32(thr))
    assert rc == 0
    return out


def tbq_decode(packed, n, thr, out=None, is_add_to=0):
    if out is None:
        out = np.zeros(n, np.float32)
    rc = lib().orc_tbq_decode(_f32(out), n, _u8(packed), np.float32(thr), int(is_add_to))
    assert rc == 0
    return out


# ---- TernGrad --------------------------------------------------------------
def terngrad_packed_size(n, bitwidth=2):
    dpb = 8 // bitwidth
    return 10 + (n + dpb - 1) // dpb


def terngrad_encode(x, bitwidth=2, enable_random=1, seed=0, out_size=None):
    n = x.size
    if out_size is None:
        out_size = terngrad_packed_size(n, bitwidth) if bitwidth in (1, 2, 4, 8) else 10 + n
    out = np.zeros(out_size, np.uint8)
    rc = lib().orc_terngrad_encode(_f32(x), n, _u8(out), out_size, bitwidth, int(enable_random), seed)
    return rc, out


def terngrad_decode(packed, n, out=None, is_add_to=0):
    if out is None:
        out = np.zeros(n, np.float32)
    rc = lib().orc_terngrad_decode(_f32(out), _u8(packed), packed.size, int(is_add_to))
    return rc, out


# ---- GradDrop / DGC --------------------------------------------------------
def gd_sizes(n, sample_rate, drop_ratio):
    a, b, c = C.c_int32(), C.c_int32(), C.c_int32()
    lib().orc_gd_sizes(n, sample_rate, drop_ratio, C.byref(a), C.byref(b), C.byref(c))
    return a.value, b.value, c.value  # sample_cnt, expected, thr_index


def gd_sample_index(seed, x, n):
    return lib().orc_gd_sample_index(seed, x, n)


def gd_encode(g, r, sample_rate, drop_ratio, seed=0):
    """Returns (message bytes trimmed to 4+8k, info dict). `r` updated in place."""
    n = g.size
    out = np.zeros(4 + 8 * n, np.uint8)
    info = (C.c_int32 * 3)()
    rc = lib().orc_gd_encode(_f32(g), n, _f32(r), _u8(out), sample_rate, drop_ratio, seed, info)
    assert rc == 0
    m = int(out[:4].view(np.int32)[0])
    thr = np.array([info[2]], np.int32).view(np.float32)[0]
    return out[:m].copy(), {"candidates": info[0], "kept": info[1], "threshold": thr}


def gd_split(msg):
    """(indices int32[k], values float32[k]) of a GradDrop message."""
    m = int(msg[:4].view(np.int32)[0])
    k = (m - 4) // 8
    idx = msg[4:4 + 4 * k].view(np.int32)
    val = msg[4 + 4 * k:4 + 8 * k].view(np.float32)
    return idx, val


def gd_decode(msg, out, is_add_to=0, in_size=None):
    rc = lib().orc_gd_decode(_u8(msg), msg.size if in_size is None else in_size, _f32(out), out.size, int(is_add_to))
    return rc


# ---- DGC without residual (dgc_body.h) ---------------------------------------
def dgc_encode(g, sample_rate, s_percent, seed=0):
    """Returns (message bytes trimmed to 4+8k, info dict). `g` is updated in place (selected entries -> 0)."""
    n = g.size
    out = np.zeros(4 + 8 * n, np.uint8)
    info = (C.c_int32 * 3)()
    rc = lib().orc_dgc_encode(_f32(g), n, _u8(out), sample_rate, s_percent, seed, info)
    assert rc == 0
    m = int(out[:4].view(np.int32)[0])
    thr = np.array([info[2]], np.int32).view(np.float32)[0]
    return out[:m].copy(), {"candidates": info[0], "kept": info[1], "threshold": thr}


def dgc_decode(msg, out, is_add_to=0, in_size=None):
    return lib().orc_dgc_decode(_u8(msg), msg.size if in_size is None else in_size, _f32(out), int(is_add_to))


# ---- ECQ (ecq_body.h), the reference's serial-policy behaviour ------------------
def ecq_packed_size(n, bitwidth):
    dpb = 8 // bitwidth
    return 10 + (n + dpb - 1) // dpb


def ecq_encode(g, h, alpha, beta, bitwidth, seed=0):
    """Returns (rc, message of 10 + M bytes, last_byte_defined).  `h` (the history) is updated in place.
    When last_byte_defined is False the last payload byte is not part of the result (the reference leaves
    whatever the caller's buffer held there)."""
    n = g.size
    if bitwidth not in (2, 4, 8):
        work = np.zeros(16, np.uint8)
        defined = C.c_int32()
        return lib().orc_ecq_encode(_f32(g), n, _f32(h), _u8(work), alpha, beta, bitwidth, seed, C.byref(defined)), None, False
    m = ecq_packed_size(n, bitwidth)
    work = np.zeros(max(4 * n, m) + 16, np.uint8)
    defined = C.c_int32()
    rc = lib().orc_ecq_encode(_f32(g), n, _f32(h), _u8(work), alpha, beta, bitwidth, seed, C.byref(defined))
    return rc, work[:m].copy(), bool(defined.value)


def ecq_decode(msg, out, is_add_to=0):
    return lib().orc_ecq_decode(_u8(msg), _f32(out), out.size, int(is_add_to))
