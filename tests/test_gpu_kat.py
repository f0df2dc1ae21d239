"""The HIP kernels against the hand-derived known answers of tests/kat_vectors.py, through the C ABI: the same
literals the CPU oracle is held to, so the GPU path is pinned to the reference's source text directly and not
only through the oracle."""
import numpy as np
import pytest
import torch

import kat_vectors as kat
from gpu_util import Tbq, Terngrad, assert_bits_equal, dev, host, stream_ptr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("route", ["tiled", "resident", "bucket", "noalloc"])
@pytest.mark.parametrize("name", sorted(kat.TERNGRAD_CASES))
def test_terngrad_known_messages(capi, name, route):
    tg = Terngrad(capi)
    case = kat.TERNGRAD_CASES[name]
    dx = dev(case["x"])
    want = np.frombuffer(case["message"], np.uint8)
    old = [capi.set_option("terngrad_resident_min", -1 if route == "tiled" else 1),
           capi.set_option("terngrad_resident_bucket", 1 if route == "bucket" else 0)]
    try:
        if route == "noalloc":
            out = tg.encode_noalloc([dx], [case["bits"]], [case["random"]], [case["seed"]])[0]
        elif route == "bucket":            # the same tensor twice in one call: one launch for both
            outs = tg.encode([dx, dx], [case["bits"]] * 2, [case["random"]] * 2, [case["seed"]] * 2)
            assert_bits_equal(host(outs[1]), want, f"case {name}, second tensor of the bucket")
            out = outs[0]
        else:
            out = tg.encode([dx], [case["bits"]], [case["random"]], [case["seed"]])[0]
        assert tg.encode_status() == 0
        torch.cuda.synchronize()
    finally:
        capi.set_option("terngrad_resident_min", old[0])
        capi.set_option("terngrad_resident_bucket", old[1])
    assert_bits_equal(host(out), want, f"case {name} through the {route} encode")


def test_terngrad_known_decode(capi):
    tg = Terngrad(capi)
    msg = dev(np.frombuffer(kat.TG_A["message"], np.uint8).copy())
    out = torch.full((8,), 9.0, device="cuda")
    tg.decode([msg], [out], [0])
    acc = torch.full((8,), 0.5, device="cuda")
    tg.decode([msg], [acc], [1])
    torch.cuda.synchronize()
    assert_bits_equal(host(out), kat.TG_A_DECODED, "write mode")
    assert_bits_equal(host(acc), kat.TG_A_DECODED + np.float32(0.5), "add mode")


@pytest.mark.parametrize("name", sorted(kat.GRADDROP_CASES))
def test_graddrop_known_messages(capi, name):
    c, L = capi, capi.load()
    case = kat.GRADDROP_CASES[name]
    dg, dr = dev(case["g"]), dev(case["r0"])
    want = kat.gd_message(case)
    out = torch.full((4 + 8 * 4 + 16,), 0xEE, dtype=torch.uint8, device="cuda")
    rc = L.hpx_gd_encode(1, c.ptr_array([dg.data_ptr()]), c.i32_array([16]), c.ptr_array([dr.data_ptr()]),
                         c.ptr_array([out.data_ptr()]), c.f64_array([case["sample_rate"]]), c.f64_array([case["drop_ratio"]]),
                         c.u64_array([case["seed"]]), stream_ptr())
    assert rc == 0, c.last_error()
    torch.cuda.synchronize()
    got = host(out)
    assert_bits_equal(got[:want.size], want, f"case {name}: message")
    assert (got[want.size:] == 0xEE).all(), "bytes past the message are untouched"
    assert_bits_equal(host(dr), case["r1"], f"case {name}: residual")
    assert_bits_equal(host(dg), case["g"], f"case {name}: gradient is read-only")
    dec = torch.full((16,), 7.0, device="cuda")
    rc = L.hpx_gd_decode(1, c.ptr_array([out.data_ptr()]), c.i32_array([want.size]), c.ptr_array([dec.data_ptr()]),
                         c.i32_array([16]), c.i32_array([0]), stream_ptr())
    assert rc == 0, c.last_error()
    torch.cuda.synchronize()
    ref = np.zeros(16, np.float32); ref[case["idx"]] = case["val"]
    assert_bits_equal(host(dec), ref, f"case {name}: decode")


def test_tbq_known_bytes(capi):
    tbq = Tbq(capi)
    c = kat.TBQ_A
    dg, dr = dev(c["g"]), torch.zeros(10, device="cuda")
    packed = tbq.encode([dg], [dr], [c["thr"]])[0]
    out = torch.full((10,), 5.0, device="cuda")
    tbq.decode([packed], [out], [c["thr"]], [0])
    torch.cuda.synchronize()
    assert host(packed).tobytes() == c["packed"]
    assert_bits_equal(host(dr), c["r1"], "residual")
    assert_bits_equal(host(out), c["decoded"], "decoded")
