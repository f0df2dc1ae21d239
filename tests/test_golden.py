"""Regression vectors written by the CPU oracle (tests/golden/make_fixtures.py; `--check` reproduces the committed
file) held against (a) the oracle as it is now and (b) the HIP kernels through the C ABI, bit for bit.  They keep the
two from drifting apart or changing unnoticed; they do NOT pin either to the reference, whose code had no part in
writing them - that is the job of the hand-derived known answers (tests/kat_vectors.py, tests/test_oracle_kat.py,
tests/test_gpu_kat.py) and of the brute-force and closed-form checks in tests/test_oracle_*.py."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_vectors.npz")


def base_values(n):
    # same formula as tests/golden/make_fixtures.py
    return ((np.arange(n, dtype=np.int64) * 7919) % 1000).astype(np.float32) / np.float32(8) - np.float32(60)


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLDEN, allow_pickle=False)


def _eq(a, b, what):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape, (what, a.dtype, b.dtype, a.shape, b.shape)
    assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), what


# ---- (a) the CPU oracle still produces the vectors it wrote --------------------------------------
def test_oracle_tbq_against_golden(gold, oracle_cpu):
    for k in range(int(gold["tbq_count"])):
        g, r, thr = gold[f"tbq_{k}_g"], gold[f"tbq_{k}_r0"].copy(), float(gold[f"tbq_{k}_thr"])
        packed = oracle_cpu.tbq_encode(g, r, thr)
        _eq(packed, gold[f"tbq_{k}_packed"], f"tbq {k} packed"); _eq(r, gold[f"tbq_{k}_r1"], f"tbq {k} residual")
        n = g.size
        _eq(oracle_cpu.tbq_decode(packed, n, thr, base_values(n), 0), gold[f"tbq_{k}_dec_write"], f"tbq {k} write")
        _eq(oracle_cpu.tbq_decode(packed, n, thr, base_values(n), 1), gold[f"tbq_{k}_dec_add"], f"tbq {k} add")
    assert gold["tbq_0_packed"].tolist() == [82, 146, 82]      # the hand-derived known answer


def test_oracle_terngrad_against_golden(gold, oracle_cpu):
    for k in range(int(gold["tgd_count"])):
        x, b = gold[f"tgd_{k}_x"], int(gold[f"tgd_{k}_bits"])
        rc, msg = oracle_cpu.terngrad_encode(x, b, 0, 0)
        assert rc == 0
        _eq(msg, gold[f"tgd_{k}_msg"], f"terngrad det {k} message")
        n = x.size
        _eq(oracle_cpu.terngrad_decode(msg, n, base_values(n), 0)[1], gold[f"tgd_{k}_dec_write"], f"terngrad {k} write")
        _eq(oracle_cpu.terngrad_decode(msg, n, base_values(n), 1)[1], gold[f"tgd_{k}_dec_add"], f"terngrad {k} add")
    assert gold["tgd_0_msg"].tobytes().hex() == "0202cccc4cbdcccc4c3dd87618b61d06"
    for k in range(int(gold["tgr_count"])):
        x, b, seed = gold[f"tgr_{k}_x"], int(gold[f"tgr_{k}_bits"]), int(gold[f"tgr_{k}_seed"])
        rc, msg = oracle_cpu.terngrad_encode(x, b, 1, seed)
        pay = gold[f"tgr_{k}_payload"]
        assert msg[2:6].view(np.float32)[0] == gold[f"tgr_{k}_min"]
        _eq(msg[10:10 + pay.size], pay, f"terngrad random {k} payload")
    assert gold["tgr_0_payload"][:5].tobytes().hex() == "c8b22cb72d"


def test_oracle_graddrop_against_golden(gold, oracle_cpu):
    branches = set()
    for k in range(int(gold["gd_count"])):
        g, r = gold[f"gd_{k}_g"], gold[f"gd_{k}_r0"].copy()
        msg, info = oracle_cpu.gd_encode(g, r, float(gold[f"gd_{k}_sr"]), float(gold[f"gd_{k}_dr"]), int(gold[f"gd_{k}_seed"]))
        _eq(msg, gold[f"gd_{k}_msg"], f"graddrop {k} message"); _eq(r, gold[f"gd_{k}_r1"], f"graddrop {k} residual")
        assert info["candidates"] == int(gold[f"gd_{k}_candidates"])
        branches.add(info["candidates"] > info["kept"])
        n = g.size
        for add, key in ((0, "dec_write"), (1, "dec_add")):
            out = base_values(n)
            assert oracle_cpu.gd_decode(msg, out, add) == 0
            _eq(out, gold[f"gd_{k}_{key}"], f"graddrop {k} {key}")
    assert branches == {True, False}


def test_oracle_lcg_against_golden(gold, oracle_cpu):
    for s, draws, reals in zip(gold["lcg_seeds"], gold["lcg_draws"], gold["lcg_real01"]):
        for k in range(2, 7):     # draw 1 is discarded by srand()
            assert oracle_cpu.lcg_kth(int(s), k) == int(draws[k - 2])
            assert oracle_cpu.u01_from_u32(int(draws[k - 2])) == reals[k - 2]
    assert gold["lcg_draws"][0][:4].tolist() == [3554416254, 2802067423, 3596950572, 229283573]


# ---- (b) the HIP kernels produce the same vectors ---------------------------------------------------
@pytest.mark.gpu
def test_gpu_against_golden(gold, capi):
    import torch
    from gpu_util import Tbq, Terngrad, dev, host, stream_ptr
    tbq, tg = Tbq(capi), Terngrad(capi)
    L = capi.load()
    for k in range(int(gold["tbq_count"])):
        g, r0, thr = gold[f"tbq_{k}_g"], gold[f"tbq_{k}_r0"], float(gold[f"tbq_{k}_thr"])
        n = g.size
        dg, dr = dev(g), dev(r0)
        packed = tbq.encode([dg], [dr], [thr])[0]
        _eq(host(packed), gold[f"tbq_{k}_packed"], f"tbq {k} packed"); _eq(host(dr), gold[f"tbq_{k}_r1"], f"tbq {k} residual")
        for add, key in ((0, "dec_write"), (1, "dec_add")):
            out = dev(base_values(n))
            tbq.decode([packed], [out], [thr], [add])
            _eq(host(out), gold[f"tbq_{k}_{key}"], f"tbq {k} {key}")
    for k in range(int(gold["tgd_count"])):
        x, b = gold[f"tgd_{k}_x"], int(gold[f"tgd_{k}_bits"])
        n = x.size
        msg = tg.encode([dev(x)], [b], [0], [0])[0]
        _eq(host(msg), gold[f"tgd_{k}_msg"], f"terngrad det {k} message")
        for add, key in ((0, "dec_write"), (1, "dec_add")):
            out = dev(base_values(n))
            tg.decode([msg], [out], [add])
            _eq(host(out), gold[f"tgd_{k}_{key}"], f"terngrad {k} {key}")
    for forced in (None, 1):        # the two-launch encode, then the resident encode
        old = capi.set_option("terngrad_resident_min", forced) if forced is not None else None
        try:
            for k in range(int(gold["tgr_count"])):
                x, b, seed = gold[f"tgr_{k}_x"], int(gold[f"tgr_{k}_bits"]), int(gold[f"tgr_{k}_seed"])
                msg = host(tg.encode([dev(x)], [b], [1], [seed])[0])
                pay = gold[f"tgr_{k}_payload"]
                _eq(msg[10:10 + pay.size], pay, f"terngrad random {k} payload (resident_min={forced})")
        finally:
            if old is not None:
                capi.set_option("terngrad_resident_min", old)
    for k in range(int(gold["gd_count"])):
        g, r0 = gold[f"gd_{k}_g"], gold[f"gd_{k}_r0"]
        n = g.size
        sr, dr_ = float(gold[f"gd_{k}_sr"]), float(gold[f"gd_{k}_dr"])
        want = gold[f"gd_{k}_msg"]
        dg, dres = dev(g), dev(r0)
        out = torch.zeros(4 + 8 * int(np.ceil(n * (1 - dr_))), dtype=torch.uint8, device="cuda")
        rc = L.hpx_gd_encode(1, capi.ptr_array([dg.data_ptr()]), capi.i32_array([n]), capi.ptr_array([dres.data_ptr()]),
                             capi.ptr_array([out.data_ptr()]), capi.f64_array([sr]), capi.f64_array([dr_]),
                             capi.u64_array([int(gold[f"gd_{k}_seed"])]), stream_ptr())
        assert rc == 0, capi.last_error()
        torch.cuda.synchronize()
        _eq(host(out)[:want.size], want, f"graddrop {k} message"); _eq(host(dres), gold[f"gd_{k}_r1"], f"graddrop {k} residual")
        for add, key in ((0, "dec_write"), (1, "dec_add")):
            dout = dev(base_values(n))
            rc = L.hpx_gd_decode(1, capi.ptr_array([out.data_ptr()]), capi.i32_array([want.size]), capi.ptr_array([dout.data_ptr()]),
                                 capi.i32_array([n]), capi.i32_array([add]), stream_ptr())
            assert rc == 0, capi.last_error()
            torch.cuda.synchronize()
            _eq(host(dout), gold[f"gd_{k}_{key}"], f"graddrop {k} {key}")
