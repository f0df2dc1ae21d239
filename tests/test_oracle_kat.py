"""The CPU oracle against known answers derived by hand from the reference's source text (tests/kat_vectors.py).
These pins do not depend on any build of the reference: every expected value is a literal whose derivation is
written next to it."""
import numpy as np
import pytest

import kat_vectors as kat


def test_the_derivations_own_arithmetic():
    # the literals the derivations quote, re-derived with Python integers (no code under test involved)
    assert kat.lcg_draws(0, 5) == [12345, 3554416254, 2802067423, 3596950572, 229283573]   # textbook ANSI-C rand()
    a2 = kat.LCG_A * kat.LCG_A % kat.M32
    c2 = (kat.LCG_A * kat.LCG_C + kat.LCG_C) % kat.M32
    assert (a2, c2) == (3265436265, 3554416254) and (a2 % 16, c2 % 16) == (9, 14)
    assert [(9 * k + 14) % 16 for k in range(16)] == kat.GD_SAMPLE_INDEX_SEED0
    assert sorted(kat.GD_SAMPLE_INDEX_SEED0) == list(range(16))
    for case in kat.TERNGRAD_CASES.values():
        if "draws_byte0" in case:
            assert kat.lcg_draws(case["seed"], 5) == case["draws_byte0"]
        if "draws_byte1" in case:
            assert kat.lcg_draws(case["seed"] + 1, 5) == case["draws_byte1"]
    assert pow(a2, -1, kat.M32) * ((0xFFFFFFFF - c2) % kat.M32) % kat.M32 == kat.TG_C1["seed"]
    assert pow(a2, -1, kat.M32) * ((0xFFFFFF7F - c2) % kat.M32) % kat.M32 == kat.TG_D["seed"]
    for seed in (kat.TG_C1["seed"], kat.TG_D["seed"]):        # byte 1 of cases C and D: no draw reaches u = 1
        assert all(d < kat.M32 - 128 for d in kat.lcg_draws(seed + 1, 5)[1:])


def test_lcg_and_uniform_known_answers(oracle_cpu):
    for k, want in enumerate(kat.lcg_draws(0, 5), start=1):
        assert oracle_cpu.lcg_kth(0, k) == want
    for x, want in kat.U01_KNOWN:
        got = oracle_cpu.u01_from_u32(x)
        assert got == np.float32(want) and np.float32(want) == want, (hex(x), got, want)


@pytest.mark.parametrize("name", sorted(kat.TERNGRAD_CASES))
def test_terngrad_known_messages(oracle_cpu, name):
    case = kat.TERNGRAD_CASES[name]
    rc, msg = oracle_cpu.terngrad_encode(case["x"].copy(), case["bits"], case["random"], case["seed"])
    assert rc == 0
    assert msg.tobytes() == case["message"], (name, msg.tobytes().hex(), case["message"].hex())


def test_terngrad_known_decode(oracle_cpu):
    msg = np.frombuffer(kat.TG_A["message"], np.uint8).copy()
    rc, out = oracle_cpu.terngrad_decode(msg, 8)
    assert rc == 0 and np.array_equal(out, kat.TG_A_DECODED)
    base = np.full(8, 0.5, np.float32)
    rc, out = oracle_cpu.terngrad_decode(msg, 8, base, 1)
    assert rc == 0 and np.array_equal(out, kat.TG_A_DECODED + np.float32(0.5))


@pytest.mark.parametrize("name", sorted(kat.GRADDROP_CASES))
def test_graddrop_known_messages(oracle_cpu, name):
    case = kat.GRADDROP_CASES[name]
    r = case["r0"].copy()
    g = case["g"].copy()
    msg, info = oracle_cpu.gd_encode(g, r, case["sample_rate"], case["drop_ratio"], case["seed"])
    assert info["threshold"] == np.float32(case["threshold"]), info
    assert np.array_equal(msg, kat.gd_message(case)), (name, oracle_cpu.gd_split(msg))
    assert np.array_equal(r.view(np.uint32), case["r1"].view(np.uint32))
    assert np.array_equal(g, case["g"])                       # the gradient is read-only
    # decode: write mode clears and scatters; add mode accumulates (gd_body.h:283-353)
    out = np.full(16, 7.0, np.float32)
    assert oracle_cpu.gd_decode(msg, out, 0) == 0
    want = np.zeros(16, np.float32); want[case["idx"]] = case["val"]
    assert np.array_equal(out, want)
    out = np.full(16, 1.0, np.float32)
    assert oracle_cpu.gd_decode(msg, out, 1) == 0
    assert np.array_equal(out, want + np.float32(1.0))


def test_graddrop_sample_index_stream(oracle_cpu):
    assert [oracle_cpu.gd_sample_index(0, k, 16) for k in range(16)] == kat.GD_SAMPLE_INDEX_SEED0


def test_tbq_known_bytes(oracle_cpu):
    c = kat.TBQ_A
    r = np.zeros(10, np.float32)
    packed = oracle_cpu.tbq_encode(c["g"].copy(), r, c["thr"])
    assert packed.tobytes() == c["packed"] and np.array_equal(r, c["r1"])
    assert np.array_equal(oracle_cpu.tbq_decode(packed, 10, c["thr"]), c["decoded"])
