"""GPU parity of the ECQ codec (hpx_ecq_encode / hpx_ecq_decode) with the CPU oracle, through the C ABI: message
bytes, history after encode, decoded tensors, bit for bit (a NaN matches a NaN: with 8-bit codes the reference's
own scratch aliasing can manufacture one in elements 2 and 3, and NaN payloads differ between machines)."""
import numpy as np
import pytest
import torch

from gpu_util import assert_bits_equal, dev, host, stream_ptr
from test_oracle_ecq import ECQ_DECODED, ECQ_G, ECQ_H1, ECQ_LONG, ECQ_MSG, _same_floats

pytestmark = pytest.mark.gpu


class Ecq:
    def __init__(self, capi):
        self.c, self.L = capi, capi.load()

    def encode(self, gs, hs, outs, alphas, betas, bits, seeds, expect_rc=0):
        c = self.c
        rc = self.L.hpx_ecq_encode(len(gs), c.ptr_array([g.data_ptr() for g in gs]), c.i32_array([g.numel() for g in gs]),
                                   c.ptr_array([h.data_ptr() for h in hs]), c.ptr_array([o.data_ptr() for o in outs]),
                                   c.i32_array([o.numel() for o in outs]), c.f64_array(alphas), c.f64_array(betas),
                                   c.i32_array(bits), c.u64_array(seeds) if seeds is not None else None, stream_ptr())
        assert rc == expect_rc, (rc, c.last_error())

    def decode(self, msgs, outs, adds, expect_rc=0):
        c = self.c
        rc = self.L.hpx_ecq_decode(len(msgs), c.ptr_array([m.data_ptr() for m in msgs]), c.i32_array([m.numel() for m in msgs]),
                                   c.ptr_array([o.data_ptr() for o in outs]), c.i32_array([o.numel() for o in outs]),
                                   c.i32_array(adds), stream_ptr())
        assert rc == expect_rc, (rc, c.last_error())


@pytest.fixture(scope="module")
def ecq(capi):
    return Ecq(capi)


def test_hand_derived_message(ecq):
    dg, dh = dev(ECQ_G), torch.zeros(8, device="cuda")
    out = torch.full((12,), 0xEE, dtype=torch.uint8, device="cuda")
    ecq.encode([dg], [dh], [out], [1.0], [0.5], [2], [0])
    dec = torch.full((8,), 9.0, device="cuda")
    ecq.decode([out], [dec], [0])
    torch.cuda.synchronize()
    assert host(out).tobytes() == ECQ_MSG, host(out).tobytes().hex()
    assert_bits_equal(host(dh), ECQ_H1, "history")
    assert_bits_equal(host(dec), ECQ_DECODED, "decoded")


@pytest.mark.parametrize("bitwidth,G,want,h_want", ECQ_LONG, ids=["8bit", "4bit"])
def test_hand_derived_messages_that_reread_the_scratch(ecq, bitwidth, G, want, h_want):
    dg, dh = dev(G), torch.zeros(G.size, device="cuda")
    out = torch.full((len(want),), 0xEE, dtype=torch.uint8, device="cuda")
    ecq.encode([dg], [dh], [out], [1.0], [0.5], [bitwidth], [0])
    torch.cuda.synchronize()
    assert host(out).tobytes() == want, host(out).tobytes().hex()
    assert_bits_equal(host(dh), h_want, "history")


@pytest.mark.parametrize("bitwidth", [2, 4, 8])
def test_sizes_seeds_and_parameters(ecq, oracle_cpu, bitwidth):
    rng = np.random.default_rng(300 + bitwidth)
    sizes = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 33, 100, 1023, 1024, 1025, 4099, 70_001, 1_000_003]
    gs, hs, als, bes, seeds = [], [], [], [], []
    for n in sizes:
        gs.append(rng.normal(0, 1e-2, n).astype(np.float32))
        hs.append(rng.normal(0, 5e-3, n).astype(np.float32))
        als.append(float(rng.choice([0.0, 0.5, 1.0])))
        bes.append(float(rng.choice([0.0, 0.9, 1.0])))
        seeds.append(int(rng.integers(0, 2**63)))
    dgs, dhs = [dev(g) for g in gs], [dev(h) for h in hs]
    outs = [torch.full((oracle_cpu.ecq_packed_size(n, bitwidth) + 8,), 0xEE, dtype=torch.uint8, device="cuda") for n in sizes]
    ecq.encode(dgs, dhs, outs, als, bes, [bitwidth] * len(sizes), seeds)      # all tensors in one call
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        h_ref = hs[i].copy()
        rc, msg, defined = oracle_cpu.ecq_encode(gs[i], h_ref, als[i], bes[i], bitwidth, seeds[i])
        got = host(outs[i])
        upto = msg.size if defined else msg.size - 1
        assert_bits_equal(got[:upto], msg[:upto], f"message n={n} b={bitwidth}")
        if not defined:
            assert got[msg.size - 1] == 0xEE, "the last byte is the caller's when 9 + M >= 4 N"
        assert (got[msg.size:] == 0xEE).all(), f"n={n}: wrote past the message"
        assert _same_floats(host(dhs[i]), h_ref), f"history n={n} b={bitwidth}"
        assert_bits_equal(host(dgs[i]), gs[i], "gradient untouched")
        # decode, write and add
        full = msg.copy()
        full[:upto] = got[:upto]
        full[upto:] = got[upto:msg.size]
        for add in (0, 1):
            base = rng.normal(0, 1, n).astype(np.float32)
            dout = dev(base)
            ecq.decode([outs[i][:msg.size]], [dout], [add])
            torch.cuda.synchronize()
            want = base.copy()
            assert oracle_cpu.ecq_decode(full, want, add) == 0
            assert_bits_equal(host(dout), want, f"decode add={add} n={n} b={bitwidth}")


def test_zero_input_and_errors(ecq, oracle_cpu, capi):
    n = 5000
    G = np.full(n, 1e-8, np.float32)
    H0 = np.full(n, 2e-8, np.float32)
    dg, dh = dev(G), dev(H0)
    out = torch.full((oracle_cpu.ecq_packed_size(n, 2),), 0xEE, dtype=torch.uint8, device="cuda")
    ecq.encode([dg], [dh], [out], [1.0], [0.5], [2], [3])
    torch.cuda.synchronize()
    h_ref = H0.copy()
    rc, msg, defined = oracle_cpu.ecq_encode(G, h_ref, 1.0, 0.5, 2, 3)
    assert defined
    assert_bits_equal(host(out), msg, "message of an all-tiny tensor")
    assert_bits_equal(host(dh), h_ref, "history *= beta")
    ecq.encode([dg], [dh], [out], [1.0], [0.5], [3], [0], expect_rc=-1)             # width not 2, 4, 8
    ecq.encode([dg], [dh], [out[:-1]], [1.0], [0.5], [2], [0], expect_rc=-3)        # output too small
    small = torch.zeros(n - 1, device="cuda")
    ecq.decode([out], [small], [0], expect_rc=-1)                                   # output smaller than the message says
    assert "too small" in capi.last_error()
