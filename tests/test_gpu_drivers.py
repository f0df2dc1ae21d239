"""GPU parity through the nine kernel-driver functions with the reference's own C++ signatures
(hp_cuda.cpp:18-102): the vector-based drivers exported by libhpx.so and the three PowerSGD drivers over
torch tensors, reached through the compiled module `hp_cuda_drivers`, which builds their argument vectors
from lists of tensors the way the reference's scheduler loops do.

TBQ, the decoders and TernGrad without random rounding are compared with the CPU oracle bit for bit.
The drivers take the RNG seed from the clock (as the reference bodies do), so the stochastic TernGrad
encode and the GradDrop encode are checked through what holds for every seed.
"""
import numpy as np
import pytest
import torch

from gpu_util import assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def drv(hp_cuda_compiled):
    import importlib
    return importlib.import_module("hp_cuda_drivers")     # same directory as the hp_cuda module


def test_tbq_drivers(drv, oracle_cpu):
    rng = np.random.default_rng(3)
    ns, thrs = [10, 4099, 300_001], [2e-3, 1e-3, 5e-3]
    gs = [rng.normal(0, 2e-3, n).astype(np.float32) for n in ns]
    rs = [rng.normal(0, 1e-3, n).astype(np.float32) for n in ns]
    dg, dr = [dev(g) for g in gs], [dev(r) for r in rs]
    outs = [torch.full(((n + 3) // 4,), 0xAA, dtype=torch.uint8, device="cuda") for n in ns]
    drv.hp_cuda_tbq(dg, dr, outs, thrs)                    # synchronous, like the reference driver
    bases = [rng.normal(0, 1, n).astype(np.float32) for n in ns]
    dec = [dev(b) for b in bases]
    adds = [0, 1, 0]
    drv.hp_cuda_tbqr(dec, outs, thrs, adds)
    for i, n in enumerate(ns):
        r_ref = rs[i].copy()
        p_ref = oracle_cpu.tbq_encode(gs[i], r_ref, thrs[i])
        assert_bits_equal(host(outs[i]), p_ref, f"packed[{i}]")
        assert_bits_equal(host(dr[i]), r_ref, f"residual[{i}]")
        assert_bits_equal(host(dec[i]), oracle_cpu.tbq_decode(p_ref, n, thrs[i], bases[i].copy(), adds[i]), f"decoded[{i}]")


def test_terngrad_drivers(drv, oracle_cpu):
    rng = np.random.default_rng(4)
    ns, bits = [22, 100_003, 3_000_001], [2, 4, 2]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in ns]
    dx = [dev(x) for x in xs]
    msgs = [torch.zeros(oracle_cpu.terngrad_packed_size(n, b), dtype=torch.uint8, device="cuda") for n, b in zip(ns, bits)]
    drv.hp_cuda_terngrad(dx, msgs, bits, [0, 0, 0])        # round to nearest: reproducible
    outs = [torch.zeros(n, device="cuda") for n in ns]
    drv.hp_cuda_terngradr(outs, msgs, [0, 0, 0])
    torch.cuda.synchronize()
    for i, n in enumerate(ns):
        rc, ref = oracle_cpu.terngrad_encode(xs[i], bits[i], 0, 0)
        assert rc == 0
        assert_bits_equal(host(msgs[i]), ref, f"message[{i}]")
        assert_bits_equal(host(outs[i]), oracle_cpu.terngrad_decode(ref, n)[1], f"decoded[{i}]")
    # stochastic rounding, seed from the clock: header exact, every element within one level of its input
    drv.hp_cuda_terngrad(dx, msgs, bits, [1, 1, 1])
    drv.hp_cuda_terngradr(outs, msgs, [0, 0, 0])
    torch.cuda.synchronize()
    for i, n in enumerate(ns):
        head = host(msgs[i][:10])
        mn, mx = head[2:6].view(np.float32)[0], head[6:10].view(np.float32)[0]
        assert head[0] == bits[i] and mn == xs[i].min() and mx == xs[i].max()
        gap = (mx - mn) / ((1 << bits[i]) - 1)
        assert float(np.abs(host(outs[i]) - xs[i]).max()) <= gap * 1.001 + 1e-7


def test_terngrad_driver_returns_a_valid_message_when_the_barrier_expires(drv, oracle_cpu, capi):
    # The reference's hp_cuda_terngrad never returns with an invalid message (hp_cuda_kernel.cu:30-65).  Here only
    # the single-launch encode, which waits at a grid barrier, can fail to write one; its bound is set to zero
    # from the host, so every workgroup gives up and leaves normally, and the driver must still hand back the
    # message of THIS call (it asks hpx_terngrad_encode_status, which encodes again through the other kernels).
    rng = np.random.default_rng(40)
    n = 3_000_001
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    rc, ref = oracle_cpu.terngrad_encode(x, 2, 0, 0)       # round to nearest: the driver takes its seed from the clock
    L = capi.load()
    torch.cuda.synchronize()
    assert L.hpx_release_workspaces() == 0                  # this stream becomes the owner of the barrier kernels
    old = [capi.set_option("terngrad_resident_min", 1 << 21), capi.set_option("terngrad_resident_bucket", 0),
           capi.set_option("terngrad_barrier_ms", 0)]
    try:
        dx = dev(x)
        msg = torch.full((ref.size,), 0x5A, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        drv.hp_cuda_terngrad([dx], [msg], [2], [0])
        assert L.hpx_terngrad_repaired(torch.cuda.current_stream().cuda_stream) == 1   # the barrier did expire
        assert_bits_equal(host(msg), ref, "message of the call whose barrier expired")
    finally:
        for name, v in zip(("terngrad_resident_min", "terngrad_resident_bucket", "terngrad_barrier_ms"), old):
            capi.set_option(name, v)
        torch.cuda.synchronize()
        assert L.hpx_release_workspaces() == 0


def test_graddrop_drivers(drv, oracle_cpu):
    rng = np.random.default_rng(5)
    n, sr, dr_ = 500_009, 0.02, 0.99
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    r0 = rng.normal(0, 1e-4, n).astype(np.float32)
    dg, dres = dev(g), dev(r0)
    _, expected, _ = oracle_cpu.gd_sizes(n, sr, dr_)
    out = torch.zeros(4 + 8 * expected, dtype=torch.uint8, device="cuda")
    drv.hp_cuda_gd([dg], [dres], [out], [sr], [dr_])       # seed from the clock (gd_body.h:138-140)
    torch.cuda.synchronize()
    msg = host(out)
    m = int(msg[:4].view(np.int32)[0])
    k = (m - 4) // 8
    assert 0 < k <= expected and m == 4 + 8 * k
    idx, val = oracle_cpu.gd_split(msg[:m])
    total = g + r0                                           # what R += G stores (fp32 add, same on both sides)
    assert np.unique(idx).size == k
    assert_bits_equal(val, total[idx], "values are the accumulated entries")
    want_r = total.copy(); want_r[idx] = 0
    assert_bits_equal(host(dres), want_r, "residual: accumulated, selected entries cleared")
    assert_bits_equal(host(dg), g, "gradient untouched")
    # every entry left behind is no larger than every entry taken (threshold, then cut to the largest)
    assert np.abs(want_r).max() <= np.abs(val).min()
    # decode: write mode clears and scatters, add mode accumulates
    dec = dev(rng.normal(0, 1, n).astype(np.float32))
    drv.hp_cuda_gdr([out], [m], [dec], [0])
    torch.cuda.synchronize()
    want = np.zeros(n, np.float32); want[idx] = val
    assert_bits_equal(host(dec), want, "decode, write mode")
    drv.hp_cuda_gdr([out], [m], [dres], [1])
    torch.cuda.synchronize()
    assert_bits_equal(host(dres), total, "decode(add) into the residual restores R + G")


def test_powersgd_drivers_equal_the_c_abi_path(drv, pkg):
    gen = torch.Generator(device="cuda").manual_seed(6)
    shapes, rk = [(256, 192), (130, 515), (1024, 64)], 4
    def fresh():
        g = torch.Generator(device="cuda").manual_seed(6)
        G = [torch.randn(a * b, device="cuda", generator=g) * 1e-2 for a, b in shapes]
        R = [torch.randn(a * b, device="cuda", generator=g) * 1e-3 for a, b in shapes]
        Q = [torch.randn(b, rk, device="cuda", generator=g) for a, b in shapes]
        M = [torch.zeros(a, b, device="cuda") for a, b in shapes]
        P = [torch.zeros(a, rk, device="cuda") for a, b in shapes]
        return G, R, Q, M, P
    G1, R1, Q1, M1, P1 = fresh()
    drv.hp_cuda_powersgd_encode1(G1, R1, Q1, M1, P1)
    drv.hp_cuda_powersgd_encode2(P1, M1, Q1)
    drv.hp_cuda_powersgd_decode(P1, Q1, M1, R1, G1)
    G2, R2, Q2, M2, P2 = fresh()
    assert pkg.hp_cuda_powersgd_encode1(G2, R2, Q2, M2, P2) == 0
    assert pkg.hp_cuda_powersgd_encode2(P2, M2, Q2) == 0
    assert pkg.hp_cuda_powersgd_decode(P2, Q2, M2, R2, G2) == 0
    torch.cuda.synchronize()
    for a, b, what in ((G1, G2, "grad"), (R1, R2, "residual"), (Q1, Q2, "Q"), (M1, M2, "M"), (P1, P2, "P")):
        for i in range(len(shapes)):
            assert_bits_equal(host(a[i]).ravel(), host(b[i]).ravel(), f"{what}[{i}]")
    del gen
