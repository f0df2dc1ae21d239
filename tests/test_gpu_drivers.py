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


# ---- the drivers used the way the reference's scheduler uses them ---------------------------------------------
# hp_cuda.cpp runs a driver on one pool stream and consumes its output on ANOTHER pool stream straight afterwards,
# with no event between the two (TernGrad: driver on the compute stream, `C.copy_(B)` on the data stream,
# hp_cuda.cpp:464-468; GradDrop: hp_cuda_gdr on the compute stream, hp_cuda_gd over the same root tensors on the
# null stream, then the copies on the data stream, hp_cuda.cpp:284-313; pool streams are non-blocking, so the null
# stream orders nothing either).  That only works because the reference's drivers return with their work done
# (terngrad_body.h:285, gd_body.h:161,201,313).  The tests below repeat those sequences on torch's pool streams
# (non-blocking, as the reference's) and hold the result to the oracle bit for bit; the option "clock_seed" stands
# in for the wall clock the drivers seed from.

@pytest.fixture()
def fixed_clock(capi):
    old = capi.set_option("clock_seed", 77)
    yield 77
    capi.set_option("clock_seed", old)


def _pinned_like(t):
    return torch.empty(t.shape, dtype=t.dtype, pin_memory=True)


def _other_streams(k=4):
    # HIP multiplexes its streams onto a few hardware queues, and two streams that share a queue are ordered by
    # accident; consecutive pool streams go to different queues, so among four at least one runs beside `compute`.
    return [torch.cuda.Stream() for _ in range(k)]


def _peek(streams, tensors):
    """Clones of `tensors` (last first) taken on each of `streams`, with no wait on anything."""
    seen = []
    for s in streams:
        with torch.cuda.stream(s):
            seen.append([t.clone() for t in reversed(tensors)][::-1])
    return seen


@pytest.mark.parametrize("resident", [False, True])
def test_terngrad_message_is_complete_for_a_consumer_on_another_stream(drv, oracle_cpu, capi, fixed_clock, resident):
    rng = np.random.default_rng(50)
    ns = [30_000_003, 28_000_000, 26_000_001, 30_000_000, 29_000_002, 27_000_001] if not resident else [25_557_032]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in ns]
    old = capi.set_option("terngrad_resident_min", (5 << 20) if resident else -1)   # -1: every tensor takes two launches
    try:
        dx = [dev(x) for x in xs]
        Bs = [torch.full((oracle_cpu.terngrad_packed_size(n, 2),), 0x5A, dtype=torch.uint8, device="cuda") for n in ns]
        Cs = [_pinned_like(b) for b in Bs]
        compute, data, others = torch.cuda.Stream(), torch.cuda.Stream(), _other_streams()
        torch.cuda.synchronize()
        with torch.cuda.stream(compute):
            drv.hp_cuda_terngrad(dx, Bs, [2] * len(ns), [1] * len(ns))
        seen = _peek(others, Bs)
        with torch.cuda.stream(data):                       # hp_cuda.cpp:466-468, no event, no wait in between
            for b, c in zip(Bs, Cs):
                c.copy_(b, non_blocking=True)
        data.synchronize()                                   # hp_cuda.cpp:485
        torch.cuda.synchronize()
        for i, x in enumerate(xs):
            rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, fixed_clock)
            assert rc == 0
            for k, sk in enumerate(seen):
                assert_bits_equal(host(sk[i]), ref, f"message[{i}] as a kernel on side stream {k} saw it")
            assert_bits_equal(Cs[i].numpy(), ref, f"message[{i}] as the copy on the data stream saw it")
    finally:
        capi.set_option("terngrad_resident_min", old)
        torch.cuda.synchronize()


@pytest.mark.parametrize("drop_ratio", [0.999, 0.99])
def test_graddrop_batch_is_complete_for_a_consumer_on_another_stream(drv, oracle_cpu, fixed_clock, drop_ratio):
    # one call over a batch on the null stream (hp_cuda.cpp:292-301), B -> C on the data stream (:304-315); over
    # the seeds and sizes below some tensors overshoot `expected` and are cut, others are not (asserted at the end)
    rng = np.random.default_rng(51)
    ns, sr = [9_000_001, 7_000_000, 3_000_003, 1_200_000, 600_000], 0.01
    gs = [rng.laplace(0, 1e-3, n).astype(np.float32) for n in ns]
    rs = [rng.normal(0, 1e-4, n).astype(np.float32) for n in ns]
    dg, dres = [dev(g) for g in gs], [dev(r) for r in rs]
    sizes = [4 + 8 * oracle_cpu.gd_sizes(n, sr, drop_ratio)[1] for n in ns]
    Bs = [torch.full((s,), 0xEE, dtype=torch.uint8, device="cuda") for s in sizes]
    Cs = [_pinned_like(b) for b in Bs]
    data, others = torch.cuda.Stream(), _other_streams()
    torch.cuda.synchronize()
    with torch.cuda.stream(torch.cuda.default_stream()):
        drv.hp_cuda_gd(dg, dres, Bs, [sr] * len(ns), [drop_ratio] * len(ns))
    seen = _peek(others, Bs)
    with torch.cuda.stream(data):
        for b, c in zip(Bs, Cs):
            c.copy_(b, non_blocking=True)
        res_seen = [r.clone() for r in dres]
    data.synchronize()
    cut = []
    for i, n in enumerate(ns):
        r_ref = rs[i].copy()
        msg, info = oracle_cpu.gd_encode(gs[i], r_ref, sr, drop_ratio, fixed_clock)
        assert_bits_equal(Cs[i].numpy()[:msg.size], msg, f"message[{i}] as the data stream saw it")
        for k, sk in enumerate(seen):
            assert_bits_equal(host(sk[i])[:msg.size], msg, f"message[{i}] as a kernel on side stream {k} saw it")
        assert_bits_equal(host(res_seen[i]), r_ref, f"residual[{i}] as the data stream saw it")
        cut.append(info["candidates"] > info["kept"])
    assert any(cut) and not all(cut), cut                   # the batch holds both branches


def test_graddrop_root_decode_then_encode_on_different_streams(drv, oracle_cpu, fixed_clock):
    # A root task: hp_cuda_gdr adds the gathered messages into the gradient on the compute stream, hp_cuda_gd encodes
    # that gradient on the null stream, the message is copied out on the data stream (hp_cuda.cpp:241-259, 284-313).
    rng = np.random.default_rng(52)
    n, sr, dr_ = 12_000_001, 0.01, 0.999
    expected = oracle_cpu.gd_sizes(n, sr, dr_)[1]
    grad = rng.laplace(0, 1e-3, n).astype(np.float32)
    res = rng.normal(0, 1e-4, n).astype(np.float32)
    peers = []
    for p in range(3):                                       # three gathered slots from other ranks
        gp = rng.laplace(0, 1e-3, n).astype(np.float32)
        rp = np.zeros(n, np.float32)
        m, _ = oracle_cpu.gd_encode(gp, rp, sr, dr_, 1000 + p)
        peers.append(m)
    dgrad, dres = dev(grad), dev(res)
    dmsgs = [dev(m) for m in peers]
    B = torch.full((4 + 8 * expected,), 0xEE, dtype=torch.uint8, device="cuda")
    C = _pinned_like(B)
    compute, data = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(compute):
        drv.hp_cuda_gdr(dmsgs, [m.size for m in peers], [dgrad] * 3, [1, 1, 1])
    with torch.cuda.stream(torch.cuda.default_stream()):
        drv.hp_cuda_gd([dgrad], [dres], [B], [sr], [dr_])
    with torch.cuda.stream(data):
        C.copy_(B, non_blocking=True)
    data.synchronize()
    want = grad.copy()
    for m in peers:
        oracle_cpu.gd_decode(m, want, 1)
    r_ref = res.copy()
    msg, _ = oracle_cpu.gd_encode(want, r_ref, sr, dr_, fixed_clock)
    assert_bits_equal(C.numpy()[:msg.size], msg, "the root's message as the data stream saw it")
    torch.cuda.synchronize()
    assert_bits_equal(host(dgrad), want, "gradient after the gathered messages")
    assert_bits_equal(host(dres), r_ref, "residual after the root's encode")


def test_powersgd_phases_are_complete_for_a_consumer_on_another_stream(drv, pkg):
    # hp_cuda.cpp:729-768: the three drivers on the compute stream, names published after waiting for the data
    # stream only; a consumer then reads P, Q and the gradient on a stream of its own.
    shapes, rk = [(4096, 4096), (1024, 4096), (4096, 1024)] * 3, 4
    def fresh():
        g = torch.Generator(device="cuda").manual_seed(8)
        G = [torch.randn(a * b, device="cuda", generator=g) * 1e-2 for a, b in shapes]
        R = [torch.randn(a * b, device="cuda", generator=g) * 1e-3 for a, b in shapes]
        Q = [torch.randn(b, rk, device="cuda", generator=g) for a, b in shapes]
        M = [torch.zeros(a, b, device="cuda") for a, b in shapes]
        P = [torch.zeros(a, rk, device="cuda") for a, b in shapes]
        return G, R, Q, M, P
    G1, R1, Q1, M1, P1 = fresh()
    compute, other = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    seen = {}
    with torch.cuda.stream(compute):
        drv.hp_cuda_powersgd_encode1(G1, R1, Q1, M1, P1)
    with torch.cuda.stream(other):
        seen["P0"] = [p.clone() for p in P1]
    with torch.cuda.stream(compute):
        drv.hp_cuda_powersgd_encode2(P1, M1, Q1)
    with torch.cuda.stream(other):
        seen["P"] = [p.clone() for p in P1]
        seen["Q"] = [q.clone() for q in Q1]
    with torch.cuda.stream(compute):
        drv.hp_cuda_powersgd_decode(P1, Q1, M1, R1, G1)
    with torch.cuda.stream(other):
        seen["G"] = [g.clone() for g in G1]
        seen["R"] = [r.clone() for r in R1]
    other.synchronize()
    G2, R2, Q2, M2, P2 = fresh()
    assert pkg.hp_cuda_powersgd_encode1(G2, R2, Q2, M2, P2) == 0
    torch.cuda.synchronize()
    P0 = [p.clone() for p in P2]
    assert pkg.hp_cuda_powersgd_encode2(P2, M2, Q2) == 0
    assert pkg.hp_cuda_powersgd_decode(P2, Q2, M2, R2, G2) == 0
    torch.cuda.synchronize()
    for key, ref in (("P0", P0), ("P", P2), ("Q", Q2), ("G", G2), ("R", R2)):
        for i in range(len(shapes)):
            assert_bits_equal(host(seen[key][i]).ravel(), host(ref[i]).ravel(), f"{key}[{i}] as the other stream saw it")
