"""Entry points that only enqueue kernels can be recorded into a HIP graph and replayed: TBQ encode and
decode (no workspace, no host wait), TernGrad decode (the header is parsed on the device) and the three
PowerSGD phases (their workspace is in place after one eager call).  Each graph is replayed several times
with fresh inputs in the same buffers and eager work in between, and every replay is checked against the
CPU oracle (PowerSGD: against the eager calls).  TernGrad encode and the GradDrop calls are not
recordable: the first bakes a per-call epoch into its kernel arguments, the others wait for the stream."""
import numpy as np
import pytest
import torch

from gpu_util import Tbq, Terngrad, assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


def test_tbq_and_terngrad_decode_in_a_graph(capi, oracle_cpu):
    tbq, tg = Tbq(capi), Terngrad(capi)
    rng = np.random.default_rng(31)
    ns, thr = [70_001, 300_000, 1_050_000], 2e-3
    dg = [torch.zeros(n, device="cuda") for n in ns]
    dr = [torch.zeros(n, device="cuda") for n in ns]
    packed = [torch.zeros((n + 3) // 4, dtype=torch.uint8, device="cuda") for n in ns]
    dec = [torch.zeros(n, device="cuda") for n in ns]
    nt = 200_003
    msg = torch.zeros(tg.packed_size(nt, 2), dtype=torch.uint8, device="cuda")
    tdec = torch.zeros(nt, device="cuda")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        tbq.encode(dg, dr, [thr] * 3, outs=packed)          # eager once on the capture stream
        tbq.decode(packed, dec, [thr] * 3, [0, 0, 0])
        tg.decode([msg], [tdec], [0])
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            tbq.encode(dg, dr, [thr] * 3, outs=packed)
            tbq.decode(packed, dec, [thr] * 3, [0, 0, 0])
            tg.decode([msg], [tdec], [0])
    for rep in range(4):
        gs = [rng.normal(0, 2e-3, n).astype(np.float32) for n in ns]
        rs = [rng.normal(0, 1e-3, n).astype(np.float32) for n in ns]
        for a, b in zip(dg, gs): a.copy_(dev(b))
        for a, b in zip(dr, rs): a.copy_(dev(b))
        x = rng.normal(0, 1e-2, nt).astype(np.float32)
        rc, ref_msg = oracle_cpu.terngrad_encode(x, 2, 1, 1000 + rep)
        msg.copy_(dev(ref_msg))
        eager = torch.randn(1 << 20, device="cuda").sum()     # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, n in enumerate(ns):
            r_ref = rs[i].copy()
            p_ref = oracle_cpu.tbq_encode(gs[i], r_ref, thr)
            assert_bits_equal(host(packed[i]), p_ref, f"replay {rep}: packed[{i}]")
            assert_bits_equal(host(dr[i]), r_ref, f"replay {rep}: residual[{i}]")
            assert_bits_equal(host(dec[i]), oracle_cpu.tbq_decode(p_ref, n, thr), f"replay {rep}: decoded[{i}]")
        assert_bits_equal(host(tdec), oracle_cpu.terngrad_decode(ref_msg, nt)[1], f"replay {rep}: TernGrad decode")
        assert np.isfinite(float(eager))
    assert tg.status() == 0


def test_powersgd_phases_in_a_graph(pkg):
    shapes, rk = [(256, 192), (130, 515)], 4
    G = [torch.zeros(a * b, device="cuda") for a, b in shapes]
    R = [torch.zeros(a * b, device="cuda") for a, b in shapes]
    Q = [torch.zeros(b, rk, device="cuda") for a, b in shapes]
    M = [torch.zeros(a, b, device="cuda") for a, b in shapes]
    P = [torch.zeros(a, rk, device="cuda") for a, b in shapes]

    def phases():
        assert pkg.hp_cuda_powersgd_encode1(G, R, Q, M, P) == 0
        assert pkg.hp_cuda_powersgd_encode2(P, M, Q) == 0
        assert pkg.hp_cuda_powersgd_decode(P, Q, M, R, G) == 0

    gen = torch.Generator(device="cuda").manual_seed(7)

    def fill():
        for t in G: t.copy_(torch.randn(t.shape, device="cuda", generator=gen) * 1e-2)
        for t in R: t.copy_(torch.randn(t.shape, device="cuda", generator=gen) * 1e-3)
        for t in Q: t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        return [t.clone() for t in G], [t.clone() for t in R], [t.clone() for t in Q]

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for t in Q: t.normal_(generator=gen)
        phases()                                             # eager once: sizes the workspace, raises the LDS limit
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            phases()
    for rep in range(3):
        g0, r0, q0 = fill()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [[t.clone() for t in ts] for ts in (G, R, Q, M, P)]
        for dst, src in ((G, g0), (R, r0), (Q, q0)):
            for a, b in zip(dst, src): a.copy_(b)
        with torch.cuda.stream(side):
            phases()
            side.synchronize()
        for ts, gs, what in zip((G, R, Q, M, P), got, ("grad", "residual", "Q", "M", "P")):
            for i in range(len(shapes)):
                assert_bits_equal(host(gs[i]).ravel(), host(ts[i]).ravel(), f"replay {rep}: {what}[{i}]")
