"""hpx_terngrad_encode_noalloc: the TernGrad encode for callers that cannot allocate (code under graph capture,
tight serving loops).  It must write the same bytes as hpx_terngrad_encode, call after call on the same
device array (the second call is smaller, so slots of the first call's later tensors are left stale and
must not matter), allocate no device memory, and refuse what does not fit its fixed array."""
import numpy as np
import pytest
import torch

from gpu_util import Terngrad, assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


def _call_pair(tg, oracle_cpu, rng, sizes, bws, rnds):
    xs = [rng.normal(0, 10.0 ** rng.uniform(-4, 0), n).astype(np.float32) for n in sizes]
    xs[0][: min(5, sizes[0])] = 0.0                         # a zero in play for the sign-of-zero rule
    seeds = [int(s) for s in rng.integers(0, 2**63, len(sizes))]
    dx = [dev(x) for x in xs]
    want = tg.encode(dx, bws, rnds, seeds)
    outs = [torch.full((tg.packed_size(n, b),), 0x5A, dtype=torch.uint8, device="cuda") for n, b in zip(sizes, bws)]
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    tg.encode_noalloc(dx, bws, rnds, seeds, outs=outs)
    torch.cuda.synchronize()
    free1 = torch.cuda.mem_get_info()[0]
    assert free1 == free0, f"device memory in use changed by {free0 - free1} bytes across the call"
    for i in range(len(sizes)):
        assert_bits_equal(host(outs[i]), host(want[i]), f"message[{i}] n={sizes[i]} b={bws[i]} vs hpx_terngrad_encode")
        rc, ref = oracle_cpu.terngrad_encode(xs[i], bws[i], rnds[i], seeds[i])
        assert rc == 0
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] n={sizes[i]} b={bws[i]} vs the oracle")


def test_no_alloc_encode_matches_the_allocating_entry_point(capi, oracle_cpu):
    tg = Terngrad(capi)
    rng = np.random.default_rng(2026)
    # first call: 12 tensors (the 192-entry table), every width, both rounding modes, ragged ends
    sizes = [1_000_003, 1, 7, 4097, 300_001, 70_000, 16_384, 33, 2_500_000, 999, 65_537, 12]
    bws = [2, 1, 4, 8, 2, 1, 4, 8, 2, 2, 1, 4]
    rnds = [1, 0, 1, 1, 0, 1, 0, 1, 1, 1, 0, 1]
    _call_pair(tg, oracle_cpu, rng, sizes, bws, rnds)
    # second call, smaller (the small table): the array still holds the first call's words
    _call_pair(tg, oracle_cpu, rng, [50_001, 9, 123_456], [2, 4, 1], [1, 1, 1])
    # and once more with the first call's shape
    _call_pair(tg, oracle_cpu, rng, sizes, bws, rnds)


def test_no_alloc_encode_limits(capi):
    tg = Terngrad(capi)
    xs = [torch.randn(64, device="cuda") for _ in range(193)]
    tg.encode_noalloc(xs, [2] * 193, [1] * 193, list(range(193)), expect_rc=-3)
    assert "at most 192" in capi.last_error()
    tg.encode_noalloc(xs[:1], [3], [1], [0], expect_rc=-1)   # bad bit width: the reference body's own failure
    outs = tg.encode_noalloc(xs[:192], [2] * 192, [0] * 192, None)   # the largest call it takes
    want = tg.encode(xs[:192], [2] * 192, [0] * 192, None)
    torch.cuda.synchronize()
    for i in (0, 100, 191):
        assert_bits_equal(host(outs[i]), host(want[i]), f"message[{i}] of 192")


def test_no_alloc_encode_in_a_graph(capi, oracle_cpu):
    # what it is for: recorded once, replayed with fresh inputs in the same buffers
    tg = Terngrad(capi)
    rng = np.random.default_rng(7)
    sizes, bws, rnds, seeds = [200_003, 4096, 31], [2, 4, 2], [1, 1, 0], [11, 12, 13]
    dx = [torch.zeros(n, device="cuda") for n in sizes]
    outs = [torch.zeros(tg.packed_size(n, b), dtype=torch.uint8, device="cuda") for n, b in zip(sizes, bws)]
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        tg.encode_noalloc(dx, bws, rnds, seeds, outs=outs)   # eager once (looks up the array's address)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            tg.encode_noalloc(dx, bws, rnds, seeds, outs=outs)
    for rep in range(3):
        xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
        for a, b in zip(dx, xs): a.copy_(dev(b))
        eager = torch.randn(1 << 20, device="cuda").sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i in range(len(sizes)):
            rc, ref = oracle_cpu.terngrad_encode(xs[i], bws[i], rnds[i], seeds[i])
            assert_bits_equal(host(outs[i]), ref, f"replay {rep}: message[{i}]")
        assert np.isfinite(float(eager))
