"""GPU parity: GradDrop ("DGC") encode/decode through the C ABI vs the CPU oracle.

Bit-exact: message bytes (header, index block, value block), residual after
encode, decoded tensors.  In the cut branch the order among equal |r| is
unspecified in the reference; the oracle and the kernels both keep ascending
index order among ties.
"""
import numpy as np
import pytest
import torch

from gpu_util import assert_bits_equal, dev, host, stream_ptr

pytestmark = pytest.mark.gpu


class Gd:
    def __init__(self, capi):
        self.c = capi
        self.L = capi.load()

    def encode(self, gs, rs, outs, srs, drs, seeds, expect_rc=0):
        c = self.c
        rc = self.L.hpx_gd_encode(len(gs), c.ptr_array([g.data_ptr() for g in gs]), c.i32_array([g.numel() for g in gs]),
                                  c.ptr_array([r.data_ptr() for r in rs]), c.ptr_array([o.data_ptr() for o in outs]),
                                  c.f64_array(srs), c.f64_array(drs), c.u64_array(seeds) if seeds is not None else None,
                                  stream_ptr())
        assert rc == expect_rc, (rc, c.last_error())

    def decode(self, msgs, in_sizes, outs, adds, expect_rc=0):
        c = self.c
        rc = self.L.hpx_gd_decode(len(msgs), c.ptr_array([m.data_ptr() for m in msgs]), c.i32_array(in_sizes),
                                  c.ptr_array([o.data_ptr() for o in outs]), c.i32_array([o.numel() for o in outs]),
                                  c.i32_array(adds), stream_ptr())
        assert rc == expect_rc, (rc, c.last_error())


@pytest.fixture(scope="module")
def gd(capi):
    assert torch.cuda.is_available()
    return Gd(capi)


@pytest.fixture(autouse=True, scope="module", params=["gather", "provisional", "provisional_fall_back"])
def threshold_path(request, capi):
    """Every test of this module runs three times: with the threshold taken from the gathered sample before the
    pass; with the pass started from a provisional threshold and the exact one found afterwards (an option, off by
    default); and with the provisional threshold put at the top of its
    samples, so that it lies above the exact one and every tensor falls back to the gather path after the pass has
    updated the residual.  The messages are the same bit for bit."""
    mode = request.param
    old = [capi.set_option("gd_provisional_min_samples", -1 if mode == "gather" else 0),
           capi.set_option("gd_provisional_margin", 0 if mode == "provisional_fall_back" else 3)]
    yield mode
    capi.set_option("gd_provisional_min_samples", old[0])
    capi.set_option("gd_provisional_margin", old[1])


def test_the_path_under_test_is_the_one_that_runs(gd, oracle_cpu, capi, threshold_path):
    rng = np.random.default_rng(99)
    n = 400_003
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    r0 = rng.normal(0, 1e-4, n).astype(np.float32)
    L = capi.load()
    before = L.hpx_gd_fallbacks(stream_ptr())
    L.hpx_profile_reset(); L.hpx_profile_enable(1)
    try:
        _check_encode(gd, oracle_cpu, g, r0, 0.01, 0.999, 5)
        launched = {k: capi.profile_query(k)[1] for k in ("gd_sample_kernel", "gd_presample_kernel", "gd_recount_kernel")}
    finally:
        L.hpx_profile_enable(0); L.hpx_profile_reset()
    fell_back = L.hpx_gd_fallbacks(stream_ptr()) - before
    if threshold_path == "gather":
        assert launched == {"gd_sample_kernel": 1, "gd_presample_kernel": 0, "gd_recount_kernel": 0} and fell_back == 0
    elif threshold_path == "provisional":
        assert launched == {"gd_sample_kernel": 0, "gd_presample_kernel": 1, "gd_recount_kernel": 1} and fell_back == 0
    else:
        assert launched == {"gd_sample_kernel": 1, "gd_presample_kernel": 1, "gd_recount_kernel": 1} and fell_back == 1


_BRANCHES = set()


def _out_bytes(n, dr):
    return 4 + 8 * int(np.ceil(n * (1 - dr)))


def _check_encode(gd, oracle_cpu, g, r0, sr, dr, seed, guard=64):
    n = g.size
    dg, dr_ = dev(g), dev(r0)
    size = _out_bytes(n, dr)
    out = torch.full((size + guard,), 0xEE, dtype=torch.uint8, device="cuda")
    gd.encode([dg], [dr_], [out], [sr], [dr], [seed])
    torch.cuda.synchronize()
    r_ref = r0.copy()
    msg, info = oracle_cpu.gd_encode(g, r_ref, sr, dr, seed)
    got = host(out)
    m = int(got[:4].view(np.int32)[0])
    assert m == msg.size, (m, msg.size, info)
    # In the cut branch equal |r| keep ascending index order on both sides (the
    # reference leaves that order unspecified), so ties need no special care here.
    assert_bits_equal(got[:m], msg, f"message n={n} seed={seed} info={info}")
    assert np.all(got[size:] == 0xEE), "wrote past 4 + 8*expected bytes"
    assert_bits_equal(host(dr_), r_ref, "residual")
    assert_bits_equal(host(dg), g, "gradient untouched")
    return out, msg, info


@pytest.mark.parametrize("n,sr,dr", [(1000, 0.05, 0.99), (4095, 0.05, 0.99), (4096, 0.01, 0.999), (4097, 0.1, 0.9),
                                     (10007, 0.1, 0.9), (65536, 0.5, 0.5), (100003, 0.01, 0.999), (300007, 0.02, 0.97),
                                     (1_000_003, 0.01, 0.999), (5_000_011, 0.01, 0.999)])
def test_encode_decode_sizes(gd, oracle_cpu, n, sr, dr):
    rng = np.random.default_rng(n)
    branches = set()
    for seed in (0, 1, 12345, 2**40 + 5, 2**64 - 2, 77):
        g = rng.laplace(0, 1e-3, n).astype(np.float32)
        r0 = rng.normal(0, 1e-4, n).astype(np.float32)
        out, msg, info = _check_encode(gd, oracle_cpu, g, r0, sr, dr, seed)
        branches.add(info["candidates"] > info["kept"])
        for add in (0, 1):
            base = rng.normal(0, 1, n).astype(np.float32)
            dout = dev(base)
            gd.decode([out], [msg.size], [dout], [add])
            torch.cuda.synchronize()
            ref = base.copy()
            assert oracle_cpu.gd_decode(msg, ref, add) == 0
            assert_bits_equal(host(dout), ref, f"decode add={add}")
    _BRANCHES.update(branches)


def test_both_branches_were_exercised():
    # runs after the size sweep above: the sweep met tensors that were cut and tensors that were not
    assert _BRANCHES == {True, False}, _BRANCHES


def test_cut_branch_small_sample(gd, oracle_cpu):
    # threshold = 2nd largest of 1000 samples: about twice as many candidates as `expected`
    rng = np.random.default_rng(3)
    n = 200_000
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    r0 = rng.normal(0, 1e-4, n).astype(np.float32)
    cuts = 0
    for seed in range(8):
        out, msg, info = _check_encode(gd, oracle_cpu, g, r0, 0.005, 0.999, seed)
        cuts += info["candidates"] > info["kept"]
    assert cuts >= 2


def test_far_more_candidates_than_reserved(gd, oracle_cpu):
    # The sampled positions (a known function of the seed) hold tiny values, everything else is
    # large: the threshold comes out tiny and nearly the whole tensor is a candidate.
    rng = np.random.default_rng(4)
    n, sr, dr, seed = 400_000, 0.01, 0.999, 9
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    g[np.abs(g) < 1e-5] = 1e-5
    sampled = np.array([oracle_cpu.gd_sample_index(seed, x, n) for x in range(4000)])
    g[sampled] = (1e-7 * (1 + np.arange(4000) / 4000.0)).astype(np.float32)
    out, msg, info = _check_encode(gd, oracle_cpu, g, np.zeros(n, np.float32), sr, dr, seed)
    assert info["threshold"] < 3e-7 and info["candidates"] > 390_000 and info["kept"] == oracle_cpu.gd_sizes(n, sr, dr)[1]


def test_cut_branch_many_ties(gd, oracle_cpu):
    # Values on a coarse grid, threshold forced tiny through the sampled positions: nearly every
    # element is a candidate, thousands share each |r|, and the cut keeps them in ascending index
    # order within a value (the sort has to be stable across its tiles and passes).
    rng = np.random.default_rng(11)
    n, sr, dr, seed = 300_000, 0.01, 0.99, 21
    g = (np.round(rng.laplace(0, 1e-3, n) * 2000) / 2000).astype(np.float32)
    g[g == 0] = np.float32(0.0005)
    sampled = np.array([oracle_cpu.gd_sample_index(seed, x, n) for x in range(3000)])
    g[sampled] = (1e-7 * (1 + np.arange(3000) / 3000.0)).astype(np.float32)
    out, msg, info = _check_encode(gd, oracle_cpu, g, np.zeros(n, np.float32), sr, dr, seed)
    kept = oracle_cpu.gd_sizes(n, sr, dr)[1]
    assert info["candidates"] > 290_000 and info["kept"] == kept
    vals = msg[4 + 4 * kept:].view(np.float32)
    assert np.unique(np.abs(vals)).size < 40      # ties dominate


@pytest.mark.parametrize("ratio,bits", [(1 + 2.0**-8, 16), (1 + 2.0**-6, 18), (1.5, 22), (6.0, 26), (300.0, 27), (1e4, 28)])
def test_cut_branch_key_widths(gd, oracle_cpu, ratio, bits):
    # The sort of the cut branch picks its digit width and number of passes from the widest key (the distance of
    # the largest |r| above the threshold, in fp32 bit patterns).  Sampled positions hold the smallest values, so
    # every other element is a candidate and the cut runs; the other values spread up to `ratio` times the
    # threshold: keys of about `bits` bits, i.e. 2 x 8, 2 x 9, 3 x 8, 3 x 9, 3 x 9 and 4 x 8 bits.
    rng = np.random.default_rng(int(bits))
    n, sr, dr, seed = 150_000, 0.01, 0.99, 5
    g = np.exp(rng.uniform(np.log(1.0005), np.log(ratio), n)).astype(np.float32) * rng.choice([-1.0, 1.0], n).astype(np.float32)
    g[np.abs(g) < 1.0005] = np.float32(1.0005)
    sampled = np.array([oracle_cpu.gd_sample_index(seed, x, n) for x in range(1500)])
    g[sampled] = (1.0 + 1e-4 * np.arange(1500) / 1500.0).astype(np.float32)
    out, msg, info = _check_encode(gd, oracle_cpu, g, np.zeros(n, np.float32), sr, dr, seed)
    kept = oracle_cpu.gd_sizes(n, sr, dr)[1]
    assert info["candidates"] > 140_000 and info["kept"] == kept
    top = np.abs(g).max().view(np.uint32) - np.float32(info["threshold"]).view(np.uint32)
    assert int(top).bit_length() in (bits - 1, bits, bits + 1), (int(top).bit_length(), bits)


def test_nothing_selected(gd, oracle_cpu):
    n = 50_000
    _check_encode(gd, oracle_cpu, np.zeros(n, np.float32), np.zeros(n, np.float32), 0.05, 0.99, 0)


def test_several_tensors_and_messages(gd, oracle_cpu):
    rng = np.random.default_rng(6)
    sizes = [1000, 70001, 4096, 250_003]
    gs = [rng.laplace(0, 1e-3, n).astype(np.float32) for n in sizes]
    rs = [rng.normal(0, 1e-4, n).astype(np.float32) for n in sizes]
    dgs, drs_ = [dev(g) for g in gs], [dev(r) for r in rs]
    outs = [torch.zeros(_out_bytes(n, 0.99), dtype=torch.uint8, device="cuda") for n in sizes]
    seeds = [3, 4, 5, 6]
    gd.encode(dgs, drs_, outs, [0.05] * 4, [0.99] * 4, seeds)
    torch.cuda.synchronize()
    msgs = []
    for i, n in enumerate(sizes):
        r_ref = rs[i].copy()
        msg, _ = oracle_cpu.gd_encode(gs[i], r_ref, 0.05, 0.99, seeds[i])
        assert_bits_equal(host(outs[i])[: msg.size], msg, f"message[{i}]")
        assert_bits_equal(host(drs_[i]), r_ref, f"residual[{i}]")
        msgs.append(msg)
    # several messages accumulate into ONE tensor sequentially (the root's gather-decode, hp_cuda.cpp:241-259)
    n = 70001
    m2 = []
    for seed in (11, 12, 13):
        r = np.zeros(n, np.float32)
        m, _ = oracle_cpu.gd_encode(rng.laplace(0, 1e-3, n).astype(np.float32), r, 0.05, 0.99, seed)
        m2.append(m)
    base = rng.normal(0, 1, n).astype(np.float32)
    dout = dev(base)
    dm = [dev(m) for m in m2]
    gd.decode(dm, [m.size for m in m2], [dout] * 3, [1, 1, 1])
    ref = base.copy()
    for m in m2:
        oracle_cpu.gd_decode(m, ref, 1)
    assert_bits_equal(host(dout), ref, "accumulated decode")


def test_bucket_of_ragged_tensors_in_one_call(gd, oracle_cpu, capi, threshold_path):
    # The scheduler hands hpx_gd_encode whole batches (hp_cuda.cpp:284-301).  260 tensors - more than one launch
    # table holds - of ragged sizes in ONE call: every phase is one launch for a table of tensors, the host
    # learns all counts at once, and only the tensors that overshoot are sorted and cut afterwards.  Among them:
    # tensors that are cut and tensors that are not, one that selects nothing, one whose candidates are far
    # more than the space reserved for the cut, single-element and tile-edge sizes.
    rng = np.random.default_rng(60)
    sizes = [int(np.exp(rng.uniform(np.log(50), np.log(400_000)))) for _ in range(150)]
    sizes += [int(np.exp(rng.uniform(np.log(50), np.log(20_000)))) for _ in range(100)]
    sizes += [1, 2, 4095, 4096, 4097, 8191, 65_536, 262_145, 1_000_003, 400_003]
    srs = [float(rng.choice([0.01, 0.05, 0.2, 0.5])) for _ in sizes]
    drs = [float(rng.choice([0.9, 0.99, 0.999])) for _ in sizes]
    seeds = [int(x) for x in rng.integers(0, 2**63, len(sizes))]
    gs = [rng.laplace(0, 1e-3, n).astype(np.float32) for n in sizes]
    rs = [rng.normal(0, 1e-4, n).astype(np.float32) for n in sizes]
    for i, n in enumerate(sizes):                                 # parameters the reference itself would accept
        sc = int(np.ceil(n * srs[i]))
        if not (sc > 0 and int(sc * (1 - drs[i])) < sc):
            srs[i], drs[i] = 1.0, 0.5
    zero_at = 17                                                  # nothing selected: header only
    gs[zero_at][:] = 0; rs[zero_at][:] = 0
    flood_at = len(sizes) - 1                                     # nearly everything is a candidate
    n_f = sizes[flood_at]
    srs[flood_at], drs[flood_at] = 0.01, 0.999
    gs[flood_at][np.abs(gs[flood_at]) < 1e-5] = 1e-5
    sampled = np.array([oracle_cpu.gd_sample_index(seeds[flood_at], x, n_f) for x in range(int(np.ceil(n_f * 0.01)))])
    gs[flood_at][sampled] = (1e-7 * (1 + np.arange(sampled.size) / sampled.size)).astype(np.float32)
    rs[flood_at][:] = 0
    dgs, drs_ = [dev(g) for g in gs], [dev(r) for r in rs]
    guard = 64
    outs = [torch.full((_out_bytes(n, d) + guard,), 0xEE, dtype=torch.uint8, device="cuda") for n, d in zip(sizes, drs)]
    L = capi.load()
    L.hpx_profile_reset(); L.hpx_profile_enable(1)
    try:
        gd.encode(dgs, drs_, outs, srs, drs, seeds)
        torch.cuda.synchronize()
        stream_launches = capi.profile_query("gd_stream_kernel")[1]
    finally:
        L.hpx_profile_enable(0); L.hpx_profile_reset()
    # 260 tensors: two launch tables, not 260 launches (on the provisional path the tensors whose provisional
    # threshold ties with or exceeds the exact one - tiny samples, the flooded tensor - share further launches)
    assert stream_launches == 2 if threshold_path == "gather" else 2 <= stream_launches <= 4, stream_launches
    cut = kept_all = 0
    for i, n in enumerate(sizes):
        r_ref = rs[i].copy()
        msg, info = oracle_cpu.gd_encode(gs[i], r_ref, srs[i], drs[i], seeds[i])
        got = host(outs[i])
        size = _out_bytes(n, drs[i])
        assert_bits_equal(got[:msg.size], msg, f"message[{i}] n={n} sr={srs[i]} dr={drs[i]} info={info}")
        assert np.all(got[size:] == 0xEE), f"tensor {i}: wrote past 4 + 8*expected bytes"
        assert_bits_equal(host(drs_[i]), r_ref, f"residual[{i}]")
        assert_bits_equal(host(dgs[i]), gs[i], f"gradient[{i}] untouched")
        cut += info["candidates"] > info["kept"]
        kept_all += info["candidates"] <= info["kept"]
        if i == zero_at:
            assert msg.size == 4
        if i == flood_at:
            assert info["candidates"] > info["kept"] + 65536       # more than the cut path's buffers were laid out for
    assert cut >= 10 and kept_all >= 10, (cut, kept_all)


def test_more_tensors_than_one_round_of_reports(gd, oracle_cpu):
    # The host learns the candidate counts from a block of pinned words that holds 4092 tensors' reports; a call
    # with more tensors goes through the phases, the wait and the cut once per such round (and through seventeen
    # launch tables).  4200 small tensors as views of one buffer, both branches among them.
    rng = np.random.default_rng(62)
    count = 4200
    sizes = [int(x) for x in rng.integers(40, 400, count)]
    starts = np.concatenate([[0], np.cumsum(sizes)])
    g_all = rng.laplace(0, 1e-3, int(starts[-1])).astype(np.float32)
    r_all = rng.normal(0, 1e-4, int(starts[-1])).astype(np.float32)
    dg_all, dr_all = dev(g_all), dev(r_all)
    dgs = [dg_all[starts[i]:starts[i + 1]] for i in range(count)]
    drs_ = [dr_all[starts[i]:starts[i + 1]] for i in range(count)]
    obytes = [(_out_bytes(n, 0.9) + 3) // 4 * 4 for n in sizes]
    ostarts = np.concatenate([[0], np.cumsum(obytes)])
    out_all = torch.full((int(ostarts[-1]),), 0xEE, dtype=torch.uint8, device="cuda")
    outs = [out_all[ostarts[i]:ostarts[i + 1]] for i in range(count)]
    seeds = [int(x) for x in rng.integers(0, 2**63, count)]
    gd.encode(dgs, drs_, outs, [0.5] * count, [0.9] * count, seeds)
    torch.cuda.synchronize()
    got_all, r_got = host(out_all), host(dr_all)
    assert_bits_equal(host(dg_all), g_all, "gradients untouched")
    cut = 0
    for i, n in enumerate(sizes):
        r_ref = r_all[starts[i]:starts[i + 1]].copy()
        msg, info = oracle_cpu.gd_encode(g_all[starts[i]:starts[i + 1]], r_ref, 0.5, 0.9, seeds[i])
        got = got_all[ostarts[i]:ostarts[i + 1]]
        assert_bits_equal(got[:msg.size], msg, f"message[{i}] n={n} info={info}")
        assert np.all(got[_out_bytes(n, 0.9):] == 0xEE), f"tensor {i}: wrote past its message"
        assert_bits_equal(r_got[starts[i]:starts[i + 1]], r_ref, f"residual[{i}]")
        cut += info["candidates"] > info["kept"]
    assert 100 < cut < count - 100, cut


def test_bad_tensor_in_a_bucket_is_reported_and_skipped(gd, oracle_cpu):
    # like the reference driver, which prints and goes on (hp_cuda_kernel.cu:90-92): the call returns the failure,
    # the other tensors are encoded
    rng = np.random.default_rng(61)
    sizes = [5000, 100, 70_001]
    gs = [rng.laplace(0, 1e-3, n).astype(np.float32) for n in sizes]
    rs = [rng.normal(0, 1e-4, n).astype(np.float32) for n in sizes]
    dgs, drs_ = [dev(g) for g in gs], [dev(r) for r in rs]
    outs = [torch.zeros(_out_bytes(n, 0.9) + 64, dtype=torch.uint8, device="cuda") for n in sizes]
    gd.encode(dgs, drs_, outs, [0.05, 0.05, 0.05], [0.9, 0.0, 0.9], [1, 2, 3], expect_rc=-3)   # tensor 1: threshold index out of range
    torch.cuda.synchronize()
    for i in (0, 2):
        r_ref = rs[i].copy()
        msg, _ = oracle_cpu.gd_encode(gs[i], r_ref, 0.05, 0.9, [1, 2, 3][i])
        assert_bits_equal(host(outs[i])[:msg.size], msg, f"message[{i}]")
        assert_bits_equal(host(drs_[i]), r_ref, f"residual[{i}]")
    assert_bits_equal(host(drs_[1]), rs[1], "the skipped tensor's residual is untouched")


def test_decode_errors(gd, oracle_cpu):
    n = 5000
    rng = np.random.default_rng(1)
    r = np.zeros(n, np.float32)
    msg, _ = oracle_cpu.gd_encode(rng.laplace(0, 1e-3, n).astype(np.float32), r, 0.05, 0.99, 3)
    good = dev(np.array([4, 0, 0, 0], np.uint8))
    o1 = torch.ones(n, device="cuda"); o2 = torch.ones(n, device="cuda")
    # a short message fails the whole call before any output is touched (gd_body.h:317-325)
    gd.decode([good, dev(msg)], [4, msg.size - 1], [o1, o2], [0, 0], expect_rc=-1)
    torch.cuda.synchronize()
    assert bool((o1 == 1).all()) and bool((o2 == 1).all())
    gd.decode([good], [4], [o1], [0])      # k == 0: write mode still zero-fills
    assert bool((o1 == 0).all())


def test_encode_argument_errors(gd):
    g = torch.zeros(100, device="cuda"); r = torch.zeros(100, device="cuda")
    out = torch.zeros(64, dtype=torch.uint8, device="cuda")
    gd.encode([g], [r], [out], [0.05], [0.0], [0], expect_rc=-3)   # threshold index == sample_cnt (out of range in the reference)
    gd.encode([g], [r], [out[1:]], [0.05], [0.9], [0], expect_rc=-3)  # misaligned output


def test_full_size_config3(gd):
    # 138,357,544 elements (VGG-16), Laplace(0,1e-3) + residual N(0,1e-4), sample 1 %, keep 0.1 %, seed 0
    from oracle import cpu
    n, sr, dr, seed = 138_357_544, 0.01, 0.999, 0
    gen = torch.Generator(device="cuda").manual_seed(0)
    u = torch.rand(n, device="cuda", generator=gen) - 0.5
    g = (-1e-3 * torch.sign(u) * torch.log1p(-2 * u.abs())).float()
    del u
    r = torch.randn(n, device="cuda", generator=gen) * 1e-4
    gh, rh = host(g), host(r)
    out = torch.zeros(_out_bytes(n, dr), dtype=torch.uint8, device="cuda")
    gd.encode([g], [r], [out], [sr], [dr], [seed])
    torch.cuda.synchronize()
    msg, info = cpu.gd_encode(gh, rh, sr, dr, seed)
    got = host(out)
    assert int(got[:4].view(np.int32)[0]) == msg.size, info
    assert_bits_equal(got[: msg.size], msg, f"full-size message {info}")
    assert_bits_equal(host(r), rh, "full-size residual")
    # size-independent property: R_after + scatter(idx, val) == R_before + G, via decode(add) on the device
    dec = r.clone()
    gd.decode([out], [msg.size], [dec], [1])
    idx, val = cpu.gd_split(msg)
    decoded = host(dec)
    rh2 = rh.copy(); rh2[idx] += val
    assert_bits_equal(decoded, rh2, "decode(add) restores the accumulated tensor")


# ---- the sparsifier without residual (dgc_body.h) ---------------------------------------------------
def _dgc_encode(gd, dg, out, sr, sp, seed, expect_rc=0):
    c = gd.c
    rc = gd.L.hpx_dgc_encode(1, c.ptr_array([dg.data_ptr()]), c.i32_array([dg.numel()]), c.ptr_array([out.data_ptr()]),
                             c.f64_array([sr]), c.f64_array([sp]), c.u64_array([seed]), stream_ptr())
    assert rc == expect_rc, (rc, c.last_error())


@pytest.mark.parametrize("n,sr,sp", [(1000, 0.05, 0.01), (4097, 0.1, 0.1), (65536, 0.5, 0.5), (100003, 0.01, 0.001),
                                     (1_000_003, 0.01, 0.001), (5_000_011, 0.01, 0.001)])
def test_dgc_without_residual(gd, oracle_cpu, n, sr, sp):
    rng = np.random.default_rng(n + 1)
    branches = set()
    for seed in (0, 1 << 22, 12345 << 20, 2**64 - 2):
        g = rng.laplace(0, 1e-3, n).astype(np.float32)
        dg = dev(g)
        size = 4 + 8 * int(np.ceil(n * sp))
        out = torch.full((size + 64,), 0xEE, dtype=torch.uint8, device="cuda")
        _dgc_encode(gd, dg, out, sr, sp, seed)
        torch.cuda.synchronize()
        g_ref = g.copy()
        msg, info = oracle_cpu.dgc_encode(g_ref, sr, sp, seed)
        got = host(out)
        m = int(got[:4].view(np.int32)[0])
        assert m == msg.size, (m, msg.size, info)
        assert_bits_equal(got[:m], msg, f"message n={n} seed={seed} info={info}")
        assert np.all(got[size:] == 0xEE), "wrote past 4 + 8*expected bytes"
        assert_bits_equal(host(dg), g_ref, "gradient after encode (selected entries cleared)")
        branches.add(info["candidates"] > info["kept"])
        # decode: write mode leaves the other entries alone (dgc_body.h:283-289), add mode accumulates
        for add in (0, 1):
            base = rng.normal(0, 1, n).astype(np.float32)
            dout = dev(base)
            c = gd.c
            rc = gd.L.hpx_dgc_decode(1, c.ptr_array([out.data_ptr()]), c.i32_array([msg.size]), c.ptr_array([dout.data_ptr()]),
                                     c.i32_array([n]), c.i32_array([add]), stream_ptr())
            assert rc == 0, c.last_error()
            torch.cuda.synchronize()
            ref = base.copy()
            assert oracle_cpu.dgc_decode(msg, ref, add) == 0
            assert_bits_equal(host(dout), ref, f"decode add={add}")
    if n >= 100003:
        assert True in branches or False in branches
