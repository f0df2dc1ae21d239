"""GPU parity: TernGrad b-bit quantiser through the C ABI vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from gpu_util import Terngrad, assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tg(capi):
    assert torch.cuda.is_available()
    return Terngrad(capi)


def _check(tg, oracle_cpu, xs, bws, rnds, seeds, adds, rng):
    dx = [dev(x) for x in xs]
    outs = tg.encode(dx, bws, rnds, seeds)
    torch.cuda.synchronize()
    for i, x in enumerate(xs):
        rc, ref = oracle_cpu.terngrad_encode(x, bws[i], rnds[i], seeds[i])
        assert rc == 0
        assert_bits_equal(host(outs[i])[:10], ref[:10], f"header[{i}] n={x.size} b={bws[i]}")
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] n={x.size} b={bws[i]} rnd={rnds[i]}")
        assert_bits_equal(host(dx[i]), x, "input untouched")
    bases = [rng.normal(0, 1, x.size).astype(np.float32) for x in xs]
    douts = [dev(b) for b in bases]
    tg.decode(outs, douts, adds)
    torch.cuda.synchronize()
    for i, x in enumerate(xs):
        rc, ref = oracle_cpu.terngrad_decode(host(outs[i]), x.size, bases[i].copy(), adds[i])
        assert rc == 0
        assert_bits_equal(host(douts[i]), ref, f"decoded[{i}] n={x.size} b={bws[i]} add={adds[i]}")
    assert tg.status() == 0


def test_known_answers(tg):
    x = (np.array([(7 * i % 11) - 5 for i in range(40)], np.float32) * np.float32(0.01)).astype(np.float32)
    out = tg.encode([dev(x)], [2], [1], [12345])[0]
    assert host(out)[10:15].tobytes().hex() == "c8b22cb72d"
    out = tg.encode([dev(x[:22].copy())], [2], [0], [0])[0]
    assert host(out).tobytes().hex() == "0202cccc4cbdcccc4c3dd87618b61d06"


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("rnd", [0, 1])
def test_sizes_and_tails(tg, oracle_cpu, b, rnd):
    rng = np.random.default_rng(100 * b + rnd)
    sizes = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 1023, 4095, 4096, 4097, 8191, 8192, 8193, 8199, 32768 + 5, 300007]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    seeds = [int(s) for s in rng.integers(0, 2**63, len(sizes))]
    _check(tg, oracle_cpu, xs, [b] * len(sizes), [rnd] * len(sizes), seeds, [i & 1 for i in range(len(sizes))], rng)


def test_more_tensors_than_one_table(tg, oracle_cpu):
    rng = np.random.default_rng(21)
    sizes = [int(s) for s in np.exp(rng.uniform(np.log(2), np.log(20000), 450))]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    bws = [int(b) for b in rng.choice([1, 2, 4, 8], len(sizes))]
    rnds = [int(r) for r in rng.integers(0, 2, len(sizes))]
    seeds = [int(s) for s in rng.integers(0, 2**64 - 1, len(sizes), dtype=np.uint64)]
    _check(tg, oracle_cpu, xs, bws, rnds, seeds, [int(a) for a in rng.integers(0, 2, len(sizes))], rng)


def test_seed_edges(tg, oracle_cpu):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 1e-2, 70001).astype(np.float32)
    seeds = [0, 1, 2**32 - 1, 2**32, 2**32 - 70001 // 4 + 5, 2**63, 2**64 - 1, 1700000000123456789]
    _check(tg, oracle_cpu, [x] * len(seeds), [2] * len(seeds), [1] * len(seeds), seeds, [0] * len(seeds), rng)


def test_scalar_preparation_many_ranges(tg, oracle_cpu):
    # gap (fp32 divide) and 1/(gap+1e-8) (fp64) are computed on the device: sweep min/max over many magnitudes
    rng = np.random.default_rng(8)
    xs, bws = [], []
    for k in range(240):
        lo = np.float32(rng.normal() * 10.0 ** rng.uniform(-30, 20))
        hi = np.float32(lo + abs(np.float32(rng.normal() * 10.0 ** rng.uniform(-38, 20))))
        n = int(rng.integers(2, 40))
        x = rng.uniform(lo, hi, n).astype(np.float32)
        x[0], x[-1] = lo, hi
        xs.append(x)
        bws.append(int(rng.choice([1, 2, 4, 8])))
    seeds = [int(s) for s in rng.integers(0, 2**63, len(xs))]
    for rnd in (0, 1):
        _check(tg, oracle_cpu, xs, bws, [rnd] * len(xs), seeds, [0] * len(xs), rng)


def test_constant_and_zero_tensors(tg, oracle_cpu):
    rng = np.random.default_rng(2)
    xs = [np.zeros(1000, np.float32), np.full(1003, -0.0, np.float32), np.full(4097, 0.125, np.float32),
          np.array([0.5, -0.0, 0.0, 0.25, 0.0], np.float32), np.array([-0.5, 0.0, -0.0, -0.25], np.float32),
          np.concatenate([np.full(20000, 0.5, np.float32), [-0.0], np.full(9000, 0.25, np.float32), [0.0]]).astype(np.float32),
          np.array([1e-45, 0, 3e-45, 2e-45] * 50, np.float32)]
    for rnd in (0, 1):
        _check(tg, oracle_cpu, xs, [2] * len(xs), [rnd] * len(xs), [77] * len(xs), [0] * len(xs), rng)


def test_outliers_config_shape_small(tg, oracle_cpu):
    # the config-2 distribution at a size the oracle finishes quickly
    rng = np.random.default_rng(0)
    n = 2_000_003
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    pos = rng.choice(n, n // 1000, replace=False)
    x[pos] = np.where(rng.random(pos.size) < 0.5, 0.5, -0.5).astype(np.float32)
    _check(tg, oracle_cpu, [x], [2], [1], [0], [0], rng)
    _check(tg, oracle_cpu, [x], [2], [0], [0], [1], rng)


def test_unaligned_views(tg, oracle_cpu):
    rng = np.random.default_rng(12)
    n = 30011
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    xbuf = torch.zeros(n + 3, device="cuda")
    dx = xbuf[3:3 + n]; dx.copy_(dev(x))
    size = tg.packed_size(n, 2)
    obuf = torch.zeros(size + 5, dtype=torch.uint8, device="cuda")
    out = obuf[1:1 + size]
    tg.encode([dx], [2], [1], [5], outs=[out])
    rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, 5)
    assert_bits_equal(host(out), ref, "message")
    assert host(obuf[:1]).tolist() == [0] and host(obuf[1 + size:]).tolist() == [0, 0, 0, 0]
    dbuf = torch.zeros(n + 1, device="cuda")
    tg.decode([out], [dbuf[1:]], [0])
    rc, dref = oracle_cpu.terngrad_decode(ref, n)
    assert_bits_equal(host(dbuf[1:]), dref, "decoded")


def test_invalid_bitwidth_paths(tg):
    x = dev(np.arange(16, dtype=np.float32))
    out = torch.zeros(26, dtype=torch.uint8, device="cuda")
    tg.encode([x], [3], [0], [0], outs=[out], expect_rc=-1)       # terngrad_body.h:207-212
    assert int(out.sum()) == 0
    # a header whose bitwidth byte is invalid decodes to nothing and is reported
    bad = torch.zeros(14, dtype=torch.uint8, device="cuda"); bad[0] = 3
    dst = torch.full((16,), 7.0, device="cuda")
    tg.decode([bad], [dst], [0])
    assert tg.status() == -1
    assert bool((dst == 7.0).all())
    assert tg.status() == 0   # the flag is cleared once reported


def test_full_size_config2_properties(tg):
    # 25,557,032 elements (ResNet-50), 0.1% outliers at +-50 sigma: size-independent properties
    n = 25_557_032
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(n, device="cuda", generator=gen) * 1e-2
    pos = torch.randperm(n, device="cuda", generator=gen)[: n // 1000]
    x[pos] = torch.where(torch.rand(pos.numel(), device="cuda", generator=gen) < 0.5, 0.5, -0.5)
    out = tg.encode([x], [2], [1], [0])[0]
    dec = torch.empty(n, device="cuda")
    tg.decode([out], [dec], [0])
    torch.cuda.synchronize()
    hdr = host(out[:10])
    assert hdr[0] == 2 and hdr[1] == 0
    mn, mx = hdr[2:6].view(np.float32)[0], hdr[6:10].view(np.float32)[0]
    assert mn == float(x.min()) and mx == float(x.max())
    gap = (float(mx) - float(mn)) / 3
    err = (dec.double() - x.double()).abs()
    assert float(err.max()) <= gap * (1 + 1e-4) + 1e-7        # stochastic rounding moves at most one level
    assert abs(float((dec.double() - x.double()).mean())) < gap * 2e-3   # and is unbiased
    levels = torch.unique(dec)
    assert levels.numel() <= 4
    # the oracle handles the full size in about a second: bit-exact message and decode
    from oracle import cpu
    xh = host(x)
    rc, ref = cpu.terngrad_encode(xh, 2, 1, 0)
    assert rc == 0
    assert_bits_equal(host(out), ref, "full-size message")
    rc, dref = cpu.terngrad_decode(ref, n)
    assert_bits_equal(host(dec), dref, "full-size decode")


@pytest.mark.parametrize("n", [7, 4096, 10007, 300001])
def test_several_messages_into_one_tensor(tg, oracle_cpu, n):
    # the root's gather-decode (hp_cuda.cpp:421-439): every gathered message names the same output tensor
    rng = np.random.default_rng(n)
    msgs = []
    for k, b in enumerate([2, 2, 1, 4, 8, 2, 2]):
        x = rng.normal(0, 1e-2 * (k + 1), n).astype(np.float32)
        rc, m = oracle_cpu.terngrad_encode(x, b, 1, 1000 + k)
        assert rc == 0
        msgs.append(m)
    dm = [dev(m) for m in msgs]
    for adds in ([1] * 7, [0] + [1] * 6, [1, 1, 0, 1, 1, 1, 1], [0] * 7):
        base = rng.normal(0, 1, n).astype(np.float32)
        out = dev(base)
        tg.decode(dm, [out] * 7, adds)
        torch.cuda.synchronize()
        ref = base.copy()
        for m, add in zip(msgs, adds):
            rc, ref = oracle_cpu.terngrad_decode(m, n, ref, add)
        assert_bits_equal(host(out), ref, f"accumulated n={n} adds={adds}")
    assert tg.status() == 0


@pytest.mark.parametrize("n", [4095, 4096, 8192 + 3, 16384, 5 * 16384 + 4096 + 17, 1_000_003])
@pytest.mark.parametrize("count", [2, 7, 8, 9])
def test_several_two_bit_messages_into_one_tensor(tg, oracle_cpu, n, count):
    # the configuration the reference ships with (2-bit messages): whole sub-tiles of 4096 elements take the
    # decoder's pipelined path when there are at most 8 messages; offsets make the payloads start at odd addresses
    rng = np.random.default_rng(1000 * count + n % 997)
    msgs, dm = [], []
    for k in range(count):
        x = rng.normal(0, 1e-2 * (k + 1), n).astype(np.float32)
        rc, m = oracle_cpu.terngrad_encode(x, 2, 1, 500 + k)
        assert rc == 0
        msgs.append(m)
        buf = torch.zeros(m.size + 8, dtype=torch.uint8, device="cuda")
        view = buf[k % 5:k % 5 + m.size]
        view.copy_(dev(m))
        dm.append(view)
    for adds in ([1] * count, [0] + [1] * (count - 1), [1] + [0] + [1] * (count - 2)):
        base = rng.normal(0, 1, n).astype(np.float32)
        out = dev(base)
        tg.decode(dm, [out] * count, adds)
        torch.cuda.synchronize()
        ref = base.copy()
        for m, add in zip(msgs, adds):
            rc, ref = oracle_cpu.terngrad_decode(m, n, ref, add)
        assert_bits_equal(host(out), ref, f"accumulated n={n} count={count} adds={adds}")
    assert tg.status() == 0


@pytest.mark.parametrize("ntensors,slots,first_add", [(3, 7, 1), (161, 7, 1), (208, 3, 0), (209, 3, 1), (4, 32, 1), (4, 33, 1)])
def test_messages_at_a_fixed_distance(tg, oracle_cpu, ntensors, slots, first_add):
    # The gathered slots of the reference's communication buffer: the messages of a tensor lie at one distance from
    # each other and have one size.  Up to 208 tensors with up to 32 such messages each are one launch with a
    # 40-byte table entry per tensor; one tensor or message more, and the call takes the general table again.
    rng = np.random.default_rng(ntensors * 100 + slots)
    sizes = [int(v) for v in rng.integers(1, 9000, ntensors)]
    sizes[0] = 5 * 16384 + 4096 + 17
    outs, refs, keep, ins, souts, adds = [], [], [], [], [], []
    for t, n in enumerate(sizes):
        nb = 10 + (n + 3) // 4
        slot = nb + int(rng.integers(0, 7))                       # distance between this tensor's messages
        buf = np.zeros(slot * slots + 3, np.uint8)
        base = rng.normal(0, 1, n).astype(np.float32)
        ref = base.copy()
        for k in range(slots):
            x = rng.normal(0, 1e-2 * (k + 1), n).astype(np.float32)
            rc, m = oracle_cpu.terngrad_encode(x, 2, 1, 7000 + 31 * t + k)
            assert rc == 0 and m.size == nb
            buf[1 + k * slot:1 + k * slot + nb] = m
            rc, ref = oracle_cpu.terngrad_decode(m, n, ref, 1 if (k or first_add) else 0)
        db = dev(buf)
        keep.append(db)
        out = dev(base)
        outs.append(out); refs.append(ref)
        for k in range(slots):
            ins.append(db[1 + k * slot:1 + k * slot + nb]); souts.append(out); adds.append(1 if (k or first_add) else 0)
    order = [t * slots + k for k in range(slots) for t in range(ntensors)]   # slot k of every tensor, then slot k + 1
    tg.decode([ins[i] for i in order], [souts[i] for i in order], [adds[i] for i in order])
    torch.cuda.synchronize()
    for t in range(ntensors):
        assert_bits_equal(host(outs[t]), refs[t], f"tensor {t} of {ntensors}, n={sizes[t]}, {slots} messages")
    assert tg.status() == 0


@pytest.mark.parametrize("size,own", [(8, 0), (8, 1), (8, 4), (8, 7), (3, 1), (2, 0), (4, 2)])
def test_gathered_slots_without_the_roots_own(tg, oracle_cpu, size, own):
    # What a root decodes (hp_cuda.cpp:421-439): the `size` slots of its piece of the communication buffer except
    # the one of its own rank, so the messages lie at one distance with one gap; also two gaps, which the
    # fixed-distance table does not describe and the general one takes.
    rng = np.random.default_rng(size * 10 + own)
    for gaps in ([own], [own, (own + 2) % size] if size >= 5 else [own]):
        sizes = [5 * 16384 + 4096 + 17, 77, 4096, 9001]
        keep, outs, refs, ins, souts = [], [], [], [], []
        for t, n in enumerate(sizes):
            nb = 10 + (n + 3) // 4
            slot = nb + int(rng.integers(0, 5))
            buf = np.zeros(slot * size + 2, np.uint8)
            base = rng.normal(0, 1, n).astype(np.float32)
            ref = base.copy()
            for k in range(size):
                rc, m = oracle_cpu.terngrad_encode(rng.normal(0, 1e-2 * (k + 1), n).astype(np.float32), 2, 1, 900 + 17 * t + k)
                assert rc == 0
                buf[k * slot:k * slot + nb] = m
                if k not in gaps:
                    rc, ref = oracle_cpu.terngrad_decode(m, n, ref, 1)
            db = dev(buf); keep.append(db)
            out = dev(base); outs.append(out); refs.append(ref)
            for k in range(size):
                if k not in gaps:
                    ins.append(db[k * slot:k * slot + nb]); souts.append(out)
        tg.decode(ins, souts, [1] * len(ins))
        torch.cuda.synchronize()
        for t in range(len(sizes)):
            assert_bits_equal(host(outs[t]), refs[t], f"tensor {t}, {size} slots without {gaps}")
    assert tg.status() == 0


def test_many_tensors_each_with_several_messages(tg, oracle_cpu):
    rng = np.random.default_rng(78)
    sizes = [int(s) for s in np.exp(rng.uniform(np.log(5), np.log(20000), 70))]
    slots = 40                                   # more than one segment of the slot table holds per tensor
    bases = [rng.normal(0, 1, n).astype(np.float32) for n in sizes]
    outs = [dev(b) for b in bases]
    call_outs, call_msgs, call_add, refs = [], [], [], [b.copy() for b in bases]
    for k in range(slots):
        for t, n in enumerate(sizes):
            rc, m = oracle_cpu.terngrad_encode(rng.normal(0, 1e-2, n).astype(np.float32), 2, 1, k * 1000 + t)
            call_outs.append(outs[t]); call_msgs.append(dev(m)); call_add.append(1)
            rc, refs[t] = oracle_cpu.terngrad_decode(m, n, refs[t], 1)
    tg.decode(call_msgs, call_outs, call_add)
    torch.cuda.synchronize()
    for t in range(len(sizes)):
        assert_bits_equal(host(outs[t]), refs[t], f"tensor {t}")


# ---- the single-launch resident encode (tensor kept on chip between the two passes) ----
@pytest.fixture
def resident_from_2m(capi):
    """By default only tensors of 5 * 2^20 elements and more take the resident encode; these tests want it at 2^21
    (and every tensor looked at on its own: the one-launch encode of a whole call has its own tests below)."""
    old = capi.set_option("terngrad_resident_min", 1 << 21)
    old_b = capi.set_option("terngrad_resident_bucket", 0)
    yield
    capi.set_option("terngrad_resident_min", old)
    capi.set_option("terngrad_resident_bucket", old_b)


@pytest.fixture
def resident_forced(capi):
    old = capi.set_option("terngrad_resident_min", 1)
    old_b = capi.set_option("terngrad_resident_bucket", 0)
    yield
    capi.set_option("terngrad_resident_min", old)
    capi.set_option("terngrad_resident_bucket", old_b)


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("rnd", [0, 1])
def test_resident_sizes_and_tails(tg, oracle_cpu, resident_forced, b, rnd):
    rng = np.random.default_rng(900 + 10 * b + rnd)
    unit = max(4, 8 // b)
    row = unit * 1024 * 256   # elements that one register row of a 256-CU grid covers
    sizes = [1, 2, 3, 5, 7, 8, 9, 17, 4097, 300007, row - 1, row, row + unit - 1, row + unit + 1, 2 * row + 13, 3 * row - 5]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    seeds = [int(s) for s in rng.integers(0, 2**63, len(sizes))]
    _check(tg, oracle_cpu, xs, [b] * len(sizes), [rnd] * len(sizes), seeds, [i & 1 for i in range(len(sizes))], rng)


def test_resident_constant_and_zero_tensors(tg, oracle_cpu, resident_forced):
    rng = np.random.default_rng(3)
    far = np.full(1_300_000, 0.5, np.float32); far[1_200_001] = -0.0; far[1_250_000] = 0.0   # first zero far from workgroup 0
    neg = np.full(2_100_001, -0.25, np.float32); neg[5] = 0.0; neg[2_000_000] = -0.0
    xs = [np.zeros(1000, np.float32), np.full(1003, -0.0, np.float32), np.full(4097, 0.125, np.float32),
          np.array([0.5, -0.0, 0.0, 0.25, 0.0], np.float32), np.array([-0.5, 0.0, -0.0, -0.25], np.float32),
          np.array([1e-45, 0, 3e-45, 2e-45] * 50, np.float32), far, neg]
    for b in (1, 2, 8):
        for rnd in (0, 1):
            _check(tg, oracle_cpu, xs, [b] * len(xs), [rnd] * len(xs), [77] * len(xs), [0] * len(xs), rng)


def test_resident_seed_edges_and_scalars(tg, oracle_cpu, resident_forced):
    rng = np.random.default_rng(41)
    x = rng.normal(0, 1e-2, 70001).astype(np.float32)
    seeds = [0, 2**32 - 1, 2**32 - 70001 // 4 + 5, 2**64 - 1]
    _check(tg, oracle_cpu, [x] * len(seeds), [2] * len(seeds), [1] * len(seeds), seeds, [0] * len(seeds), rng)
    xs, bws = [], []
    for k in range(60):
        lo = np.float32(rng.normal() * 10.0 ** rng.uniform(-30, 20))
        hi = np.float32(lo + abs(np.float32(rng.normal() * 10.0 ** rng.uniform(-38, 20))))
        v = rng.uniform(lo, hi, int(rng.integers(2, 40))).astype(np.float32)
        v[0], v[-1] = lo, hi
        xs.append(v)
        bws.append(int(rng.choice([1, 2, 4, 8])))
    _check(tg, oracle_cpu, xs, bws, [1] * len(xs), [int(s) for s in rng.integers(0, 2**63, len(xs))], [0] * len(xs), rng)


@pytest.mark.parametrize("b,n", [(2, 33_554_432), (1, 23_068_671), (1, 33_554_431), (4, 33_554_432 + 4096), (8, 29_000_003)])
def test_resident_capacity_edge(tg, oracle_cpu, b, n):
    # the largest tensors the chip holds (24 register rows + 8 LDS rows per lane; 14 + 8 at 1 bit with
    # stochastic rounding), and some just past it
    rng = np.random.default_rng(n % 1000 + b)
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    x[rng.integers(0, n, 1000)] = 0.0
    dx = dev(x)
    out = tg.encode([dx], [b], [1], [123456789])[0]
    rc, ref = oracle_cpu.terngrad_encode(x, b, 1, 123456789)
    assert rc == 0
    assert_bits_equal(host(out), ref, f"message n={n} b={b}")


@pytest.mark.parametrize("b,rnd,n", [(2, 1, 7_000_003), (2, 1, 13_631_489), (4, 0, 17_111_111), (2, 1, 24_000_001), (8, 1, 25_165_823),
                                     (2, 1, 25_165_824), (2, 0, 25_231_361)])
def test_resident_shares_between_one_row_and_the_register_rows(tg, oracle_cpu, resident_forced, b, rnd, n):
    # shares of 7 ... 24 rows per workgroup, not whole rows, and one that ends a few units into the first LDS row:
    # every wave holds a part of the share, the last waves a ragged one
    rng = np.random.default_rng(n % 1000 + b)
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    x[rng.integers(0, n, 1000)] = 0.0
    out = tg.encode([dev(x)], [b], [rnd], [987654321])[0]
    rc, ref = oracle_cpu.terngrad_encode(x, b, rnd, 987654321)
    assert rc == 0
    assert_bits_equal(host(out), ref, f"message n={n} b={b}")


@pytest.mark.parametrize("wgs", [1, 17, 63, 64, 65, 128, 200, 255])
def test_resident_launches_with_fewer_workgroups_than_cus(tg, oracle_cpu, capi, resident_forced, wgs):
    # the grid-wide exchange with a quarter that is partly filled, exactly filled, or empty; shares grow with
    # the smaller grid, so the sizes keep within what that many workgroups hold
    old = capi.set_option("terngrad_resident_workgroups", wgs)
    try:
        rng = np.random.default_rng(wgs)
        per_wg = 32 * 1024 * 4                                   # elements one workgroup can hold at 2 bits
        sizes = [max(5, min(3_000_001, wgs * per_wg - 7)), 100_003, 7]
        xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
        xs[0][rng.integers(0, sizes[0], 50)] = 0.0
        _check(tg, oracle_cpu, xs, [2, 2, 4], [1, 0, 1], [11, 12, 13], [0, 0, 0], rng)
        # and several tensors in one launch
        capi.set_option("terngrad_resident_bucket", 1)
        ys = [rng.normal(0, 1e-2, n).astype(np.float32) for n in (40_001, 90_000, 13, 70_007)]
        _check(tg, oracle_cpu, ys, [2] * 4, [1] * 4, [21, 22, 23, 24], [0] * 4, rng)
    finally:
        capi.set_option("terngrad_resident_workgroups", old)
        capi.set_option("terngrad_resident_bucket", 0)


def test_resident_and_tiled_tensors_in_one_call(tg, oracle_cpu, resident_from_2m):
    rng = np.random.default_rng(77)
    sizes = [3_000_001, 1000, 2_500_000, 70001, 2_097_152, 2_097_151]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    _check(tg, oracle_cpu, xs, [2, 4, 1, 8, 2, 2], [1, 0, 1, 1, 0, 1], [5, 6, 7, 8, 9, 10], [0] * len(sizes), rng)


def test_resident_barrier_expiry_is_repaired(tg, oracle_cpu, capi, resident_from_2m):
    # A zero bound makes the barrier wait give up at once: every workgroup still leaves normally and the
    # launch writes no message.  hpx_terngrad_encode_status then finds the expiry and encodes the SAME
    # call's tensor again through the two-launch path: the message of that call is valid when it returns,
    # as the reference's driver guarantees (hp_cuda_kernel.cu:30-65).  The stream keeps to the two-launch
    # path afterwards.
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1e-2, 3_000_000).astype(np.float32)
    y = rng.normal(0, 1e-2, 2_500_003).astype(np.float32)
    rc, ref_x = oracle_cpu.terngrad_encode(x, 2, 1, 9)
    rc, ref_y = oracle_cpu.terngrad_encode(y, 4, 1, 10)
    side = torch.cuda.Stream()
    # Only one stream per device may launch barrier kernels (the first that asks): forget the
    # workspaces so that the side stream becomes that stream here, and again afterwards so that the
    # stream of the other tests gets the resident path back.
    torch.cuda.synchronize()
    assert capi.load().hpx_release_workspaces() == 0
    old_ms = capi.set_option("terngrad_barrier_ms", 0)
    try:
        with torch.cuda.stream(side):
            dx, dy = dev(x), dev(y)
            assert tg.encode_status() == 0                     # nothing outstanding: returns at once
            out = torch.full((tg.packed_size(x.size, 2),), 0x5A, dtype=torch.uint8, device="cuda")
            tg.encode([dx], [2], [1], [9], outs=[out])
            assert tg.encode_status() == 0, capi.last_error()
            assert tg.repaired() == 1
            assert_bits_equal(host(out), ref_x, "the expired call's own message after the status call")
            capi.set_option("terngrad_barrier_ms", old_ms)
            out2 = tg.encode([dx], [2], [1], [9])[0]           # two-launch path from now on
            assert tg.encode_status() == 0 and tg.repaired() == 1
            side.synchronize()
            assert_bits_equal(host(out2), ref_x, "message after fallback")
        # The same without a status call in between: the next encode on the stream finds the expiry and
        # queues the repair before its own work.
        torch.cuda.synchronize()
        assert capi.load().hpx_release_workspaces() == 0
        capi.set_option("terngrad_barrier_ms", 0)
        with torch.cuda.stream(side):
            out = torch.full((tg.packed_size(x.size, 2),), 0x5A, dtype=torch.uint8, device="cuda")
            tg.encode([dx], [2], [1], [9], outs=[out])
            side.synchronize()
            capi.set_option("terngrad_barrier_ms", old_ms)
            out_y = tg.encode([dy], [4], [1], [10])[0]
            assert tg.repaired() == 1
            assert tg.encode_status() == 0, capi.last_error()
            assert_bits_equal(host(out), ref_x, "earlier call's message, repaired by the next encode")
            assert_bits_equal(host(out_y), ref_y, "the next encode's own message")
    finally:
        capi.set_option("terngrad_barrier_ms", old_ms)
        torch.cuda.synchronize()
        assert capi.load().hpx_release_workspaces() == 0


# ---- tensors larger than the chip: one launch keeps the head on chip and streams the rest twice ----
def _streamed_case(tg, oracle_cpu, capi, n, b, rnd, seed, expect_streamed=True):
    gen = torch.Generator(device="cuda").manual_seed(n % 1000 + b)
    x = torch.randn(n, device="cuda", generator=gen) * 1e-2
    x[n // 3] = 0.75; x[n - 5] = -0.625                       # extremes in the part kept on chip and in the streamed part
    L = capi.load()
    L.hpx_profile_reset(); L.hpx_profile_enable(1)
    try:
        out = tg.encode([x], [b], [rnd], [seed])[0]
        torch.cuda.synchronize()
        launches = capi.profile_query("terngrad_resident_streamed_kernel")[1]
    finally:
        L.hpx_profile_enable(0); L.hpx_profile_reset()
    assert launches == (1 if expect_streamed else 0), launches
    xh = host(x)
    rc, ref = oracle_cpu.terngrad_encode(xh, b, rnd, seed)
    assert rc == 0
    assert_bits_equal(host(out), ref, f"message n={n} b={b} rnd={rnd}")
    del xh, ref
    return x, out


@pytest.mark.parametrize("n", [40_000_000, 64_000_000, 102_760_448])
@pytest.mark.parametrize("b,rnd", [(2, 1), (2, 0), (8, 1), (8, 0)])
def test_tensors_larger_than_the_chip(tg, oracle_cpu, capi, n, b, rnd):
    # 102,760,448 elements is VGG-16's first fully connected layer
    x, out = _streamed_case(tg, oracle_cpu, capi, n, b, rnd, seed=7 + b)
    if n == 40_000_000:
        dec = torch.empty(n, device="cuda")
        tg.decode([out], [dec], [0])
        torch.cuda.synchronize()
        rc, dref = oracle_cpu.terngrad_decode(host(out), n)
        assert_bits_equal(host(dec), dref, "decode of the streamed encode's message")


@pytest.mark.parametrize("b,rnd,n", [(1, 1, 40_000_003), (1, 0, 50_000_001), (4, 1, 36_000_002), (4, 0, 34_000_001),
                                     (2, 1, 33_554_432 + 4096 + 3), (2, 1, 134_000_001), (1, 1, 23_100_007), (2, 0, 2**27 + 2**25 + 5)])
def test_streamed_encode_other_widths_ragged_ends_and_the_edges_of_its_range(tg, oracle_cpu, capi, b, rnd, n):
    # just above what the chip holds (a streamed part of a few rows, most workgroups without one), several times
    # what it holds, 1-bit codes with random rounding (fewer register rows: the chip holds 23 M), tails n % 8
    _streamed_case(tg, oracle_cpu, capi, n, b, rnd, seed=2**32 - 9)


def test_streamed_encode_zero_sign_and_switch(tg, oracle_cpu, capi):
    # a zero extreme takes the sign of the FIRST zero of the tensor, wherever it lies: in the streamed part only,
    # or in both parts; and the option that sends such tensors to the two-launch encode
    n = 36_000_000
    for first_zero, sign in ((35_900_017, -0.0), (1234, -0.0), (34_000_000, 0.0)):
        x = torch.rand(n, device="cuda") * 1e-2 + 1e-3            # all positive: the minimum is the zero
        x[first_zero] = sign
        x[35_999_999] = 0.0
        out = tg.encode([x], [2], [1], [11])[0]
        torch.cuda.synchronize()
        rc, ref = oracle_cpu.terngrad_encode(host(x), 2, 1, 11)
        assert_bits_equal(host(out), ref, f"first zero at {first_zero}")
    old = capi.set_option("terngrad_resident_streamed", 0)
    try:
        _streamed_case(tg, oracle_cpu, capi, 36_000_000, 2, 1, seed=3, expect_streamed=False)
    finally:
        capi.set_option("terngrad_resident_streamed", old)


def test_repair_leaves_the_buffers_of_finished_calls_alone(tg, oracle_cpu, capi, resident_from_2m):
    # Two single-launch encodes that finish well, no status call; their buffers are then overwritten, as a caller
    # whose allocator hands the memory on would.  A third encode's barrier expires.  The repair must encode the third
    # call's tensor only: the records of the first two were dropped when the third call found their events reached
    # with the expiry flag down.
    rng = np.random.default_rng(15)
    n = 3_000_000
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for _ in range(3)]
    refs = [oracle_cpu.terngrad_encode(x, 2, 1, 20 + i)[1] for i, x in enumerate(xs)]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    assert capi.load().hpx_release_workspaces() == 0
    prev = None
    try:
        with torch.cuda.stream(side):
            dxs = [dev(x) for x in xs]
            outs = [torch.full((tg.packed_size(n, 2),), 0x5A, dtype=torch.uint8, device="cuda") for _ in range(3)]
            for i in range(2):
                tg.encode([dxs[i]], [2], [1], [20 + i], outs=[outs[i]])
            side.synchronize()
            for i in range(2):
                assert_bits_equal(host(outs[i]), refs[i], f"message of good call {i}")
            # the caller reuses the memory of the finished calls
            outs[0].fill_(0x11); outs[1].fill_(0x22); dxs[0].zero_(); dxs[1].zero_()
            side.synchronize()
            prev = capi.set_option("terngrad_barrier_ms", 0)
            tg.encode([dxs[2]], [2], [1], [22], outs=[outs[2]])
            assert tg.encode_status() == 0, capi.last_error()
            capi.set_option("terngrad_barrier_ms", prev); prev = None
            assert tg.repaired() == 1                          # only the call whose barrier expired
            assert_bits_equal(host(outs[2]), refs[2], "the expired call's message after the repair")
            assert bool((outs[0] == 0x11).all()) and bool((outs[1] == 0x22).all()), "buffers of finished calls were written again"
    finally:
        if prev is not None:
            capi.set_option("terngrad_barrier_ms", prev)
        torch.cuda.synchronize()
        assert capi.load().hpx_release_workspaces() == 0


def test_release_stream_hands_the_resident_kernel_on(tg, oracle_cpu, capi, resident_from_2m):
    # The first stream that encodes a large tensor owns the barrier kernels; once it has been released
    # (as the scheduler's worker does before it destroys its stream) another stream gets them.
    rng = np.random.default_rng(8)
    x = rng.normal(0, 1e-2, 3_000_000).astype(np.float32)
    rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, 9)
    L = capi.load()
    torch.cuda.synchronize()
    assert L.hpx_release_workspaces() == 0
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    capi.load().hpx_profile_enable(1)
    try:
        def resident_launches():
            return capi.profile_query("terngrad_resident_kernel")[1]
        L.hpx_profile_reset()
        with torch.cuda.stream(a):
            dx = dev(x)
            out_a = tg.encode([dx], [2], [1], [9])[0]
            a.synchronize()
        assert resident_launches() == 1
        with torch.cuda.stream(b):
            out_b = tg.encode([dx], [2], [1], [9])[0]
            b.synchronize()
        assert resident_launches() == 1                       # b does not own them
        assert L.hpx_release_stream(a.cuda_stream) == 0
        with torch.cuda.stream(b):
            out_b2 = tg.encode([dx], [2], [1], [9])[0]
            b.synchronize()
        assert resident_launches() == 2                       # now it does
        for o, what in ((out_a, "owner"), (out_b, "other stream"), (out_b2, "new owner")):
            assert_bits_equal(host(o), ref, what)
    finally:
        L.hpx_profile_enable(0)
        L.hpx_profile_reset()
        torch.cuda.synchronize()
        assert L.hpx_release_workspaces() == 0


def test_calls_that_cannot_be_recorded_refuse_a_capturing_stream(tg, capi):
    # hpx_terngrad_encode tags its kernels per call and the GradDrop calls wait for the stream: recorded into a
    # graph they would replay stale tags / deadlock.  They return -3 instead; the capture itself ends cleanly.
    L = capi.load()
    c = capi
    x = torch.randn(70_001, device="cuda")
    r = torch.zeros_like(x)
    msg = torch.zeros(tg.packed_size(x.numel(), 2), dtype=torch.uint8, device="cuda")
    gd_out = torch.zeros(4 + 8 * 1024, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        tg.encode([x], [2], [1], [3], outs=[msg])          # eager once: workspaces exist
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            sp = torch.cuda.current_stream().cuda_stream
            tg.encode([x], [2], [1], [3], outs=[msg], expect_rc=-3)
            assert "captured" in capi.last_error()
            assert L.hpx_terngrad_encode_status(sp) == -3
            assert L.hpx_terngrad_decode_status(sp) == -3
            rc = L.hpx_gd_encode(1, c.ptr_array([x.data_ptr()]), c.i32_array([x.numel()]), c.ptr_array([r.data_ptr()]),
                                 c.ptr_array([gd_out.data_ptr()]), c.f64_array([0.05]), c.f64_array([0.99]), c.u64_array([1]), sp)
            assert rc == -3
            rc = L.hpx_gd_decode(1, c.ptr_array([gd_out.data_ptr()]), c.i32_array([gd_out.numel()]), c.ptr_array([r.data_ptr()]),
                                 c.i32_array([r.numel()]), c.i32_array([1]), sp)
            assert rc == -3
            r.add_(1.0)                                     # something recordable, so that the graph is not empty
    graph.replay()
    torch.cuda.synchronize()
    assert float(r[0]) == 1.0


def test_resident_kernel_belongs_to_one_stream(tg, oracle_cpu, capi, resident_from_2m):
    # A second stream encoding a large tensor takes the two-launch path (same bytes out).
    rng = np.random.default_rng(6)
    x = rng.normal(0, 1e-2, 3_000_000).astype(np.float32)
    rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, 9)
    dx = dev(x)
    L = capi.load()
    out0 = tg.encode([dx], [2], [1], [9])[0]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    L.hpx_profile_reset(); L.hpx_profile_enable(1)
    try:
        with torch.cuda.stream(side):
            out1 = tg.encode([dx], [2], [1], [9])[0]
            side.synchronize()
        assert capi.profile_query("terngrad_resident_kernel")[1] == 0
        assert capi.profile_query("terngrad_quant_kernel")[1] == 1
    finally:
        L.hpx_profile_enable(0); L.hpx_profile_reset()
    assert_bits_equal(host(out0), ref, "owning stream")
    assert_bits_equal(host(out1), ref, "second stream")


# ---- the resident encode of a whole call (several tensors in one launch) ----
@pytest.fixture
def bucket_forced(capi):
    """Every call with two or more tensors of one width and rounding mode takes the one-launch encode."""
    old = capi.set_option("terngrad_resident_min", 1)
    old_b = capi.set_option("terngrad_resident_bucket", 1)
    L = capi.load()
    L.hpx_profile_reset(); L.hpx_profile_enable(1)
    yield
    L.hpx_profile_enable(0); L.hpx_profile_reset()
    capi.set_option("terngrad_resident_min", old)
    capi.set_option("terngrad_resident_bucket", old_b)


def _bucket_launches(capi):
    return capi.profile_query("terngrad_resident_multi_kernel")[1]


@pytest.mark.parametrize("b", [1, 2, 4, 8])
@pytest.mark.parametrize("rnd", [0, 1])
def test_resident_bucket_sizes_and_tails(tg, oracle_cpu, capi, bucket_forced, b, rnd):
    rng = np.random.default_rng(1900 + 10 * b + rnd)
    unit = max(4, 8 // b)
    sizes = [1, 2, 3, 5, 7, 8, 9, 17, unit * 64 - 1, unit * 64, unit * 64 + 1, 4097, 300007, 64, 256, 2048, 70001, 1_000_003]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    seeds = [int(s) for s in rng.integers(0, 2**63, len(sizes))]
    before = _bucket_launches(capi)
    _check(tg, oracle_cpu, xs, [b] * len(sizes), [rnd] * len(sizes), seeds, [i & 1 for i in range(len(sizes))], rng)
    assert _bucket_launches(capi) == before + 1


def test_resident_bucket_zero_extremes_and_constants(tg, oracle_cpu, capi, bucket_forced):
    rng = np.random.default_rng(31)
    far = np.full(1_300_000, 0.5, np.float32); far[1_200_001] = -0.0; far[1_250_000] = 0.0   # first zero many pieces in
    neg = np.full(2_100_001, -0.25, np.float32); neg[5] = 0.0; neg[2_000_000] = -0.0
    xs = [np.zeros(1000, np.float32), np.full(1003, -0.0, np.float32), np.full(4097, 0.125, np.float32),
          np.array([0.5, -0.0, 0.0, 0.25, 0.0], np.float32), np.array([-0.5, 0.0, -0.0, -0.25], np.float32),
          np.array([1e-45, 0, 3e-45, 2e-45] * 50, np.float32), far, neg]
    for b in (1, 2, 8):
        for rnd in (0, 1):
            before = _bucket_launches(capi)
            _check(tg, oracle_cpu, xs, [b] * len(xs), [rnd] * len(xs), [77] * len(xs), [0] * len(xs), rng)
            assert _bucket_launches(capi) == before + 1


def test_resident_bucket_many_rows_and_full_table(tg, oracle_cpu, capi, bucket_forced):
    # 192 tensors (a full table) that need LDS rows as well: about 27 M elements
    rng = np.random.default_rng(32)
    sizes = [int(s) for s in rng.integers(1, 2000, 150)] + [int(s) for s in rng.integers(500_000, 800_000, 41)] + [27_000_000 - 41 * 650_000]
    assert len(sizes) == 192
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    dx = [dev(x) for x in xs]
    seeds = [int(s) for s in rng.integers(0, 2**64 - 1, len(sizes), dtype=np.uint64)]
    before = _bucket_launches(capi)
    outs = tg.encode(dx, [2] * len(xs), [1] * len(xs), seeds)
    torch.cuda.synchronize()
    assert _bucket_launches(capi) == before + 1
    for i, x in enumerate(xs):
        rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, seeds[i])
        assert rc == 0
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] n={x.size}")


def _resnet50_sizes():
    sizes = [64 * 3 * 7 * 7, 64, 64]
    inp = 64
    for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for blk in range(blocks):
            sizes += [planes * inp, planes, planes, planes * planes * 9, planes, planes, planes * 4 * planes, planes * 4, planes * 4]
            if blk == 0:
                sizes += [planes * 4 * inp, planes * 4, planes * 4]
            inp = planes * 4
    return sizes + [1000 * 2048, 1000]


@pytest.mark.parametrize("b,rnd", [(2, 1), (2, 0), (1, 1), (8, 1)])
def test_resident_bucket_of_resnet50s_tensors(tg, oracle_cpu, capi, bucket_forced, b, rnd):
    """The 161 parameter tensors of ResNet-50 (25 557 032 elements; 107 of them biases and normalisation parameters of
    at most 2048 elements, which the waves without a piece encode on their own) in one launch, every message against
    the oracle."""
    sizes = _resnet50_sizes()
    assert len(sizes) == 161 and sum(sizes) == 25_557_032
    rng = np.random.default_rng(3300 + b)
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    xs[1][:] = 0.0; xs[2][3] = -0.0; xs[2][7] = 0.0; xs[2] = np.abs(xs[2]); xs[2][3] = -0.0   # tiny tensors with zero extremes
    dx = [dev(x) for x in xs]
    seeds = [int(v) for v in rng.integers(0, 2**63, len(sizes))]
    before = _bucket_launches(capi)
    outs = tg.encode(dx, [b] * len(xs), [rnd] * len(xs), seeds)
    torch.cuda.synchronize()
    # (one bit with stochastic rounding keeps fewer rows in registers: the list then takes two launches)
    assert _bucket_launches(capi) == before + (2 if (b, rnd) == (1, 1) else 1)
    for i, x in enumerate(xs):
        rc, ref = oracle_cpu.terngrad_encode(x, b, rnd, seeds[i])
        assert rc == 0
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] n={x.size}")


def test_resident_bucket_of_nothing_but_tiny_tensors(tg, oracle_cpu, capi, bucket_forced):
    rng = np.random.default_rng(35)
    for b in (1, 2, 4, 8):
        unit = max(4, 8 // b)
        sizes = [1, unit - 1, unit, 63, 64, 1000, 2048, 8 * 64 * unit, 8 * 64 * unit - 1] + [int(v) for v in rng.integers(1, 8 * 64 * unit, 40)]
        xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
        before = _bucket_launches(capi)
        _check(tg, oracle_cpu, xs, [b] * len(xs), [1] * len(xs), [int(v) for v in rng.integers(0, 2**63, len(xs))], [0] * len(xs), rng)
        assert _bucket_launches(capi) == before + 1
        # one tensor just above the limit among them: the others ride on the waves it leaves free
        xs.append(rng.normal(0, 1e-2, 8 * 64 * unit + unit).astype(np.float32))
        _check(tg, oracle_cpu, xs, [b] * len(xs), [1] * len(xs), [int(v) for v in rng.integers(0, 2**63, len(xs))], [0] * len(xs), rng)


def test_resident_bucket_groups_of_a_large_call(tg, oracle_cpu, capi, bucket_forced):
    # 77 M elements: more than the chip holds, so the call becomes three resident launches (5 + 5 + 3 tensors);
    # then a call whose widths change half way: two launches
    capi.set_option("terngrad_resident_min", 10 << 20)
    rng = np.random.default_rng(34)
    sizes = [6_000_000 + int(d) for d in rng.integers(-3, 4, 11)] + [1000, 5_000_003]
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in sizes]
    dx = [dev(x) for x in xs]
    seeds = [int(s) for s in rng.integers(0, 2**63, len(sizes))]
    before = _bucket_launches(capi)
    outs = tg.encode(dx, [2] * len(xs), [1] * len(xs), seeds)
    torch.cuda.synchronize()
    assert _bucket_launches(capi) == before + 3
    for i, x in enumerate(xs):
        rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, seeds[i])
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] n={x.size}")
    # the same call again, then decoded: the launches of the second call wait for nothing they should not
    outs2 = tg.encode(dx, [2] * len(xs), [1] * len(xs), seeds)
    back = [torch.empty(x.size, device="cuda") for x in xs]
    tg.decode(outs2, back, [0] * len(xs))
    torch.cuda.synchronize()
    for i, x in enumerate(xs):
        rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, seeds[i])
        assert_bits_equal(host(outs2[i]), ref, f"second call, message[{i}]")
        rc, dec = oracle_cpu.terngrad_decode(ref, x.size)
        assert_bits_equal(host(back[i]), dec, f"decoded[{i}]")
    bws = [2, 2, 2, 4, 4, 4]
    before = _bucket_launches(capi)
    outs = tg.encode(dx[:6], bws, [1] * 6, seeds[:6])
    torch.cuda.synchronize()
    assert _bucket_launches(capi) == before + 2
    for i in range(6):
        rc, ref = oracle_cpu.terngrad_encode(xs[i], bws[i], 1, seeds[i])
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] b={bws[i]}")
    # a group too small for the threshold between two that reach it: tiled kernels for that one, same bytes
    bws = [2, 2, 4, 2, 2]
    sz = [0, 1, 11, 2, 3]                       # tensor 11 has 1000 elements
    before = _bucket_launches(capi)
    outs = tg.encode([dx[k] for k in sz], bws, [1] * 5, [seeds[k] for k in sz])
    torch.cuda.synchronize()
    assert _bucket_launches(capi) == before + 2
    for i, k in enumerate(sz):
        rc, ref = oracle_cpu.terngrad_encode(xs[k], bws[i], 1, seeds[k])
        assert_bits_equal(host(outs[i]), ref, f"message[{i}] b={bws[i]}")


def test_resident_bucket_barrier_expiry_is_repaired(tg, oracle_cpu, capi, bucket_forced):
    # As for the single-tensor kernel: with a zero bound every workgroup gives up at the barrier and leaves; the
    # status call encodes all tensors of that launch again, and the stream keeps to the tiled kernels afterwards.
    rng = np.random.default_rng(35)
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in (1_500_000, 70_001, 900_000)]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    assert capi.load().hpx_release_workspaces() == 0       # the side stream becomes the owner of the barrier kernels
    old_ms = capi.set_option("terngrad_barrier_ms", 0)
    try:
        with torch.cuda.stream(side):
            dx = [dev(x) for x in xs]
            before = _bucket_launches(capi)
            outs = [torch.full((tg.packed_size(x.size, 2),), 0x5A, dtype=torch.uint8, device="cuda") for x in xs]
            tg.encode(dx, [2] * 3, [1] * 3, [9, 10, 11], outs=outs)
            assert tg.encode_status() == 0, capi.last_error()
            assert _bucket_launches(capi) == before + 1 and tg.repaired() == 3
            for i, x in enumerate(xs):
                rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, 9 + i)
                assert_bits_equal(host(outs[i]), ref, f"message[{i}] of the expired call")
            capi.set_option("terngrad_barrier_ms", old_ms)
            outs = tg.encode(dx, [2] * 3, [1] * 3, [9, 10, 11])
            side.synchronize()
            assert _bucket_launches(capi) == before + 1
            for i, x in enumerate(xs):
                rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, 9 + i)
                assert_bits_equal(host(outs[i]), ref, f"message[{i}] after fallback")
    finally:
        capi.set_option("terngrad_barrier_ms", old_ms)
        torch.cuda.synchronize()
        assert capi.load().hpx_release_workspaces() == 0


def test_resident_bucket_falls_back(tg, oracle_cpu, capi, bucket_forced):
    rng = np.random.default_rng(33)
    xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in (5000, 70001, 1234)]
    before = _bucket_launches(capi)
    # alternating widths or rounding modes: no two neighbours can share a launch
    _check(tg, oracle_cpu, xs, [2, 4, 2], [1, 1, 1], [1, 2, 3], [0, 0, 0], rng)
    _check(tg, oracle_cpu, xs, [2, 2, 2], [1, 0, 1], [1, 2, 3], [0, 0, 0], rng)
    assert _bucket_launches(capi) == before
    # more tensors than one table holds: 192 in one launch, the last one on its own
    many = [rng.normal(0, 1e-2, 300).astype(np.float32) for _ in range(193)]
    _check(tg, oracle_cpu, many, [2] * 193, [1] * 193, list(range(193)), [0] * 193, rng)
    assert _bucket_launches(capi) == before + 1
    before += 1
    # below the threshold
    capi.set_option("terngrad_resident_min", 1 << 20)
    _check(tg, oracle_cpu, xs, [2, 2, 2], [1, 1, 1], [1, 2, 3], [0, 0, 0], rng)
    assert _bucket_launches(capi) == before
    capi.set_option("terngrad_resident_min", 1)
    _check(tg, oracle_cpu, xs, [2, 2, 2], [1, 1, 1], [1, 2, 3], [0, 0, 0], rng)
    assert _bucket_launches(capi) == before + 1


def test_random_sweep_of_calls(tg, oracle_cpu, capi):
    # seeded sweep over sizes, widths, rounding modes, seeds and call shapes; the threshold for the resident
    # encode is lowered so that about half of the tensors take it
    rng = np.random.default_rng(2024)
    old = capi.set_option("terngrad_resident_min", 300_000)
    try:
        for call in range(12):
            count = int(rng.integers(1, 7))
            sizes = [int(np.exp(rng.uniform(np.log(1), np.log(3_000_000)))) for _ in range(count)]
            xs = []
            for n in sizes:
                kind = int(rng.integers(0, 4))
                x = rng.normal(0, 10.0 ** rng.uniform(-6, 2), n).astype(np.float32)
                if kind == 1:
                    x = np.abs(x)                       # minimum may be a zero
                    x[rng.integers(0, n, max(1, n // 50))] = 0.0
                elif kind == 2:
                    x[rng.integers(0, n, max(1, n // 3))] = -0.0
                elif kind == 3:
                    x = np.round(x / x.std() * 2).astype(np.float32) if n > 1 and x.std() > 0 else x
                xs.append(x)
            bws = [int(b) for b in rng.choice([1, 2, 4, 8], count)]
            rnds = [int(r) for r in rng.integers(0, 2, count)]
            seeds = [int(s) for s in rng.integers(0, 2**64 - 1, count, dtype=np.uint64)]
            _check(tg, oracle_cpu, xs, bws, rnds, seeds, [int(a) for a in rng.integers(0, 2, count)], rng)
    finally:
        capi.set_option("terngrad_resident_min", old)
