"""GPU parity: TBQ encode/decode through the C ABI vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from gpu_util import Tbq, assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tbq(capi):
    assert torch.cuda.is_available()
    return Tbq(capi)


def _roundtrip(tbq, oracle_cpu, gs, rs, thrs, adds, rng):
    dg = [dev(g) for g in gs]
    dr = [dev(r) for r in rs]
    packed = tbq.encode(dg, dr, thrs)
    torch.cuda.synchronize()
    for i, (g, r, thr) in enumerate(zip(gs, rs, thrs)):
        r_ref = r.copy()
        p_ref = oracle_cpu.tbq_encode(g, r_ref, thr)
        assert_bits_equal(host(packed[i]), p_ref, f"packed[{i}] n={g.size}")
        assert_bits_equal(host(dr[i]), r_ref, f"residual[{i}] n={g.size}")
        assert_bits_equal(host(dg[i]), g, f"gradient[{i}] must be untouched")
    bases = [rng.normal(0, 1, g.size).astype(np.float32) for g in gs]
    douts = [dev(b) for b in bases]
    tbq.decode(packed, douts, thrs, adds)
    torch.cuda.synchronize()
    for i, (g, thr, add) in enumerate(zip(gs, thrs, adds)):
        ref = oracle_cpu.tbq_decode(host(packed[i]), g.size, thr, bases[i].copy(), add)
        assert_bits_equal(host(douts[i]), ref, f"decoded[{i}] n={g.size} add={add}")


def test_known_answer(tbq, oracle_cpu):
    g = np.array([.003, -.003, .001, -.001, .002, -.002, 0, .0041, .5, -.5], np.float32)
    dr = dev(np.zeros(10, np.float32))
    packed = tbq.encode([dev(g)], [dr], [0.002])
    torch.cuda.synchronize()
    assert host(packed[0]).tolist() == [82, 146, 82]
    out = dev(np.zeros(10, np.float32))
    tbq.decode(packed, [out], [0.002], [0])
    np.testing.assert_array_equal(host(out), np.array([.002, -.002, 0, 0, .002, -.002, 0, .002, .002, -.002], np.float32))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 255, 4095, 4096, 4097, 4099, 8191, 1 << 20, (1 << 20) + 1, 3000001])
def test_single_tensor_sizes(tbq, oracle_cpu, n):
    rng = np.random.default_rng(n)
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    r = rng.normal(0, 1e-3, n).astype(np.float32)
    for add in (0, 1):
        _roundtrip(tbq, oracle_cpu, [g], [r], [2e-3], [add], rng)


def test_config1_zero_residual(tbq, oracle_cpu):
    # 1,048,576 elements ~N(0,1e-3), threshold 2e-3, zero residual, seed 0
    rng = np.random.default_rng(0)
    g = rng.normal(0, 1e-3, 1 << 20).astype(np.float32)
    _roundtrip(tbq, oracle_cpu, [g], [np.zeros_like(g)], [2e-3], [0], rng)


def test_special_values(tbq, oracle_cpu):
    rng = np.random.default_rng(5)
    thr = np.float32(2e-3)
    g = np.array([thr, -thr, np.nextafter(thr, 0), -np.nextafter(thr, 0), 0.0, -0.0, 1e-45, -1e-45, 1e30, -1e30,
                  3 * thr, -3 * thr, 1.5e-3, -1.5e-3, 7.0], np.float32)
    r = np.array([0, 0, 0, 0, thr, -thr, 0, 0, 0, 0, 0, 0, 1e-3, -1e-3, -7.0], np.float32)
    _roundtrip(tbq, oracle_cpu, [g], [r], [float(thr)], [1], rng)
    # zero and negative thresholds follow the same comparisons
    _roundtrip(tbq, oracle_cpu, [g], [r], [0.0], [0], rng)
    _roundtrip(tbq, oracle_cpu, [g], [r], [-1e-3], [0], rng)


def test_unaligned_views(tbq, oracle_cpu):
    # tensors that start at an odd element / odd byte of their allocation
    rng = np.random.default_rng(9)
    n = 10007
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    r = rng.normal(0, 1e-3, n).astype(np.float32)
    gbuf = torch.zeros(n + 3, device="cuda"); rbuf = torch.zeros(n + 3, device="cuda")
    obuf = torch.zeros((n + 3) // 4 + 3, dtype=torch.uint8, device="cuda")
    dg, dr, do = gbuf[1:1 + n], rbuf[3:3 + n], obuf[3:3 + (n + 3) // 4]
    dg.copy_(dev(g)); dr.copy_(dev(r))
    tbq.encode([dg], [dr], [2e-3], outs=[do])
    torch.cuda.synchronize()
    r_ref = r.copy()
    p_ref = oracle_cpu.tbq_encode(g, r_ref, 2e-3)
    assert_bits_equal(host(do), p_ref, "packed")
    assert_bits_equal(host(dr), r_ref, "residual")
    assert host(obuf[:3]).tolist() == [0, 0, 0] and float(rbuf[:3].abs().sum()) == 0.0
    out = torch.zeros(n + 1, device="cuda")
    tbq.decode([do], [out[1:]], [2e-3], [0])
    assert_bits_equal(host(out[1:]), oracle_cpu.tbq_decode(p_ref, n, 2e-3), "decoded")
    assert float(out[0]) == 0.0


def test_tiles_on_address_boundaries(tbq, oracle_cpu):
    # Workgroup tiles start on 16 KiB address boundaries; the groups before the first boundary form a short
    # first tile.  Tensors that start at chosen distances from a boundary, with sizes around the first
    # tile's length, must encode and decode as anywhere else; all of them go out in one call.
    rng = np.random.default_rng(21)
    thr = 2e-3
    span = 3 * 4096 + 64
    gs, rs, views_g, views_r, views_o, views_d, bases = [], [], [], [], [], [], []
    for off in (0, 4, 2048, 4092, 4095, 1, 3073):          # elements past a 16 KiB boundary
        to_boundary = (-(off * 4)) % 16384
        head = (to_boundary + 15) // 16                     # groups before the first boundary
        for n in sorted({1, 3, 4, 5, max(1, 4 * head - 1), 4 * head, 4 * head + 1, 4 * head + 3, 4 * head + 4,
                         4 * head + 4096, 4 * head + 4097, 4 * head + 2 * 4096 + 2}):
            if n > span - 8 or n < 1:
                continue
            gbuf = torch.zeros(4096 * 2 + span, device="cuda")
            rbuf = torch.zeros(4096 * 2 + span, device="cuda")
            dbuf = torch.zeros(4096 * 2 + span, device="cuda")
            obuf = torch.full(((span + 3) // 4 + 8,), 0xAA, dtype=torch.uint8, device="cuda")
            # first element of the view sits `off` elements past a 16 KiB boundary of ITS buffer's address
            def view(buf, n_):
                skip = ((-buf.data_ptr()) % 16384) // 4 + off
                return buf[skip:skip + n_]
            g = rng.normal(0, 2e-3, n).astype(np.float32)
            r = rng.normal(0, 1e-3, n).astype(np.float32)
            b = rng.normal(0, 1, n).astype(np.float32)
            vg, vr, vd = view(gbuf, n), view(rbuf, n), view(dbuf, n)
            vg.copy_(dev(g)); vr.copy_(dev(r)); vd.copy_(dev(b))
            gs.append(g); rs.append(r); bases.append(b)
            views_g.append(vg); views_r.append(vr); views_d.append(vd); views_o.append(obuf[5:5 + (n + 3) // 4])
    tbq.encode(views_g, views_r, [thr] * len(gs), outs=views_o)
    adds = [i % 2 for i in range(len(gs))]
    tbq.decode(views_o, views_d, [thr] * len(gs), adds)
    torch.cuda.synchronize()
    for i, (g, r) in enumerate(zip(gs, rs)):
        r_ref = r.copy()
        p_ref = oracle_cpu.tbq_encode(g, r_ref, thr)
        assert_bits_equal(host(views_o[i]), p_ref, f"packed, case {i} n={g.size}")
        assert_bits_equal(host(views_r[i]), r_ref, f"residual, case {i} n={g.size}")
        assert_bits_equal(host(views_d[i]), oracle_cpu.tbq_decode(p_ref, g.size, thr, bases[i].copy(), adds[i]),
                          f"decoded, case {i} n={g.size} add={adds[i]}")


def test_bucket_of_many_tensors(tbq, oracle_cpu):
    # More tensors than one launch table holds, ragged sizes, per-tensor thresholds,
    # an empty tensor in the middle; two consecutive steps exercise residual feedback.
    rng = np.random.default_rng(1)
    sizes = [int(s) for s in np.exp(rng.uniform(np.log(3), np.log(30000), 600))]
    sizes[17] = 0
    gs = [rng.normal(0, 5e-3, n).astype(np.float32) for n in sizes]
    rs = [np.zeros(n, np.float32) for n in sizes]
    thrs = [float(np.float32(rng.uniform(5e-3, 2e-2))) for _ in sizes]
    dg = [dev(g) if g.size else torch.empty(0, device="cuda") for g in gs]
    dr = [dev(r) if r.size else torch.empty(0, device="cuda") for r in rs]
    for step in range(2):
        packed = tbq.encode(dg, dr, thrs)
        torch.cuda.synchronize()
        for i, n in enumerate(sizes):
            p_ref = oracle_cpu.tbq_encode(gs[i], rs[i], thrs[i])
            assert_bits_equal(host(packed[i]), p_ref, f"step {step} packed[{i}] n={n}")
            assert_bits_equal(host(dr[i]), rs[i], f"step {step} residual[{i}] n={n}")
    outs = [torch.zeros(n, device="cuda") for n in sizes]
    tbq.decode(packed, outs, thrs, [i & 1 for i in range(len(sizes))])
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        assert_bits_equal(host(outs[i]), oracle_cpu.tbq_decode(host(packed[i]), n, thrs[i]), f"decoded[{i}]")


def test_full_size_bucket_two_steps(tbq):
    # 110M-element bucket (BERT-base-like): size-independent properties, then all 200 tensors against the oracle.
    rng = np.random.default_rng(0)
    sizes = np.exp(rng.uniform(np.log(768), np.log(3e7), 200))
    sizes = np.clip(np.floor(sizes * 110e6 / sizes.sum()), 768, 3e7).astype(np.int64)
    sizes[np.argmax(sizes)] += 110_000_000 - sizes.sum()
    assert sizes.sum() == 110_000_000
    thr = 1e-2
    gen = torch.Generator(device="cuda").manual_seed(0)
    gs = [torch.randn(int(n), device="cuda", generator=gen) * 5e-3 for n in sizes]
    rs = [torch.zeros(int(n), device="cuda") for n in sizes]
    g_sum = [float(g.double().sum()) for g in gs[:5]]
    packed = tbq.encode(gs, rs, [thr] * len(gs))
    outs = [torch.empty(int(n), device="cuda") for n in sizes]
    tbq.decode(packed, outs, [thr] * len(gs), [0] * len(gs))
    torch.cuda.synchronize()
    t = torch.tensor(thr, dtype=torch.float32, device="cuda")
    for i in (0, 1, 2, int(np.argmax(sizes)), len(gs) - 1):
        g, r, o = gs[i], rs[i], outs[i]
        # decode takes only the values {-thr, 0, thr}; decode + residual == gradient (residual started at 0)
        assert bool(((o == 0) | (o == t) | (o == -t)).all())
        assert float((o.double() + r.double() - g.double()).abs().max()) < 1e-9
        small = g.abs() < 2 * t - 1e-7
        assert bool((r[small].abs() < t).all())
        codes = packed[i]
        assert int(((codes >> 0) & 3 == 3).sum() + ((codes >> 2) & 3 == 3).sum()) == 0
    assert [float(g.double().sum()) for g in gs[:5]] == g_sum  # gradients untouched
    # Two consecutive steps, every one of the 200 tensors bit-exact against the oracle: packed bytes, residual
    # (the second step starts from the first one's residuals: the error feedback at full size) and decoded tensor.
    from oracle import cpu
    r_host = [np.zeros(int(n), np.float32) for n in sizes]
    for step in range(2):
        if step == 1:
            gs = [torch.randn(int(n), device="cuda", generator=gen) * 5e-3 for n in sizes]
            packed = tbq.encode(gs, rs, [thr] * len(gs))
            tbq.decode(packed, outs, [thr] * len(gs), [0] * len(gs))
            torch.cuda.synchronize()
        for i in range(len(gs)):
            gh = host(gs[i])
            p_ref = cpu.tbq_encode(gh, r_host[i], thr)
            assert_bits_equal(host(packed[i]), p_ref, f"step {step} bucket packed[{i}]")
            assert_bits_equal(host(rs[i]), r_host[i], f"step {step} bucket residual[{i}]")
            assert_bits_equal(host(outs[i]), cpu.tbq_decode(p_ref, gh.size, thr), f"step {step} bucket decoded[{i}]")


@pytest.mark.parametrize("n", [7, 4096, 10007, 300001])
def test_several_messages_into_one_tensor(tbq, oracle_cpu, n):
    # the root's gather-decode (hp_cuda.cpp:241-259): every gathered message names the same output tensor
    rng = np.random.default_rng(n)
    msgs, thrs = [], []
    for k in range(7):
        thr = float(np.float32(rng.uniform(1e-3, 5e-3)))
        g = rng.normal(0, 2e-3, n).astype(np.float32)
        msgs.append(oracle_cpu.tbq_encode(g, np.zeros(n, np.float32), thr))
        thrs.append(thr)
    dm = [dev(m) for m in msgs]
    for adds in ([1] * 7, [0] + [1] * 6, [1, 1, 0, 1, 1, 1, 1], [0] * 7):
        base = rng.normal(0, 1, n).astype(np.float32)
        out = dev(base)
        tbq.decode(dm, [out] * 7, thrs, adds)
        torch.cuda.synchronize()
        ref = base.copy()
        for m, thr, add in zip(msgs, thrs, adds):      # one message after the other, as the reference applies them
            ref = oracle_cpu.tbq_decode(m, n, thr, ref, add)
        assert_bits_equal(host(out), ref, f"accumulated n={n} adds={adds}")


@pytest.mark.parametrize("ntensors,slots,first_add", [(3, 7, 1), (200, 7, 1), (208, 3, 0), (209, 3, 1), (5, 32, 1), (5, 33, 1)])
def test_messages_at_a_fixed_distance(tbq, oracle_cpu, ntensors, slots, first_add):
    # The gathered slots of the reference's communication buffer: the messages of a tensor lie at one distance from
    # each other and share the tensor's threshold.  Up to 208 tensors with up to 32 such messages each are one
    # launch with a 40-byte table entry per tensor; one tensor or message more, and the call takes the general
    # table again.  Odd slot sizes, so that messages start at any byte.
    rng = np.random.default_rng(ntensors * 100 + slots)
    sizes = [int(v) for v in rng.integers(1, 9000, ntensors)]
    sizes[0] = 3 * 4096 + 1027
    outs, refs, dms, thrs, ins, adds, souts = [], [], [], [], [], [], []
    for t, n in enumerate(sizes):
        thr = float(np.float32(rng.uniform(1e-3, 5e-3)))
        slot = (n + 3) // 4 + int(rng.integers(0, 7))                      # distance between this tensor's messages
        buf = np.zeros(slot * slots + 3, np.uint8)
        base = rng.normal(0, 1, n).astype(np.float32)
        ref = base.copy()
        for k in range(slots):
            g = rng.normal(0, 2e-3, n).astype(np.float32)
            m = oracle_cpu.tbq_encode(g, np.zeros(n, np.float32), thr)
            buf[1 + k * slot:1 + k * slot + m.size] = m
            ref = oracle_cpu.tbq_decode(m, n, thr, ref, 1 if (k or first_add) else 0)
        db = dev(buf)
        dms.append(db)
        out = dev(base)
        outs.append(out); refs.append(ref)
        for k in range(slots):
            ins.append(db[1 + k * slot:1 + k * slot + (n + 3) // 4]); souts.append(out); thrs.append(thr)
            adds.append(1 if (k or first_add) else 0)
    # messages of different tensors interleaved, as the scheduler's batches hand them over: slot k of every tensor, then slot k + 1
    order = [t * slots + k for k in range(slots) for t in range(ntensors)]
    tbq.decode([ins[i] for i in order], [souts[i] for i in order], [thrs[i] for i in order], [adds[i] for i in order])
    torch.cuda.synchronize()
    for t in range(ntensors):
        assert_bits_equal(host(outs[t]), refs[t], f"tensor {t} of {ntensors}, n={sizes[t]}, {slots} messages")


@pytest.mark.parametrize("size,own", [(8, 0), (8, 1), (8, 4), (8, 7), (3, 1), (2, 0), (4, 2)])
def test_gathered_slots_without_the_roots_own(tbq, oracle_cpu, size, own):
    # What a root decodes (hp_cuda.cpp:241-259): the `size` slots of its piece of the communication buffer except
    # the one of its own rank, so the messages lie at one distance with one gap; also two gaps, which the
    # fixed-distance table does not describe and the general one takes.
    rng = np.random.default_rng(size * 10 + own)
    for gaps in ([own], [own, (own + 2) % size] if size >= 5 else [own]):
        sizes = [3 * 4096 + 1027, 77, 4096, 9001]
        keep, outs, refs, ins, souts, thrs = [], [], [], [], [], []
        for n in sizes:
            thr = float(np.float32(rng.uniform(1e-3, 5e-3)))
            slot = (n + 3) // 4 + int(rng.integers(0, 5))
            buf = np.zeros(slot * size + 2, np.uint8)
            base = rng.normal(0, 1, n).astype(np.float32)
            ref = base.copy()
            for k in range(size):
                m = oracle_cpu.tbq_encode(rng.normal(0, 2e-3, n).astype(np.float32), np.zeros(n, np.float32), thr)
                buf[k * slot:k * slot + m.size] = m
                if k not in gaps:
                    ref = oracle_cpu.tbq_decode(m, n, thr, ref, 1)
            db = dev(buf); keep.append(db)
            out = dev(base); outs.append(out); refs.append(ref)
            for k in range(size):
                if k not in gaps:
                    ins.append(db[k * slot:k * slot + (n + 3) // 4]); souts.append(out); thrs.append(thr)
        tbq.decode(ins, souts, thrs, [1] * len(ins))
        torch.cuda.synchronize()
        for t in range(len(sizes)):
            assert_bits_equal(host(outs[t]), refs[t], f"tensor {t}, {size} slots without {gaps}")


@pytest.mark.parametrize("count", [2, 3, 5, 8, 9])
def test_message_counts_of_the_straight_line_path(tbq, oracle_cpu, count):
    # whole tiles with 2 to 8 messages take code generated per message count; payloads start at odd addresses
    rng = np.random.default_rng(300 + count)
    n = 3 * 4096 + 4096 // 2 + 3
    msgs, thrs, dm = [], [], []
    for k in range(count):
        thr = float(np.float32(rng.uniform(1e-3, 5e-3))) * (-1 if k == 1 else 1)
        g = rng.normal(0, 2e-3, n).astype(np.float32)
        m = oracle_cpu.tbq_encode(g, np.zeros(n, np.float32), abs(thr))
        msgs.append(m); thrs.append(thr)
        buf = torch.zeros(m.size + 8, dtype=torch.uint8, device="cuda")
        view = buf[k % 5:k % 5 + m.size]
        view.copy_(dev(m))
        dm.append(view)
    for adds in ([1] * count, [0] + [1] * (count - 1), [1, 0] + [1] * (count - 2)):
        base = rng.normal(0, 1, n).astype(np.float32)
        out = dev(base)
        tbq.decode(dm, [out] * count, thrs, adds)
        torch.cuda.synchronize()
        ref = base.copy()
        for m, thr, add in zip(msgs, thrs, adds):
            ref = oracle_cpu.tbq_decode(m, n, thr, ref, add)
        assert_bits_equal(host(out), ref, f"accumulated count={count} adds={adds}")


def test_many_tensors_each_with_several_messages(tbq, oracle_cpu):
    rng = np.random.default_rng(77)
    sizes = [int(s) for s in np.exp(rng.uniform(np.log(5), np.log(20000), 70))]
    slots = 35                                  # more than one segment of the slot table holds per tensor
    bases = [rng.normal(0, 1, n).astype(np.float32) for n in sizes]
    outs = [dev(b) for b in bases]
    call_outs, call_msgs, call_thr, call_add, refs = [], [], [], [], [b.copy() for b in bases]
    for k in range(slots):                      # interleaved: slot-major, as a gathered buffer is walked
        for t, n in enumerate(sizes):
            thr = float(np.float32(rng.uniform(1e-3, 5e-3)))
            m = oracle_cpu.tbq_encode(rng.normal(0, 2e-3, n).astype(np.float32), np.zeros(n, np.float32), thr)
            call_outs.append(outs[t]); call_msgs.append(dev(m)); call_thr.append(thr); call_add.append(1)
            refs[t] = oracle_cpu.tbq_decode(m, n, thr, refs[t], 1)
    tbq.decode(call_msgs, call_outs, call_thr, call_add)     # 2450 messages: several launches of the slot table
    torch.cuda.synchronize()
    for t in range(len(sizes)):
        assert_bits_equal(host(outs[t]), refs[t], f"tensor {t}")


def test_partially_overlapping_outputs_keep_call_order(tbq, oracle_cpu):
    rng = np.random.default_rng(5)
    n = 5000
    buf = torch.zeros(n + 1000, device="cuda")
    m1 = oracle_cpu.tbq_encode(rng.normal(0, 2e-3, n).astype(np.float32), np.zeros(n, np.float32), 2e-3)
    m2 = oracle_cpu.tbq_encode(rng.normal(0, 2e-3, n).astype(np.float32), np.zeros(n, np.float32), 3e-3)
    tbq.decode([dev(m1), dev(m2)], [buf[:n], buf[1000:1000 + n]], [2e-3, 3e-3], [1, 1])
    ref = np.zeros(n + 1000, np.float32)
    ref[:n] = oracle_cpu.tbq_decode(m1, n, 2e-3, ref[:n].copy(), 1)
    ref[1000:1000 + n] = oracle_cpu.tbq_decode(m2, n, 3e-3, ref[1000:1000 + n].copy(), 1)
    assert_bits_equal(host(buf), ref, "overlapping views")
