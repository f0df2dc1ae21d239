"""GPU parity: seeded random sweeps of whole calls against the CPU oracle (bit-exact).

The parametrised tests pin chosen cases; these draw the shape of a call itself — how many tensors, their sizes,
parameters and value distributions, where a tensor's messages lie and in which order they are handed over — so
that the host-side planning (launch tables, rounds of reports, cut jobs, fixed-distance and general decode
plans) sees combinations nobody wrote down.
"""
import numpy as np
import pytest
import torch

from gpu_util import Tbq, Terngrad, assert_bits_equal, dev, host, stream_ptr

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [1, 2])
def test_sparsifier_calls_with_random_buckets(capi, oracle_cpu, seed):
    # hpx_gd_encode / hpx_dgc_encode over buckets of 1 ... 700 ragged tensors (views of one buffer), sample rates
    # and kept fractions mixed within a call, heavy-tailed, normal, few-valued (ties at the cut) and mostly-zero
    # gradients; hp_cuda_kernel.cu:67-94 loops over such a list, hp_cuda.cpp:284-301 hands it over.
    L = capi.load()
    c = capi
    rng = np.random.default_rng(seed)
    cut = kept_all = 0
    for it in range(25):
        count = int(np.exp(rng.uniform(np.log(1), np.log(700))))
        hi = 3_000_000 if count < 20 else 200_000 if count < 200 else 20_000
        sizes = [int(np.exp(rng.uniform(np.log(1), np.log(hi)))) for _ in range(count)]
        srs = [float(rng.choice([0.01, 0.05, 0.2, 0.5, 1.0])) for _ in sizes]
        drs = [float(rng.choice([0.5, 0.9, 0.99, 0.999])) for _ in sizes]
        for i, n in enumerate(sizes):                             # parameters the reference itself would accept
            sc = int(np.ceil(n * srs[i]))
            if not (sc > 0 and int(sc * (1 - drs[i])) < sc):
                srs[i], drs[i] = 1.0, 0.5
        dist = rng.integers(0, 4, count)
        gs, rs = [], []
        for i, n in enumerate(sizes):
            if dist[i] == 0:
                g = rng.laplace(0, 1e-3, n)
            elif dist[i] == 1:
                g = rng.normal(0, 1e-3, n)
            elif dist[i] == 2:
                g = rng.choice([0.0, 1e-3, -1e-3, 2e-3], n)
            else:
                g = rng.laplace(0, 1e-3, n) * (rng.random(n) < 0.05)
            gs.append(g.astype(np.float32))
            rs.append(np.zeros(n, np.float32) if dist[i] == 2 else rng.normal(0, 1e-4, n).astype(np.float32))
        seeds = [int(x) for x in rng.integers(0, 2**63, count)]
        residual = bool(rng.integers(0, 2))
        starts = np.concatenate([[0], np.cumsum(sizes)])
        dg_all, dr_all = dev(np.concatenate(gs)), dev(np.concatenate(rs))
        dgs = [dg_all[starts[i]:starts[i + 1]] for i in range(count)]
        drs_ = [dr_all[starts[i]:starts[i + 1]] for i in range(count)]
        need = [4 + 8 * int(np.ceil(n * (1 - d))) for n, d in zip(sizes, drs)]
        ob = [(b + 3) // 4 * 4 + 8 for b in need]
        ostarts = np.concatenate([[0], np.cumsum(ob)])
        out_all = torch.full((int(ostarts[-1]),), 0xEE, dtype=torch.uint8, device="cuda")
        outs = [out_all[ostarts[i]:ostarts[i + 1]] for i in range(count)]
        if residual:
            rc = L.hpx_gd_encode(count, c.ptr_array([g.data_ptr() for g in dgs]), c.i32_array(sizes),
                                 c.ptr_array([r.data_ptr() for r in drs_]), c.ptr_array([o.data_ptr() for o in outs]),
                                 c.f64_array(srs), c.f64_array(drs), c.u64_array(seeds), stream_ptr())
        else:
            rc = L.hpx_dgc_encode(count, c.ptr_array([g.data_ptr() for g in dgs]), c.i32_array(sizes),
                                  c.ptr_array([o.data_ptr() for o in outs]), c.f64_array(srs),
                                  c.f64_array([1 - d for d in drs]), c.u64_array(seeds), stream_ptr())
        assert rc == 0, (it, c.last_error())
        torch.cuda.synchronize()
        got_all, g_got, r_got = host(out_all), host(dg_all), host(dr_all)
        for i, n in enumerate(sizes):
            what = f"call {it} tensor {i}: n={n} sample_rate={srs[i]} drop={drs[i]} seed={seeds[i]} values {dist[i]} residual={residual}"
            if residual:
                r_ref = rs[i].copy()
                msg, info = oracle_cpu.gd_encode(gs[i], r_ref, srs[i], drs[i], seeds[i])
                assert_bits_equal(r_got[starts[i]:starts[i + 1]], r_ref, "residual, " + what)
                assert_bits_equal(g_got[starts[i]:starts[i + 1]], gs[i], "gradient untouched, " + what)
            else:
                g_ref = gs[i].copy()
                msg, info = oracle_cpu.dgc_encode(g_ref, srs[i], 1 - drs[i], seeds[i])
                assert_bits_equal(g_got[starts[i]:starts[i + 1]], g_ref, "gradient, " + what)
            got = got_all[ostarts[i]:ostarts[i + 1]]
            assert_bits_equal(got[:msg.size], msg, "message, " + what)
            assert np.all(got[need[i]:] == 0xEE), "wrote past the message, " + what
            cut += info["candidates"] > info["kept"]
            kept_all += info["candidates"] <= info["kept"]
    assert cut > 100 and kept_all > 100, (cut, kept_all)


@pytest.mark.parametrize("seed", [1, 2])
def test_decode_calls_with_random_message_layouts(capi, oracle_cpu, seed):
    # Several messages per tensor in one hpx_tbq_decode / hpx_terngrad_decode call, as a root's ROOT_DECOMP task
    # hands them over (hp_cuda.cpp:241-259, :421-439): the messages of a tensor at one distance, with one gap, with
    # the gap first, with two gaps, or anywhere; tensor-major, slot-major or interleaved order; first message written
    # or added.  Every combination must equal applying the messages one at a time in call order.
    rng = np.random.default_rng(seed)
    tbq, tg = Tbq(capi), Terngrad(capi)
    for it in range(40):
        codec = "tbq" if rng.integers(0, 2) else "terngrad"
        ntens = int(np.exp(rng.uniform(0, np.log(260))))
        nslot = int(rng.integers(1, 10)) if ntens > 30 else int(rng.integers(1, 36))
        layout = int(rng.integers(0, 5))
        order_mode = int(rng.integers(0, 3))
        hi = 40_000 if ntens < 20 else 6000
        keep, outs, refs, per_tensor = [], [], [], []
        for t in range(ntens):
            n = int(np.exp(rng.uniform(0, np.log(hi))))
            if t == 0 and rng.integers(0, 2):
                n = 3 * 4096 + int(rng.integers(0, 4096))
            width = int(rng.choice([1, 2, 2, 2, 4, 8]))
            mbytes = (n + 3) // 4 if codec == "tbq" else 10 + (n + 8 // width - 1) // (8 // width)
            slot = mbytes + int(rng.integers(0, 9))
            gaps = {0: [], 1: [int(rng.integers(1, max(2, nslot)))], 2: [1], 3: [1, 3], 4: None}[layout]
            if gaps is None:
                positions = np.sort(rng.choice((nslot + 3) * 2, nslot, replace=False)).tolist()
            else:
                positions = [k for k in range(nslot + 3) if k not in gaps][:nslot]
            buf = np.zeros(slot * (max(positions) + 1) + 5, np.uint8)
            base = rng.normal(0, 1, n).astype(np.float32)
            ref = base.copy()
            thr = float(np.float32(rng.uniform(1e-3, 5e-3)))
            first_add = int(rng.integers(0, 2))
            off0 = int(rng.integers(0, 4))
            mine = []
            for j, k in enumerate(positions):
                g = rng.normal(0, 2e-3, n).astype(np.float32)
                add = 1 if (j or first_add) else 0
                if codec == "tbq":
                    m = oracle_cpu.tbq_encode(g, np.zeros(n, np.float32), thr)
                    ref = oracle_cpu.tbq_decode(m, n, thr, ref, add)
                else:
                    _, m = oracle_cpu.terngrad_encode(g, width, 1, int(rng.integers(0, 2**32)))
                    _, ref = oracle_cpu.terngrad_decode(m, n, ref, add)
                buf[off0 + k * slot:off0 + k * slot + m.size] = m
                mine.append((off0 + k * slot, m.size, add))
            db = dev(buf)
            out = dev(base)
            keep.append(db); outs.append(out); refs.append(ref)
            per_tensor.append([(db[o:o + s], out, thr, a) for o, s, a in mine])
        if order_mode == 0:
            seq = [x for p in per_tensor for x in p]
        elif order_mode == 1:
            seq = [p[k] for k in range(nslot) for p in per_tensor]
        else:                                                     # interleaved; a tensor's messages stay in order
            at = [0] * ntens
            live = list(range(ntens))
            seq = []
            while live:
                t = live[int(rng.integers(0, len(live)))]
                seq.append(per_tensor[t][at[t]])
                at[t] += 1
                if at[t] == nslot:
                    live.remove(t)
        if codec == "tbq":
            tbq.decode([s[0] for s in seq], [s[1] for s in seq], [s[2] for s in seq], [s[3] for s in seq])
        else:
            tg.decode([s[0] for s in seq], [s[1] for s in seq], [s[3] for s in seq])
        torch.cuda.synchronize()
        for t in range(ntens):
            assert_bits_equal(host(outs[t]), refs[t], f"call {it} ({codec}, {ntens} tensors x {nslot} messages, layout {layout}, order {order_mode}) tensor {t}")


@pytest.mark.parametrize("seed", [1, 2])
def test_tbq_calls_with_random_buckets(capi, oracle_cpu, seed):
    # hpx_tbq_encode / hpx_tbq_decode over buckets of 1 ... 700 tensors that start at any element of their buffers,
    # thresholds per tensor (zero and negative ones among them, which the reference accepts: tbq_body.h:70-84),
    # residuals carried over a second step, decode written or added.
    rng = np.random.default_rng(seed)
    tbq = Tbq(capi)
    for it in range(20):
        count = int(np.exp(rng.uniform(0, np.log(700))))
        hi = 3_000_000 if count < 20 else 100_000 if count < 200 else 10_000
        sizes = [int(np.exp(rng.uniform(0, np.log(hi)))) for _ in range(count)]
        offs = [int(rng.integers(0, 9)) for _ in sizes]
        thrs = [float(np.float32(rng.choice([2e-3, 1e-3, 5e-2, 0.0, -1e-3]))) for _ in sizes]
        span = [n + 16 for n in sizes]
        starts = np.concatenate([[0], np.cumsum(span)])
        g_all, r_all, o_all = (torch.zeros(int(starts[-1]), device="cuda") for _ in range(3))
        view = lambda buf: [buf[starts[i] + offs[i]:starts[i] + offs[i] + sizes[i]] for i in range(count)]
        dg, dr, do = view(g_all), view(r_all), view(o_all)
        rs = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
        for a, b in zip(dr, rs):
            a.copy_(dev(b))
        for step in range(2):
            gs = [rng.normal(0, 2e-3, n).astype(np.float32) for n in sizes]
            bases = [rng.normal(0, 1, n).astype(np.float32) for n in sizes]
            adds = [int(rng.integers(0, 2)) for _ in sizes]
            for a, b in zip(dg, gs):
                a.copy_(dev(b))
            for a, b in zip(do, bases):
                a.copy_(dev(b))
            packed = tbq.encode(dg, dr, thrs)
            tbq.decode(packed, do, thrs, adds)
            torch.cuda.synchronize()
            for i, n in enumerate(sizes):
                what = f"call {it} step {step} tensor {i}: n={n} offset={offs[i]} thr={thrs[i]} add={adds[i]}"
                pr = oracle_cpu.tbq_encode(gs[i], rs[i], thrs[i])          # rs[i] is updated in place: the next step's residual
                assert_bits_equal(host(packed[i]), pr, "codes, " + what)
                assert_bits_equal(host(dr[i]), rs[i], "residual, " + what)
                assert_bits_equal(host(do[i]), oracle_cpu.tbq_decode(pr, n, thrs[i], bases[i].copy(), adds[i]), "decoded, " + what)
        inside = np.zeros(int(starts[-1]), bool)
        for i, n in enumerate(sizes):
            inside[starts[i] + offs[i]:starts[i] + offs[i] + n] = True
        for name, buf in (("gradients", g_all), ("residuals", r_all), ("decoded tensors", o_all)):
            assert not host(buf)[~inside].any(), f"call {it}: wrote between the {name}"
