"""The C-ABI entry points called from several host threads at once - each on its own stream, and all on one -, as the
reference's five background threads call its drivers (hp_cuda.cpp:776-827): every thread loops over
TBQ, TernGrad and GradDrop encode/decode calls of its own tensors and every result must equal the CPU
oracle's.  The library keeps one workspace per (device, stream); nothing is shared between the threads but
the library itself."""
import threading

import numpy as np
import pytest
import torch

from gpu_util import host

pytestmark = pytest.mark.gpu


def test_four_threads_four_streams(capi, oracle_cpu):
    L, c = capi.load(), capi
    errors = []

    def worker(tid):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            sp = stream.cuda_stream
            rng = np.random.default_rng(100 + tid)
            with torch.cuda.stream(stream):
                for it in range(6):
                    n = int(rng.integers(1000, 400_000))
                    # TBQ
                    g = rng.normal(0, 2e-3, n).astype(np.float32)
                    r = rng.normal(0, 1e-3, n).astype(np.float32)
                    dg, dr = torch.from_numpy(g).cuda(), torch.from_numpy(r).cuda()
                    p = torch.zeros((n + 3) // 4, dtype=torch.uint8, device="cuda")
                    assert L.hpx_tbq_encode(1, c.ptr_array([dg.data_ptr()]), c.i32_array([n]), c.ptr_array([dr.data_ptr()]),
                                            c.ptr_array([p.data_ptr()]), c.f32_array([2e-3]), sp) == 0, c.last_error()
                    # TernGrad, stochastic rounding with a fixed seed
                    x = rng.normal(0, 1e-2, n).astype(np.float32)
                    dx = torch.from_numpy(x).cuda()
                    m = torch.zeros(10 + (n + 3) // 4, dtype=torch.uint8, device="cuda")
                    assert L.hpx_terngrad_encode(1, c.ptr_array([dx.data_ptr()]), c.i32_array([n]), c.ptr_array([m.data_ptr()]),
                                                 c.i32_array([m.numel()]), c.u8_array([2]), c.i32_array([1]),
                                                 c.u64_array([tid * 1000 + it]), sp) == 0, c.last_error()
                    dec = torch.zeros(n, device="cuda")
                    assert L.hpx_terngrad_decode(1, c.ptr_array([dec.data_ptr()]), c.i32_array([n]), c.ptr_array([m.data_ptr()]),
                                                 c.i32_array([m.numel()]), c.i32_array([0]), sp) == 0, c.last_error()
                    # GradDrop (waits for its stream inside the call)
                    gg = rng.laplace(0, 1e-3, n).astype(np.float32)
                    rr = rng.normal(0, 1e-4, n).astype(np.float32)
                    dgg, drr = torch.from_numpy(gg).cuda(), torch.from_numpy(rr).cuda()
                    _, expected, _ = oracle_cpu.gd_sizes(n, 0.05, 0.99)
                    out = torch.zeros(4 + 8 * expected, dtype=torch.uint8, device="cuda")
                    assert L.hpx_gd_encode(1, c.ptr_array([dgg.data_ptr()]), c.i32_array([n]), c.ptr_array([drr.data_ptr()]),
                                           c.ptr_array([out.data_ptr()]), c.f64_array([0.05]), c.f64_array([0.99]),
                                           c.u64_array([tid * 77 + it]), sp) == 0, c.last_error()
                    stream.synchronize()
                    r_ref = r.copy()
                    assert np.array_equal(host(p), oracle_cpu.tbq_encode(g, r_ref, 2e-3)), f"thread {tid} it {it}: TBQ bytes"
                    assert np.array_equal(host(dr).view(np.uint32), r_ref.view(np.uint32)), f"thread {tid} it {it}: TBQ residual"
                    rc, ref = oracle_cpu.terngrad_encode(x, 2, 1, tid * 1000 + it)
                    assert rc == 0 and np.array_equal(host(m), ref), f"thread {tid} it {it}: TernGrad message"
                    assert np.array_equal(host(dec).view(np.uint32), oracle_cpu.terngrad_decode(ref, n)[1].view(np.uint32))
                    rr_ref = rr.copy()
                    msg, info = oracle_cpu.gd_encode(gg, rr_ref, 0.05, 0.99, tid * 77 + it)
                    assert np.array_equal(host(out)[:msg.size], msg), f"thread {tid} it {it}: GradDrop message {info}"
                    assert np.array_equal(host(drr).view(np.uint32), rr_ref.view(np.uint32)), f"thread {tid} it {it}: GradDrop residual"
        except BaseException as e:  # noqa: BLE001 - reported to the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread is stuck"
    assert not errors, errors


def test_five_threads_on_one_stream_and_graddrop_on_the_null_stream(capi, pkg, oracle_cpu):
    """The reference's own pattern: its five background threads all enqueue on ONE function-static compute
    stream (hp_cuda.cpp:789, :867-873) and GradDrop encode goes out on the legacy null stream (hp_cuda.cpp:300).
    Here five host threads issue TBQ, TernGrad (among them tensors large enough for the single-launch encode
    and a bucket of tensors) and PowerSGD calls on one shared stream at the same time while a sixth issues
    hpx_gd_encode / hpx_gd_decode on the null stream; every result must equal the CPU oracle's.  All device
    tensors are made beforehand, so the threads do nothing but call the C ABI."""
    from oracle import powersgd as ps
    L, c = capi.load(), capi
    torch.cuda.synchronize()
    assert L.hpx_release_workspaces() == 0          # the shared stream will be the one that owns the barrier kernels
    old = [capi.set_option("terngrad_resident_min", 1 << 21), capi.set_option("terngrad_resident_bucket", 1)]
    shared = torch.cuda.Stream()
    sp = shared.cuda_stream
    iters = 4
    rng = np.random.default_rng(4242)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    jobs, checks, errors = {}, [], []

    # thread 0: TBQ encode + decode of three tensors per call
    def make_tbq(it):
        ns = [int(rng.integers(1000, 300_000)) for _ in range(3)]
        gs = [rng.normal(0, 2e-3, n).astype(np.float32) for n in ns]
        rs = [rng.normal(0, 1e-3, n).astype(np.float32) for n in ns]
        d = dict(ns=ns, gs=gs, rs=rs, dg=[dev(g) for g in gs], dr=[dev(r) for r in rs],
                 p=[torch.zeros((n + 3) // 4, dtype=torch.uint8, device="cuda") for n in ns],
                 o=[torch.zeros(n, device="cuda") for n in ns])
        def run():
            assert L.hpx_tbq_encode(3, c.ptr_array([t.data_ptr() for t in d["dg"]]), c.i32_array(ns), c.ptr_array([t.data_ptr() for t in d["dr"]]),
                                    c.ptr_array([t.data_ptr() for t in d["p"]]), c.f32_array([2e-3] * 3), sp) == 0, c.last_error()
            assert L.hpx_tbq_decode(3, c.ptr_array([t.data_ptr() for t in d["o"]]), c.i32_array(ns), c.ptr_array([t.data_ptr() for t in d["p"]]),
                                    c.f32_array([2e-3] * 3), c.i32_array([0] * 3), sp) == 0, c.last_error()
        def check():
            for i, n in enumerate(ns):
                r_ref = rs[i].copy()
                p_ref = oracle_cpu.tbq_encode(gs[i], r_ref, 2e-3)
                assert np.array_equal(host(d["p"][i]), p_ref), f"TBQ bytes it {it} tensor {i}"
                assert np.array_equal(host(d["dr"][i]).view(np.uint32), r_ref.view(np.uint32)), f"TBQ residual it {it}"
                assert np.array_equal(host(d["o"][i]), oracle_cpu.tbq_decode(p_ref, n, 2e-3)), f"TBQ decode it {it}"
        return run, check

    # threads 1, 2, 4: TernGrad calls of the given sizes (one call per iteration), then a decode of the first message
    def make_tg(sizes_fn, seed0):
        def make(it):
            ns = sizes_fn()
            xs = [rng.normal(0, 1e-2, n).astype(np.float32) for n in ns]
            dx = [dev(x) for x in xs]
            ms = [torch.zeros(10 + (n + 3) // 4, dtype=torch.uint8, device="cuda") for n in ns]
            dec = torch.zeros(ns[0], device="cuda")
            seeds = [seed0 + 100 * it + k for k in range(len(ns))]
            def run():
                k = len(ns)
                assert L.hpx_terngrad_encode(k, c.ptr_array([t.data_ptr() for t in dx]), c.i32_array(ns), c.ptr_array([t.data_ptr() for t in ms]),
                                             c.i32_array([t.numel() for t in ms]), c.u8_array([2] * k), c.i32_array([1] * k),
                                             c.u64_array(seeds), sp) == 0, c.last_error()
                assert L.hpx_terngrad_decode(1, c.ptr_array([dec.data_ptr()]), c.i32_array([ns[0]]), c.ptr_array([ms[0].data_ptr()]),
                                             c.i32_array([ms[0].numel()]), c.i32_array([0]), sp) == 0, c.last_error()
            def check():
                for i in range(len(ns)):
                    rc, ref = oracle_cpu.terngrad_encode(xs[i], 2, 1, seeds[i])
                    assert rc == 0 and np.array_equal(host(ms[i]), ref), f"TernGrad message it {it} tensor {i} n={ns[i]}"
                    if i == 0:
                        assert np.array_equal(host(dec).view(np.uint32), oracle_cpu.terngrad_decode(ref, ns[0])[1].view(np.uint32))
            return run, check
        return make

    # thread 3: the three PowerSGD phases of two matrices
    def make_psgd(it):
        shapes, rk = [(256, 192), (130, 515)], 4
        G = [rng.normal(0, 1e-2, a * b).astype(np.float32) for a, b in shapes]
        Q0 = [rng.normal(0, 1, (b, rk)).astype(np.float32) for a, b in shapes]
        dG, dQ = [dev(g) for g in G], [dev(q) for q in Q0]
        dR = [torch.zeros(a * b, device="cuda") for a, b in shapes]
        dM = [torch.zeros(a, b, device="cuda") for a, b in shapes]
        dP = [torch.zeros(a, rk, device="cuda") for a, b in shapes]
        def run():
            assert pkg.hp_cuda_powersgd_encode1(dG, dR, dQ, dM, dP, stream=sp) == 0
            assert pkg.hp_cuda_powersgd_encode2(dP, dM, dQ, stream=sp) == 0
            assert pkg.hp_cuda_powersgd_decode(dP, dQ, dM, dR, dG, stream=sp) == 0
        def check():
            for i, (a, b) in enumerate(shapes):
                Mref, Pref = ps.encode1(G[i], np.zeros_like(G[i]), Q0[i], np.zeros((a, b), np.float32))
                Po, Qn = ps.encode2(Pref, Mref)
                Mn, Rn, Gn = ps.decode(Po, Qn, G[i])
                assert ps.rel_fro(host(dM[i]), Mn) < 1e-4 and ps.rel_fro(host(dG[i]), Gn) < 1e-4, f"PowerSGD it {it} matrix {i}"
        return run, check

    # thread 5: GradDrop on the NULL stream
    def make_gd(it):
        ns = [int(rng.integers(50_000, 600_000)) for _ in range(2)]
        gs = [rng.laplace(0, 1e-3, n).astype(np.float32) for n in ns]
        rs = [rng.normal(0, 1e-4, n).astype(np.float32) for n in ns]
        dg, dr = [dev(g) for g in gs], [dev(r) for r in rs]
        outs = [torch.zeros(4 + 8 * oracle_cpu.gd_sizes(n, 0.05, 0.99)[1], dtype=torch.uint8, device="cuda") for n in ns]
        dec = torch.zeros(ns[0], device="cuda")
        seeds = [900 + 10 * it, 901 + 10 * it]
        def run():
            assert L.hpx_gd_encode(2, c.ptr_array([t.data_ptr() for t in dg]), c.i32_array(ns), c.ptr_array([t.data_ptr() for t in dr]),
                                   c.ptr_array([t.data_ptr() for t in outs]), c.f64_array([0.05] * 2), c.f64_array([0.99] * 2),
                                   c.u64_array(seeds), None) == 0, c.last_error()
            assert L.hpx_gd_decode(1, c.ptr_array([outs[0].data_ptr()]), c.i32_array([outs[0].numel()]), c.ptr_array([dec.data_ptr()]),
                                   c.i32_array([ns[0]]), c.i32_array([0]), None) == 0, c.last_error()
        def check():
            for i, n in enumerate(ns):
                r_ref = rs[i].copy()
                msg, info = oracle_cpu.gd_encode(gs[i], r_ref, 0.05, 0.99, seeds[i])
                assert np.array_equal(host(outs[i])[:msg.size], msg), f"GradDrop message it {it} tensor {i} {info}"
                assert np.array_equal(host(dr[i]).view(np.uint32), r_ref.view(np.uint32)), f"GradDrop residual it {it}"
                if i == 0:
                    want = np.zeros(n, np.float32)
                    oracle_cpu.gd_decode(msg, want, 0)
                    assert np.array_equal(host(dec), want), f"GradDrop decode it {it}"
        return run, check

    makers = {0: make_tbq,
              1: make_tg(lambda: [int(rng.integers(1000, 400_000))], 1000),
              2: make_tg(lambda: [3_000_000 + int(rng.integers(0, 5000))], 2000),                  # single-launch resident encode
              3: make_psgd,
              4: make_tg(lambda: [int(rng.integers(200_000, 900_000)) for _ in range(5)], 4000),   # a bucket: one resident launch
              5: make_gd}
    try:
        for tid, make in makers.items():
            jobs[tid] = [make(it) for it in range(iters)]
        torch.cuda.synchronize()

        def worker(tid):
            try:
                torch.cuda.set_device(0)
                for run, _ in jobs[tid]:
                    run()
            except BaseException as e:  # noqa: BLE001 - reported to the main thread
                errors.append((tid, repr(e)))

        threads = [threading.Thread(target=worker, args=(t,)) for t in makers]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
        assert not any(t.is_alive() for t in threads), "a worker thread is stuck"
        assert not errors, errors
        shared.synchronize()
        torch.cuda.synchronize()
        assert L.hpx_terngrad_encode_status(sp) == 0 and L.hpx_terngrad_repaired(sp) == 0
        for tid in makers:                                   # stop at the first failure
            for _, check in jobs[tid]:
                check()
    finally:
        capi.set_option("terngrad_resident_min", old[0])
        capi.set_option("terngrad_resident_bucket", old[1])
        torch.cuda.synchronize()
        assert L.hpx_release_workspaces() == 0
