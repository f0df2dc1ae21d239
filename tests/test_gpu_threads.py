"""The C-ABI entry points called from several host threads at once, each on its own stream, as the
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
