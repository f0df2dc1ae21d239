"""GPU parity of the task scheduler (hp_cuda.init / submit_task / getResults over libhpx.so) against the
CPU oracle: what a COMP, DECOMP and ROOT_DECOMP_COMP task leaves in C, in the gradient and in the
residual, and which finished queue its name appears in (hp_cuda.cpp:163-772, :1043-1066).  Every test
runs through both front ends of the scheduler: the compiled `hp_cuda` extension module and the ctypes
module of the package."""
import numpy as np
import pytest
import torch

from gpu_util import assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["compiled", "ctypes"])
def hp(request, pkg, hp_cuda_compiled):
    assert torch.cuda.is_available()
    mod = hp_cuda_compiled if request.param == "compiled" else pkg.hp_cuda
    yield mod
    mod.end()
    for q in (10, 20, 30):
        mod.getResults(q)


def _collect(hp, task_id, names, timeout_s=20.0):
    got = []
    import time
    t0 = time.time()
    while len(got) < len(names) and time.time() - t0 < timeout_s:
        hp.wait(task_id, 200)
        got += hp.getResults(task_id)
    assert sorted(got) == sorted(names), (got, names, hp.last_error())
    return got


def _host_buf(nbytes, pinned):
    return torch.zeros(nbytes, dtype=torch.uint8, pin_memory=bool(pinned))


@pytest.mark.parametrize("pinned", [0, 1])
def test_terngrad_comp_decomp_root(hp, oracle_cpu, pinned):
    rng = np.random.default_rng(1)
    n, b, seed, size, rank = 100_003, 2, 5, 3, 1
    assert hp.init("terngrad", {"enable_random": 1, "bitwidth": b, "seed": seed}, 0, rank, size)
    msg_bytes = oracle_cpu.terngrad_packed_size(n, b)

    # COMP: tensor -> B -> C
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    dx = dev(x)
    B = torch.zeros(msg_bytes, dtype=torch.uint8, device="cuda")
    Cc = _host_buf(msg_bytes, pinned)
    torch.cuda.synchronize()
    assert hp.submit_task("layer0.weight", dx, B, Cc, 0, 10)
    _collect(hp, 10, ["layer0.weight"])
    rc, ref = oracle_cpu.terngrad_encode(x, b, 1, seed)
    assert_bits_equal(Cc.numpy(), ref, "COMP message in C")
    assert hp.getResults(20) == [] and hp.getResults(30) == []

    # DECOMP, write (is_root 0) and add (is_root 1): C -> B -> tensor
    for is_root in (0, 1):
        base = rng.normal(0, 1, n).astype(np.float32)
        dt = dev(base)
        Cd = _host_buf(msg_bytes, pinned); Cd.numpy()[:] = ref
        Bd = torch.zeros(msg_bytes, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        assert hp.submit_task(f"dec{is_root}", dt, Bd, Cd, is_root, 20)
        _collect(hp, 20, [f"dec{is_root}"])
        rc, want = oracle_cpu.terngrad_decode(ref, n, base.copy(), is_root)
        assert_bits_equal(host(dt), want, f"DECOMP is_root={is_root}")

    # ROOT: decode every gathered slot but our own rank's (add), then re-encode the sum
    others = [rng.normal(0, 1e-2, n).astype(np.float32) for _ in range(size)]
    slots = np.zeros(size * msg_bytes, np.uint8)
    for i in range(size):
        rc, m = oracle_cpu.terngrad_encode(others[i], b, 1, 100 + i)
        slots[i * msg_bytes:(i + 1) * msg_bytes] = m
    slots[rank * msg_bytes:(rank + 1) * msg_bytes] = 0xEE            # never read
    mine = rng.normal(0, 1e-2, n).astype(np.float32)
    dmine = dev(mine)
    Cr = _host_buf(size * msg_bytes, pinned); Cr.numpy()[:] = slots
    Br = torch.zeros(msg_bytes, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    assert hp.submit_task("root.w", dmine, Br, Cr, 1, 30)
    _collect(hp, 30, ["root.w"])
    want = mine.copy()
    for i in range(size):
        if i != rank:
            rc, want = oracle_cpu.terngrad_decode(slots[i * msg_bytes:(i + 1) * msg_bytes], n, want, 1)
    assert_bits_equal(host(dmine), want, "ROOT: gradient after the gathered slots were added")
    rc, ref2 = oracle_cpu.terngrad_encode(want, b, 1, seed)
    assert_bits_equal(Cr.numpy()[:msg_bytes], ref2, "ROOT: re-encoded message in C")
    assert_bits_equal(Cr.numpy()[msg_bytes:], slots[msg_bytes:], "ROOT: the other slots of C are untouched")
    assert hp.error_count() == 0, hp.last_error()


def test_terngrad_comp_task_survives_an_expired_barrier(hp, oracle_cpu, capi):
    # A COMP task whose tensor takes the single-launch encode, with that kernel's barrier bound forced to zero
    # from the host (all workgroups give up and leave normally): the scheduler asks for the encode status
    # before it copies B to C, so the name is published with the valid message of that very task in C.
    rng = np.random.default_rng(41)
    n, b, seed = 3_000_001, 2, 77
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    rc, ref = oracle_cpu.terngrad_encode(x, b, 1, seed)
    L = capi.load()
    torch.cuda.synchronize()
    assert L.hpx_release_workspaces() == 0                  # the worker's compute stream will own the barrier kernels
    old = [capi.set_option("terngrad_resident_min", 1 << 21), capi.set_option("terngrad_resident_bucket", 0),
           capi.set_option("terngrad_barrier_ms", 0)]
    L.hpx_profile_reset(); L.hpx_profile_enable(1)
    try:
        assert hp.init("terngrad", {"enable_random": 1, "bitwidth": b, "seed": seed}, 0, 0, 2)
        dx = dev(x)
        B = torch.full((ref.size,), 0x5A, dtype=torch.uint8, device="cuda")
        Cc = _host_buf(ref.size, 1)
        torch.cuda.synchronize()
        assert hp.submit_task("big.weight", dx, B, Cc, 0, 10)
        _collect(hp, 10, ["big.weight"])
        assert_bits_equal(Cc.numpy(), ref, "COMP message in C after the barrier expired")
        assert hp.error_count() == 0, hp.last_error()
        assert capi.profile_query("terngrad_resident_kernel")[1] == 1      # the single-launch encode ran (and gave up) ...
        assert capi.profile_query("terngrad_quant_kernel")[1] == 1         # ... and the two-launch path encoded it again
    finally:
        L.hpx_profile_enable(0); L.hpx_profile_reset()
        for name, v in zip(("terngrad_resident_min", "terngrad_resident_bucket", "terngrad_barrier_ms"), old):
            capi.set_option(name, v)
        hp.end()
        torch.cuda.synchronize()
        assert L.hpx_release_workspaces() == 0


@pytest.mark.parametrize("lo,hi,count", [(5, 70_000, 24), (2 << 20, 5 << 20, 18)])
def test_tbq_batch_of_mixed_tasks(hp, oracle_cpu, lo, hi, count):
    # the large case: messages of 0.5 to 1.25 MB, so the batch's transfers and codec calls are cut into several runs
    rng = np.random.default_rng(2)
    thr, size, rank = 2e-3, 4, 0
    assert hp.init("tbq", {"threshold": thr}, 0, rank, size)
    keep, checks = [], []
    sizes = [int(s) for s in rng.integers(lo, hi, count)]
    for k, n in enumerate(sizes):
        kind = (10, 20, 30)[k % 3]
        mb = oracle_cpu.tbq_packed_size(n)
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        r = rng.normal(0, 1e-3, n).astype(np.float32)
        dg, dr = dev(g), dev(r)
        B = torch.zeros(mb, dtype=torch.uint8, device="cuda")
        if kind == 10:
            Cc = _host_buf(mb, k & 1)
            checks.append((kind, f"t{k}", g, r, dg, dr, Cc, None))
        elif kind == 20:
            src = rng.normal(0, 1e-3, n).astype(np.float32)
            msg = oracle_cpu.tbq_encode(src, np.zeros(n, np.float32), thr)
            Cc = _host_buf(mb, k & 1); Cc.numpy()[:] = msg
            checks.append((kind, f"t{k}", g, r, dg, dr, Cc, msg))
        else:
            slots = np.zeros(size * mb, np.uint8)
            for i in range(size):
                slots[i * mb:(i + 1) * mb] = oracle_cpu.tbq_encode(rng.normal(0, 2e-3, n).astype(np.float32), np.zeros(n, np.float32), thr)
            Cc = _host_buf(size * mb, k & 1); Cc.numpy()[:] = slots
            checks.append((kind, f"t{k}", g, r, dg, dr, Cc, slots))
        keep.append(B)
    torch.cuda.synchronize()
    for (kind, name, g, r, dg, dr, Cc, extra), B in zip(checks, keep):
        assert hp.submit_task(name, dg, dr, B, Cc, 1, kind)
    for kind in (10, 20, 30):
        _collect(hp, kind, [c[1] for c in checks if c[0] == kind])
    for kind, name, g, r, dg, dr, Cc, extra in checks:
        n = g.size
        mb = oracle_cpu.tbq_packed_size(n)
        if kind == 10:
            rr = r.copy()
            msg = oracle_cpu.tbq_encode(g, rr, thr)
            assert_bits_equal(Cc.numpy(), msg, f"{name} COMP message"); assert_bits_equal(host(dr), rr, f"{name} residual")
            assert_bits_equal(host(dg), g, f"{name} gradient untouched")
        elif kind == 20:
            want = oracle_cpu.tbq_decode(extra, n, thr, g.copy(), 1)
            assert_bits_equal(host(dg), want, f"{name} DECOMP add")
        else:
            want = g.copy()
            for i in range(size):
                if i != rank:
                    want = oracle_cpu.tbq_decode(extra[i * mb:(i + 1) * mb], n, thr, want, 1)
            rr = r.copy()
            msg = oracle_cpu.tbq_encode(want, rr, thr)
            assert_bits_equal(host(dg), want, f"{name} ROOT gradient"); assert_bits_equal(host(dr), rr, f"{name} ROOT residual")
            assert_bits_equal(Cc.numpy()[:mb], msg, f"{name} ROOT message")
    assert hp.error_count() == 0, hp.last_error()


def test_terngrad_batch_spanning_several_runs(hp, oracle_cpu):
    # 10 COMP and 10 DECOMP tasks with messages of about 1 MB each, submitted in one go
    rng = np.random.default_rng(21)
    b, seed = 2, 9
    assert hp.init("terngrad", {"enable_random": 1, "bitwidth": b, "seed": seed}, 0, 0, 2)
    comp, dec, keep = [], [], []
    for k in range(10):
        n = int(rng.integers(3 << 20, 5 << 20))
        mb = oracle_cpu.terngrad_packed_size(n, b)
        x = rng.normal(0, 1e-2, n).astype(np.float32)
        comp.append((f"c{k}", x, dev(x), torch.zeros(mb, dtype=torch.uint8, device="cuda"), _host_buf(mb, k & 1)))
        src = rng.normal(0, 1e-2, n).astype(np.float32)
        rc, msg = oracle_cpu.terngrad_encode(src, b, 1, 100 + k)
        base = rng.normal(0, 1, n).astype(np.float32)
        C = _host_buf(mb, (k + 1) & 1); C.numpy()[:] = msg
        dec.append((f"d{k}", msg, base, dev(base), torch.zeros(mb, dtype=torch.uint8, device="cuda"), C, k % 2))
    torch.cuda.synchronize()
    for (cn, x, dx, B, C), (dn, msg, base, dt, Bd, Cd, add) in zip(comp, dec):
        assert hp.submit_task(cn, dx, B, C, 0, 10)
        assert hp.submit_task(dn, dt, Bd, Cd, add, 20)
    _collect(hp, 10, [c[0] for c in comp])
    _collect(hp, 20, [d[0] for d in dec])
    for cn, x, dx, B, C in comp:
        rc, ref = oracle_cpu.terngrad_encode(x, b, 1, seed)
        assert_bits_equal(C.numpy(), ref, f"{cn} message in C")
    for dn, msg, base, dt, Bd, Cd, add in dec:
        rc, want = oracle_cpu.terngrad_decode(msg, base.size, base.copy(), add)
        assert_bits_equal(host(dt), want, f"{dn} decoded")
    assert hp.error_count() == 0, hp.last_error()


def test_graddrop_comp_and_decomp(hp, oracle_cpu):
    rng = np.random.default_rng(3)
    n, sr, dr_, seed = 300_007, 0.02, 0.97, 11
    assert hp.init("graddrop", {"sample_rate": sr, "drop_ratio": dr_, "seed": seed}, 0, 0, 2)
    fixed = 4 + int(2 * np.ceil(n * (1 - dr_))) * 4          # hp_cuda.cpp:230
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    r = rng.normal(0, 1e-4, n).astype(np.float32)
    dg, dres = dev(g), dev(r)
    B = torch.zeros(fixed, dtype=torch.uint8, device="cuda")
    Cc = _host_buf(fixed, 0)
    torch.cuda.synchronize()
    assert hp.submit_task("fc.weight", dg, dres, B, Cc, 0, 10)
    _collect(hp, 10, ["fc.weight"])
    rr = r.copy()
    msg, info = oracle_cpu.gd_encode(g, rr, sr, dr_, seed)
    assert_bits_equal(Cc.numpy()[:msg.size], msg, "COMP message"); assert_bits_equal(host(dres), rr, "residual")
    # DECOMP of that message, add mode
    base = rng.normal(0, 1, n).astype(np.float32)
    dt = dev(base)
    Bd = torch.zeros(fixed, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    assert hp.submit_task("fc.weight", dt, dres, Bd, Cc, 1, 20)
    _collect(hp, 20, ["fc.weight"])
    want = base.copy()
    assert oracle_cpu.gd_decode(msg, want, 1) == 0
    assert_bits_equal(host(dt), want, "DECOMP add")
    assert hp.error_count() == 0, hp.last_error()


def test_powersgd_tasks_equal_direct_calls(hp, pkg, capi):
    rng = np.random.default_rng(4)
    assert hp.init("powersgd", {"matrix_approximation_rank": 4}, 0, 0, 2)
    shapes = [(256, 512), (300, 70), (64, 64)]
    tasks, refs = [], []
    for k, (n, m) in enumerate(shapes):
        G = dev(rng.normal(0, 1e-2, n * m).astype(np.float32)); R = dev(rng.normal(0, 1e-3, n * m).astype(np.float32))
        Q = dev(rng.normal(0, 1, (m, 4)).astype(np.float32)); M = torch.zeros(n, m, device="cuda"); P = torch.zeros(n, 4, device="cuda")
        tasks.append((f"w{k}", G, R, M, P, Q))
        refs.append(tuple(x.clone() for x in (G, R, M, P, Q)))
    torch.cuda.synchronize()
    for phase, tid, queue in ((1, 40, 40), (2, 50, 50), (3, 60, 60)):
        for name, G, R, M, P, Q in tasks:
            assert hp.submit_task(name, G, R, M, P, Q, tid)
        _collect(hp, queue, [t[0] for t in tasks])
        for G, R, M, P, Q in refs:
            if phase == 1:
                pkg.hp_cuda_powersgd_encode1([G], [R], [Q], [M], [P])
            elif phase == 2:
                pkg.hp_cuda_powersgd_encode2([P], [M], [Q])
            else:
                pkg.hp_cuda_powersgd_decode([P], [Q], [M], [R], [G])
        torch.cuda.synchronize()
        for (name, *ts), rs in zip(tasks, refs):
            for a, b_, what in zip(ts, rs, "GRMPQ"):
                assert_bits_equal(host(a), host(b_), f"{name} {what} after phase {phase}")
    assert hp.error_count() == 0, hp.last_error()


def test_argument_checks_and_restart(hp, capsys):
    assert hp.init("tbq", {"threshold": 1e-3}, 0, 0, 2)
    t = torch.zeros(16, device="cuda"); B = torch.zeros(4, dtype=torch.uint8, device="cuda"); Cc = torch.zeros(4, dtype=torch.uint8)
    assert hp.submit_task("x", t, t.clone(), B, Cc, 2, 10) is False            # hp_cuda.cpp:947-950
    assert "is_root should be 0 (~root) or 1 (root), find is_root is 2" in hp.last_error()
    assert hp.submit_task("x", t, t.clone(), B, Cc, 0, 40) is False            # hp_cuda.cpp:951-954
    assert "task_id should be 10 (comp) or 20 (decomp) or 30" in hp.last_error()
    with pytest.raises(RuntimeError, match="CPU tensor"):
        hp.submit_task("x", t, t.clone(), B, B, 0, 10)
    with pytest.raises(RuntimeError, match="contiguous"):
        hp.submit_task("x", torch.zeros(4, 8, device="cuda").t(), t.clone(), B, Cc, 0, 10)
    assert hp.end()
    with pytest.raises(RuntimeError, match="not running"):                     # check_thread(), hp_cuda.cpp:892-900
        hp.submit_task("x", t, t.clone(), B, Cc, 0, 10)
    assert hp.init("tbq", {"threshold": 1e-3}, 0, 0, 2)                        # start again after end()
    torch.cuda.synchronize()
    assert hp.submit_task("y", t, t.clone(), B, Cc, 0, 10)
    _collect(hp, 10, ["y"])


def test_graddrop_root_task(hp, oracle_cpu):
    rng = np.random.default_rng(8)
    n, sr, dr_, seed, size, rank = 120_001, 0.05, 0.98, 3, 3, 2
    assert hp.init("graddrop", {"sample_rate": sr, "drop_ratio": dr_, "seed": seed}, 0, rank, size)
    fixed = 4 + int(2 * np.ceil(n * (1 - dr_))) * 4
    slots = np.zeros(size * fixed, np.uint8)
    msgs = []
    for i in range(size):
        m, _ = oracle_cpu.gd_encode(rng.laplace(0, 1e-3, n).astype(np.float32), np.zeros(n, np.float32), sr, dr_, 50 + i)
        slots[i * fixed:i * fixed + m.size] = m
        msgs.append(m)
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    r = rng.normal(0, 1e-4, n).astype(np.float32)
    dg, dres = dev(g), dev(r)
    B = torch.zeros(fixed, dtype=torch.uint8, device="cuda")
    Cc = _host_buf(size * fixed, 0); Cc.numpy()[:] = slots
    torch.cuda.synchronize()
    assert hp.submit_task("emb", dg, dres, B, Cc, 1, 30)
    _collect(hp, 30, ["emb"])
    want = g.copy()
    for i in range(size):
        if i != rank:
            assert oracle_cpu.gd_decode(msgs[i], want, 1) == 0
    rr = r.copy()
    msg, info = oracle_cpu.gd_encode(want, rr, sr, dr_, seed)
    assert_bits_equal(host(dg), want, "ROOT gradient"); assert_bits_equal(host(dres), rr, "ROOT residual")
    assert_bits_equal(Cc.numpy()[:msg.size], msg, "ROOT message")
    assert hp.error_count() == 0, hp.last_error()


def test_submitters_on_several_threads(hp, oracle_cpu):
    # tasks arrive from four host threads while the worker is busy; every name comes back once
    import threading
    rng = np.random.default_rng(9)
    thr = 1e-3
    assert hp.init("tbq", {"threshold": thr}, 0, 0, 2)
    items = []
    for k in range(64):
        n = int(rng.integers(100, 200_000))
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        items.append((f"p{k}", g, dev(g), torch.zeros(n, device="cuda"),
                      torch.zeros(oracle_cpu.tbq_packed_size(n), dtype=torch.uint8, device="cuda"),
                      _host_buf(oracle_cpu.tbq_packed_size(n), k & 1)))
    torch.cuda.synchronize()

    def feed(part):
        for name, g, dg, dr, B, Cc in part:
            assert hp.submit_task(name, dg, dr, B, Cc, 0, 10)
    threads = [threading.Thread(target=feed, args=(items[i::4],)) for i in range(4)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    _collect(hp, 10, [it[0] for it in items])
    for name, g, dg, dr, B, Cc in items:
        rr = np.zeros(g.size, np.float32)
        msg = oracle_cpu.tbq_encode(g, rr, thr)
        assert_bits_equal(Cc.numpy(), msg, f"{name} message"); assert_bits_equal(host(dr), rr, f"{name} residual")
    assert hp.error_count() == 0, hp.last_error()


def test_codec_failure_is_counted_and_the_task_still_finishes(hp):
    # A body failure (here: bitwidth 3, terngrad_body.h:207-212) is printed and the loop carries on in the
    # reference (hp_cuda_kernel.cu:63); the task's name is still pushed to its finished queue.
    assert hp.init("terngrad", {"enable_random": 0, "bitwidth": 3}, 0, 0, 2)
    x = torch.randn(1000, device="cuda")
    B = torch.zeros(10 + 1000, dtype=torch.uint8, device="cuda")
    Cc = torch.full((10 + 1000,), 7, dtype=torch.uint8)
    torch.cuda.synchronize()
    assert hp.submit_task("bad", x, B, Cc, 0, 10)
    _collect(hp, 10, ["bad"])
    assert hp.error_count() >= 1 and "bitwidth" in hp.last_error()
    assert int(B.sum()) == 0            # nothing was encoded


def test_task_with_too_small_buffers_is_skipped_counted_and_still_named(hp):
    n, sr, dr_ = 100_003, 0.05, 0.99
    assert hp.init("graddrop", {"sample_rate": sr, "drop_ratio": dr_, "seed": 1}, 0, 0, 2)
    g = torch.randn(n, device="cuda") * 1e-3
    res = torch.zeros(n, device="cuda")
    before = hp.error_count()
    B = torch.zeros(64, dtype=torch.uint8, device="cuda")            # far less than 4 + 8*ceil(n*(1-drop))
    Cc = torch.zeros(64, dtype=torch.uint8, pin_memory=True)
    torch.cuda.synchronize()
    assert hp.submit_task("tiny", g, res, B, Cc, 0, 20)
    _collect(hp, 20, ["tiny"])
    assert hp.error_count() == before + 1 and "does not fit" in hp.last_error()
    assert float(g.abs().max()) > 0 and int(Cc.sum()) == 0           # nothing was decoded, nothing written
