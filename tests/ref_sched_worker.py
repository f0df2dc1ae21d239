"""One algorithm's worth of tasks through the REFERENCE'S OWN scheduler (hp_cuda.cpp:163-1080, built over this
library's drivers by oracle/ref_host.py into oracle/_ref/), checked against the CPU oracle bit for bit.

Run as `python tests/ref_sched_worker.py <terngrad|tbq|graddrop|powersgd>` in a process of its own: the reference's
module keeps its algorithm, its threads and its streams in statics, chosen at the first `init` (hp_cuda.cpp:3-12,
:789, :814).  tests/test_gpu_reference_scheduler.py starts one such process per algorithm.  The environment variable
HPX_CLOCK_SEED stands in for the wall clock the drivers seed from, so stochastic rounding and GradDrop's sample are
the oracle's.  Prints `OK <alg>` and exits 0 when everything matched.

What this exercises that no other test does: the reference's stream usage around the drivers — the driver on the
shared compute stream (or the null stream: hp_cuda_gd), the copy of B into C on the thread's data stream straight
afterwards with no event in between (hp_cuda.cpp:284-313, :464-481, :610-622), five host threads calling the
drivers at once for every algorithm but TBQ (:843-852, :875-881).
"""
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, os.path.join(ROOT, "oracle", "_ref"))

SEED = 77


def _collect(hp, task_id, names, timeout_s=60.0):
    got, t0 = [], time.time()
    while len(got) < len(names) and time.time() - t0 < timeout_s:
        got += hp.getResults(task_id)                        # the reference has no blocking wait: poll as its users do
        time.sleep(0.001)
    assert sorted(got) == sorted(names), (task_id, sorted(got), sorted(names))


def _cbuf(nbytes, pinned):
    return torch.zeros(nbytes, dtype=torch.uint8, pin_memory=bool(pinned))


def _eq(a, b, what):
    from gpu_util import assert_bits_equal
    assert_bits_equal(a, b, what)


def run_terngrad(hp, cpu):
    from gpu_util import dev, host
    rng = np.random.default_rng(11)
    b, size, rank = 2, 3, 1
    assert hp.init("terngrad", {"enable_random": 1, "bitwidth": b}, 0, rank, size)
    comp, dec, root = [], [], []
    # COMP: sizes on both sides of the single-launch encode's range, so that two-launch and resident launches mix
    for k, n in enumerate([25_557_032, 3_000_001, 6_500_000, 400_003, 11_000_000, 70_001, 2_100_000, 5_000_001]):
        x = rng.normal(0, 1e-2, n).astype(np.float32)
        mb = cpu.terngrad_packed_size(n, b)
        comp.append((f"comp{k}", x, dev(x), torch.full((mb,), 0x5A, dtype=torch.uint8, device="cuda"), _cbuf(mb, k & 1)))
    for k, n in enumerate([4_000_003, 900_000, 7_000_001, 50_001]):
        src = rng.normal(0, 1e-2, n).astype(np.float32)
        rc, msg = cpu.terngrad_encode(src, b, 1, 500 + k)
        base = rng.normal(0, 1, n).astype(np.float32)
        C = _cbuf(msg.size, k & 1); C.numpy()[:] = msg
        dec.append((f"dec{k}", msg, base, dev(base), torch.zeros(msg.size, dtype=torch.uint8, device="cuda"), C, k & 1))
    for k, n in enumerate([3_000_002, 1_000_001, 8_000_003]):
        mb = cpu.terngrad_packed_size(n, b)
        slots = np.zeros(size * mb, np.uint8)
        for i in range(size):
            rc, m = cpu.terngrad_encode(rng.normal(0, 1e-2, n).astype(np.float32), b, 1, 900 + 10 * k + i)
            slots[i * mb:(i + 1) * mb] = m
        slots[rank * mb:(rank + 1) * mb] = 0xEE              # our own slot: never read
        mine = rng.normal(0, 1e-2, n).astype(np.float32)
        C = _cbuf(size * mb, k & 1); C.numpy()[:] = slots
        root.append((f"root{k}", slots, mine, dev(mine), torch.zeros(mb, dtype=torch.uint8, device="cuda"), C))
    torch.cuda.synchronize()
    for name, x, dx, B, C in comp:
        assert hp.submit_task(name, dx, B, C, 0, 10)
    for name, msg, base, dt, B, C, is_root in dec:
        assert hp.submit_task(name, dt, B, C, is_root, 20)
    for name, slots, mine, dm, B, C in root:
        assert hp.submit_task(name, dm, B, C, 1, 30)
    _collect(hp, 10, [c[0] for c in comp]); _collect(hp, 20, [d[0] for d in dec]); _collect(hp, 30, [r[0] for r in root])
    # what C holds at the moment the name was published is what a consumer reads: compare it before any sync
    for name, x, dx, B, C in comp:
        rc, ref = cpu.terngrad_encode(x, b, 1, SEED)
        _eq(C.numpy(), ref, f"{name}: COMP message in C")
    torch.cuda.synchronize()
    for name, msg, base, dt, B, C, is_root in dec:
        rc, want = cpu.terngrad_decode(msg, base.size, base.copy(), is_root)
        _eq(host(dt), want, f"{name}: DECOMP is_root={is_root}")
    for name, slots, mine, dm, B, C in root:
        n = mine.size
        mb = cpu.terngrad_packed_size(n, b)
        want = mine.copy()
        for i in range(size):
            if i != rank:
                rc, want = cpu.terngrad_decode(slots[i * mb:(i + 1) * mb], n, want, 1)
        _eq(host(dm), want, f"{name}: ROOT gradient")
        rc, ref = cpu.terngrad_encode(want, b, 1, SEED)
        _eq(C.numpy()[:mb], ref, f"{name}: ROOT message in C")


def run_tbq(hp, cpu):
    from gpu_util import dev, host
    rng = np.random.default_rng(12)
    thr, size, rank = 2e-3, 4, 2
    assert hp.init("tbq", {"threshold": thr}, 0, rank, size)
    checks, keep = [], []
    sizes = [int(s) for s in rng.integers(1 << 20, 6 << 20, 15)] + [5, 4099, 70_001]
    for k, n in enumerate(sizes):
        kind = (10, 20, 30)[k % 3]
        mb = cpu.tbq_packed_size(n)
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        r = rng.normal(0, 1e-3, n).astype(np.float32)
        dg, dr = dev(g), dev(r)
        B = torch.zeros(mb, dtype=torch.uint8, device="cuda")
        if kind == 10:
            C, extra = _cbuf(mb, k & 1), None
        elif kind == 20:
            extra = cpu.tbq_encode(rng.normal(0, 1e-3, n).astype(np.float32), np.zeros(n, np.float32), thr)
            C = _cbuf(mb, k & 1); C.numpy()[:] = extra
        else:
            extra = np.zeros(size * mb, np.uint8)
            for i in range(size):
                extra[i * mb:(i + 1) * mb] = cpu.tbq_encode(rng.normal(0, 2e-3, n).astype(np.float32), np.zeros(n, np.float32), thr)
            C = _cbuf(size * mb, k & 1); C.numpy()[:] = extra
        checks.append((kind, f"t{k}", g, r, dg, dr, C, extra)); keep.append(B)
    torch.cuda.synchronize()
    for (kind, name, g, r, dg, dr, C, extra), B in zip(checks, keep):
        assert hp.submit_task(name, dg, dr, B, C, 1, kind)
    for kind in (10, 20, 30):
        _collect(hp, kind, [c[1] for c in checks if c[0] == kind])
    for kind, name, g, r, dg, dr, C, extra in checks:
        n = g.size
        mb = cpu.tbq_packed_size(n)
        if kind == 10:
            rr = r.copy()
            msg = cpu.tbq_encode(g, rr, thr)
            _eq(C.numpy(), msg, f"{name}: COMP message"); _eq(host(dr), rr, f"{name}: residual"); _eq(host(dg), g, f"{name}: gradient")
        elif kind == 20:
            _eq(host(dg), cpu.tbq_decode(extra, n, thr, g.copy(), 1), f"{name}: DECOMP add")
        else:
            want = g.copy()
            for i in range(size):
                if i != rank:
                    want = cpu.tbq_decode(extra[i * mb:(i + 1) * mb], n, thr, want, 1)
            rr = r.copy()
            msg = cpu.tbq_encode(want, rr, thr)
            _eq(host(dg), want, f"{name}: ROOT gradient"); _eq(host(dr), rr, f"{name}: ROOT residual")
            _eq(C.numpy()[:mb], msg, f"{name}: ROOT message")


def run_graddrop(hp, cpu):
    from gpu_util import dev, host
    rng = np.random.default_rng(13)
    sr, drop, size, rank = 0.01, 0.999, 3, 0
    assert hp.init("graddrop", {"sample_rate": sr, "drop_ratio": drop}, 0, rank, size)
    csize = lambda n: 4 + int(2 * np.ceil(n * (1 - drop))) * 4          # hp_cuda.cpp:230
    comp, dec, root = [], [], []
    for k, n in enumerate([9_000_001, 3_000_003, 12_000_000, 1_200_000, 600_000, 5_000_001]):
        g = rng.laplace(0, 1e-3, n).astype(np.float32)
        r = rng.normal(0, 1e-4, n).astype(np.float32)
        comp.append((f"comp{k}", g, r, dev(g), dev(r), torch.full((csize(n),), 0xEE, dtype=torch.uint8, device="cuda"), _cbuf(csize(n), k & 1)))
    for k, n in enumerate([4_000_003, 2_000_000]):
        msg, _ = cpu.gd_encode(rng.laplace(0, 1e-3, n).astype(np.float32), np.zeros(n, np.float32), sr, drop, 300 + k)
        base = rng.normal(0, 1, n).astype(np.float32)
        C = _cbuf(csize(n), k & 1); C.numpy()[:msg.size] = msg
        dec.append((f"dec{k}", msg, base, dev(base), dev(np.zeros(n, np.float32)), torch.zeros(csize(n), dtype=torch.uint8, device="cuda"), C, k & 1))
    for k, n in enumerate([6_000_001, 2_500_000]):
        cs = csize(n)
        slots = np.zeros(size * cs, np.uint8)
        for i in range(size):
            m, _ = cpu.gd_encode(rng.laplace(0, 1e-3, n).astype(np.float32), np.zeros(n, np.float32), sr, drop, 700 + 10 * k + i)
            slots[i * cs:i * cs + m.size] = m
        mine = rng.laplace(0, 1e-3, n).astype(np.float32)
        res = rng.normal(0, 1e-4, n).astype(np.float32)
        C = _cbuf(size * cs, k & 1); C.numpy()[:] = slots
        root.append((f"root{k}", slots, mine, res, dev(mine), dev(res), torch.full((cs,), 0xEE, dtype=torch.uint8, device="cuda"), C))
    torch.cuda.synchronize()
    for name, g, r, dg, dr, B, C in comp:
        assert hp.submit_task(name, dg, dr, B, C, 0, 10)
    for name, msg, base, dt, dres, B, C, is_root in dec:
        assert hp.submit_task(name, dt, dres, B, C, is_root, 20)
    for name, slots, mine, res, dm, dres, B, C in root:
        assert hp.submit_task(name, dm, dres, B, C, 1, 30)
    _collect(hp, 10, [c[0] for c in comp]); _collect(hp, 20, [d[0] for d in dec]); _collect(hp, 30, [r[0] for r in root])
    cut = []
    for name, g, r, dg, dr, B, C in comp:
        rr = r.copy()
        msg, info = cpu.gd_encode(g, rr, sr, drop, SEED)
        cut.append(info["candidates"] > info["kept"])
        _eq(C.numpy()[:msg.size], msg, f"{name}: COMP message in C")
    torch.cuda.synchronize()
    for name, g, r, dg, dr, B, C in comp:
        rr = r.copy(); cpu.gd_encode(g, rr, sr, drop, SEED)
        _eq(host(dr), rr, f"{name}: residual"); _eq(host(dg), g, f"{name}: gradient untouched")
    assert any(cut) and not all(cut), cut
    for name, msg, base, dt, dres, B, C, is_root in dec:
        want = base.copy(); cpu.gd_decode(msg, want, is_root)
        _eq(host(dt), want, f"{name}: DECOMP is_root={is_root}")
    for name, slots, mine, res, dm, dres, B, C in root:
        n, cs = mine.size, csize(mine.size)
        want = mine.copy()
        for i in range(size):
            if i != rank:
                cpu.gd_decode(slots[i * cs:(i + 1) * cs], want, 1)
        rr = res.copy()
        msg, _ = cpu.gd_encode(want, rr, sr, drop, SEED)
        _eq(C.numpy()[:msg.size], msg, f"{name}: ROOT message in C")
        _eq(host(dm), want, f"{name}: ROOT gradient"); _eq(host(dres), rr, f"{name}: ROOT residual")


def run_powersgd(hp, cpu):
    import importlib
    from gpu_util import host
    pkg = importlib.import_module("torch-hipress-extension_amd")
    shapes, rk = [(4096, 4096), (1024, 4096), (4096, 1024), (130, 515)] * 2, 4
    assert hp.init("powersgd", {"matrix_approximation_rank": rk}, 0, 0, 2)

    def fresh():
        g = torch.Generator(device="cuda").manual_seed(8)
        G = [torch.randn(a * b, device="cuda", generator=g) * 1e-2 for a, b in shapes]
        R = [torch.randn(a * b, device="cuda", generator=g) * 1e-3 for a, b in shapes]
        Q = [torch.randn(b, rk, device="cuda", generator=g) for a, b in shapes]
        M = [torch.zeros(a, b, device="cuda") for a, b in shapes]
        P = [torch.zeros(a, rk, device="cuda") for a, b in shapes]
        return G, R, Q, M, P
    G1, R1, Q1, M1, P1 = fresh()
    torch.cuda.synchronize()
    names = [f"w{i}" for i in range(len(shapes))]
    other, seen = torch.cuda.Stream(), {}
    for task_id in (40, 50, 60):
        for i, nm in enumerate(names):
            assert hp.submit_task(nm, G1[i], R1[i], M1[i], P1[i], Q1[i], task_id)
        _collect(hp, task_id, names)
        with torch.cuda.stream(other):                       # a consumer on a stream of its own, right after the names
            seen[task_id] = [t.clone() for t in {40: P1, 50: Q1, 60: G1}[task_id]]
    other.synchronize()
    G2, R2, Q2, M2, P2 = fresh()
    assert pkg.hp_cuda_powersgd_encode1(G2, R2, Q2, M2, P2) == 0
    torch.cuda.synchronize()
    P0 = [p.clone() for p in P2]
    assert pkg.hp_cuda_powersgd_encode2(P2, M2, Q2) == 0
    assert pkg.hp_cuda_powersgd_decode(P2, Q2, M2, R2, G2) == 0
    torch.cuda.synchronize()
    for i in range(len(shapes)):
        _eq(host(seen[40][i]).ravel(), host(P0[i]).ravel(), f"P[{i}] after encode1 as the consumer saw it")
        _eq(host(seen[50][i]).ravel(), host(Q2[i]).ravel(), f"Q[{i}] after encode2 as the consumer saw it")
        _eq(host(seen[60][i]).ravel(), host(G2[i]).ravel(), f"grad[{i}] after decode as the consumer saw it")
        _eq(host(R1[i]).ravel(), host(R2[i]).ravel(), f"residual[{i}]")


def main():
    alg = sys.argv[1]
    os.environ.setdefault("HPX_CLOCK_SEED", str(SEED))
    assert int(os.environ["HPX_CLOCK_SEED"]) == SEED
    from oracle import cpu
    cpu.lib()
    import hp_cuda as hp                                      # oracle/_ref/: the reference's module over libhpx.so
    assert "oracle/_ref" in hp.__file__.replace(os.sep, "/"), hp.__file__
    torch.cuda.set_device(0)
    print(f"reference scheduler, algorithm {alg}", flush=True)
    try:
        {"terngrad": run_terngrad, "tbq": run_tbq, "graddrop": run_graddrop, "powersgd": run_powersgd}[alg](hp, cpu)
    finally:
        hp.end()
    torch.cuda.synchronize()
    print(f"OK {alg}", flush=True)


if __name__ == "__main__":
    main()
