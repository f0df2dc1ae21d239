"""Pins the plain-C GradDrop ("DGC") oracle (CPU only): brute force on small
inputs with numpy's full sort, the closed-form sample index stream, the
invariants gd_body.h implies, and the reference's own functors where built."""
import numpy as np
import pytest

A2, C2 = 3265436265, 3554416254   # two LCG steps: x2 = A2*s + C2 (mod 2^32)


def _brute_force(g, r0, sample_rate, drop_ratio, seed):
    """Independent numpy statement of gd_body.h:102-232 (sorts instead of selects)."""
    n = g.size
    s = 1 - drop_ratio
    sample_cnt = int(np.ceil(n * sample_rate))
    expected = int(np.ceil(n * s))
    r = (g + r0).astype(np.float32)
    x = (seed + np.arange(sample_cnt, dtype=np.uint64)) & np.uint64(0xFFFFFFFF)
    idx = ((x * np.uint64(A2) + np.uint64(C2)) & np.uint64(0xFFFFFFFF)) % np.uint64(n)
    sample = np.sort(np.abs(r[idx.astype(np.int64)]))[::-1]
    thr = sample[int(sample_cnt * s)]
    cand = np.flatnonzero((r > thr) | (r < -thr))
    total = cand.size
    if total > expected:
        order = np.lexsort((cand, -np.abs(r[cand]).astype(np.float64)))  # |r| descending, ties by index
        cand = cand[order][:expected]
    vals = r[cand].copy()
    r[cand] = 0
    return cand.astype(np.int32), vals, r, thr, total


@pytest.mark.parametrize("n,sr,dr", [(1000, 0.05, 0.99), (4096, 0.01, 0.999), (10007, 0.1, 0.9), (100003, 0.01, 0.999),
                                     (65536, 0.5, 0.5), (300007, 0.02, 0.97), (5000, 1.0, 0.999)])
def test_gd_encode_matches_brute_force(oracle_cpu, n, sr, dr):
    rng = np.random.default_rng(n)
    for seed in (0, 1, 12345, 2**40 + 5, 2**64 - 2):
        g = rng.laplace(0, 1e-3, n).astype(np.float32)
        r0 = rng.normal(0, 1e-4, n).astype(np.float32)
        g_copy, r = g.copy(), r0.copy()
        msg, info = oracle_cpu.gd_encode(g, r, sr, dr, seed)
        idx, val, r_ref, thr, total = _brute_force(g, r0, sr, dr, seed)
        assert np.array_equal(g, g_copy)
        assert info["candidates"] == total and info["threshold"] == thr
        oi, ov = oracle_cpu.gd_split(msg)
        assert msg[:4].view(np.int32)[0] == 4 + 8 * idx.size == msg.size
        assert np.array_equal(oi, idx) and np.array_equal(ov.view(np.uint32), val.view(np.uint32))
        assert np.array_equal(r.view(np.uint32), r_ref.view(np.uint32))


def test_gd_sizes_and_index_stream(oracle_cpu):
    # config 3: N = 138,357,544, sample 1 %, drop 99.9 %
    assert oracle_cpu.gd_sizes(138_357_544, 0.01, 0.999) == (1_383_576, 138_358, 1383)
    for seed in (0, 7, 2**32 - 1, 2**50):
        for x in (0, 1, 99, 1_000_000):
            for n in (1000, 138_357_544):
                s = (seed + x) & 0xFFFFFFFF
                assert oracle_cpu.gd_sample_index(seed, x, n) == ((A2 * s + C2) & 0xFFFFFFFF) % n


def test_gd_invariants(oracle_cpu):
    rng = np.random.default_rng(5)
    n, sr, dr = 200003, 0.02, 0.995
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    r0 = rng.normal(0, 1e-4, n).astype(np.float32)
    for seed in range(6):
        r = r0.copy()
        msg, info = oracle_cpu.gd_encode(g, r, sr, dr, seed)
        idx, val = oracle_cpu.gd_split(msg)
        acc = (g + r0).astype(np.float32)
        _, expected, _ = oracle_cpu.gd_sizes(n, sr, dr)
        assert idx.size == min(info["candidates"], expected) == info["kept"]
        assert np.unique(idx).size == idx.size                      # indices unique
        assert np.all(np.abs(val) > info["threshold"])              # every selected |v| > thr
        rebuilt = r.copy(); rebuilt[idx] += val                     # R_after + scatter == R_before + G, exactly
        assert np.array_equal(rebuilt.view(np.uint32), acc.view(np.uint32))
        assert np.all(r[idx] == 0)
        if info["candidates"] > expected:                           # cut: kept dominate the rejected candidates
            rejected = np.setdiff1d(np.flatnonzero(np.abs(acc) > info["threshold"]), idx)
            assert np.abs(val).min() >= np.abs(acc[rejected]).max()
            assert np.all(np.diff(np.abs(val)) <= 0)                # descending |v|
        else:
            assert np.all(np.diff(idx) > 0)                         # ascending index
        # decode (write) of the message is the masked accumulated tensor
        out = np.full(n, 3.0, np.float32)
        assert oracle_cpu.gd_decode(msg, out, 0) == 0
        mask = np.zeros(n, bool); mask[idx] = True
        assert np.array_equal(out, np.where(mask, acc, 0).astype(np.float32))
        base = rng.normal(0, 1, n).astype(np.float32)
        out = base.copy()
        assert oracle_cpu.gd_decode(msg, out, 1) == 0
        exp = base.copy(); exp[idx] += val
        assert np.array_equal(out, exp)


def test_gd_decode_short_message_and_empty(oracle_cpu):
    n = 5000
    rng = np.random.default_rng(1)
    g = rng.laplace(0, 1e-3, n).astype(np.float32); r = np.zeros(n, np.float32)
    msg, _ = oracle_cpu.gd_encode(g, r, 0.05, 0.99, 3)
    out = np.ones(n, np.float32)
    assert oracle_cpu.gd_decode(msg, out, 0, in_size=msg.size - 1) == -1     # gd_body.h:317-325
    assert np.all(out == 1)
    empty = np.array([4, 0, 0, 0], np.uint8)                                   # k == 0: header only
    assert oracle_cpu.gd_decode(empty, out, 0) == 0 and np.all(out == 0)


def test_gd_all_zero_gradient_selects_nothing(oracle_cpu):
    n = 4096
    g = np.zeros(n, np.float32); r = np.zeros(n, np.float32)
    msg, info = oracle_cpu.gd_encode(g, r, 0.05, 0.99, 0)
    assert msg.size == 4 and info["kept"] == 0


def test_gd_decode_against_numpy_scatter(oracle_cpu):
    # gd_r_body, gd_body.h:283-353: write mode clears the whole output and scatters, add mode accumulates
    # (indices inside one message are unique, so numpy's fancy-index update is the same operation); a message
    # longer than the bytes provided is refused with -1 before anything is written (gd_body.h:317-325)
    rng = np.random.default_rng(3)
    for n in (1000, 100003):
        g = rng.laplace(0, 1e-3, n).astype(np.float32); r = np.zeros(n, np.float32)
        m, _ = oracle_cpu.gd_encode(g, r, 0.05, 0.99, 3)
        idx, val = oracle_cpu.gd_split(m)
        assert np.unique(idx).size == idx.size
        for add in (0, 1):
            base = rng.normal(0, 1, n).astype(np.float32)
            a = base.copy()
            want = base.copy() if add else np.zeros(n, np.float32)
            if add:
                want[idx] = val + want[idx]
            else:
                want[idx] = val
            assert oracle_cpu.gd_decode(m, a, add) == 0
            assert np.array_equal(a.view(np.uint32), want.view(np.uint32))
        untouched = base.copy()
        assert oracle_cpu.gd_decode(m, untouched, 0, in_size=m.size - 1) == -1
        assert np.array_equal(untouched, base)


# ---- the sparsifier without residual (dgc_body.h) ------------------------------------------------
def _brute_force_dgc(g0, sample_rate, s_percent, seed):
    """Independent numpy statement of dgc_body.h:71-152."""
    n = g0.size
    sample_cnt = int(np.ceil(n * sample_rate))
    expected = int(np.ceil(n * s_percent))
    g = g0.copy()
    x = (seed + np.arange(sample_cnt, dtype=np.uint64)) & np.uint64(0xFFFFFFFF)
    idx = ((x * np.uint64(A2) + np.uint64(C2)) & np.uint64(0xFFFFFFFF)) % np.uint64(n)
    sample = np.sort(np.abs(g[idx.astype(np.int64)]))[::-1]
    thr = sample[int(sample_cnt * s_percent)]
    cand = np.flatnonzero((g > thr) | (g < -thr))
    total = cand.size
    if total > expected:
        order = np.lexsort((cand, -np.abs(g[cand]).astype(np.float64)))
        cand = cand[order][:expected]
    vals = g[cand].copy()
    g[cand] = 0
    return cand.astype(np.int32), vals, g, thr, total


@pytest.mark.parametrize("n,sr,sp", [(1000, 0.05, 0.01), (4096, 0.01, 0.001), (10007, 0.1, 0.1), (100003, 0.01, 0.001),
                                     (65536, 0.5, 0.5), (300007, 0.02, 0.03)])
def test_dgc_encode_matches_brute_force(oracle_cpu, n, sr, sp):
    rng = np.random.default_rng(n + 7)
    cuts = set()
    for seed in (0, 1, 12345, 2**40 + 5, 2**64 - 2):
        g0 = rng.laplace(0, 1e-3, n).astype(np.float32)
        g = g0.copy()
        msg, info = oracle_cpu.dgc_encode(g, sr, sp, seed)
        idx, val, g_ref, thr, total = _brute_force_dgc(g0, sr, sp, seed)
        assert info["candidates"] == total and info["threshold"] == thr
        oi, ov = oracle_cpu.gd_split(msg)
        assert msg[:4].view(np.int32)[0] == 4 + 8 * idx.size == msg.size
        assert np.array_equal(oi, idx) and np.array_equal(ov.view(np.uint32), val.view(np.uint32))
        assert np.array_equal(g.view(np.uint32), g_ref.view(np.uint32))
        cuts.add(total > idx.size)


def test_dgc_equals_graddrop_with_zero_residual(oracle_cpu):
    # R = 0 + G is G itself (except that -0.0 becomes +0.0), so GradDrop with a zero residual and
    # s = 1 - drop_ratio must produce the same message and leave R as DGC leaves G.
    rng = np.random.default_rng(5)
    for n, sr, dr in ((50_000, 0.02, 0.99), (200_001, 0.01, 0.999), (8192, 0.3, 0.75)):
        g0 = rng.laplace(0, 1e-3, n).astype(np.float32)
        g0[g0 == 0] = 1e-9
        for seed in (3, 2**33 + 1):
            r = np.zeros(n, np.float32)
            m_gd, i_gd = oracle_cpu.gd_encode(g0, r, sr, dr, seed)
            g = g0.copy()
            m_dgc, i_dgc = oracle_cpu.dgc_encode(g, sr, 1 - dr, seed)
            assert np.array_equal(m_gd, m_dgc) and i_gd == i_dgc
            assert np.array_equal(r.view(np.uint32), g.view(np.uint32))


def test_dgc_decode_write_mode_keeps_other_entries(oracle_cpu):
    rng = np.random.default_rng(6)
    n = 10_000
    g = rng.laplace(0, 1e-3, n).astype(np.float32)
    msg, info = oracle_cpu.dgc_encode(g.copy(), 0.05, 0.01, 9)
    idx, val = oracle_cpu.gd_split(msg)
    base = rng.normal(0, 1, n).astype(np.float32)
    out = base.copy()
    assert oracle_cpu.dgc_decode(msg, out, 0) == 0                 # dgc_body.h:283-289: no zero fill
    want = base.copy(); want[idx] = val
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    out = base.copy()
    assert oracle_cpu.dgc_decode(msg, out, 1) == 0
    want = base.copy(); want[idx] += val
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert oracle_cpu.dgc_decode(msg, out, 0, in_size=msg.size - 1) == -1   # dgc_body.h:268-274
