"""Writes tests/golden/hotpath_vectors.npz: small input/output vectors of the hot path, written by the CPU oracle
(oracle/hpx_oracle.c through oracle/cpu.py).

    python tests/golden/make_fixtures.py          # rewrites the file; --check only compares with the committed one

What the vectors are, and are not.  They are REGRESSION vectors: tests/test_golden.py holds the HIP kernels and
the oracle to them on every machine, so neither can drift unnoticed.  They do not pin the oracle to the
reference (the oracle wrote them); that is the job of the hand-derived known answers in tests/kat_vectors.py
and of the brute-force and invariant tests in tests/test_oracle_*.py.  History: the committed file was first
produced by a host build of the reference's own header bodies on rocThrust; that build had to replace one of
the reference's headers (get_policy_general.h, which includes Thrust's CUDA backend unconditionally) by a
stand-in, so it is not kept, and the reference counts as unbuildable here.  The oracle reproduces the committed
file array for array (--check).

The file holds plain numeric arrays only (numpy.load without pickle).

What each group is:
  tbq_<k>_*       tbq_body / tbq_r_body (tbq_body.h:90-200): g, r before -> packed bytes, r after; decode in
                  write and add mode
  tgd_<k>_*       terngrad_body with enable_random = 0 (terngrad_body.h:162-307): x -> whole message; decode
                  (terngrad_r_body, :309-409) in write and add mode
  tgr_<k>_*       compress_with_random (terngrad_body.h:60-99) with a fixed seed: x, min, 1/gap, seed -> payload
  gd_<k>_*        gd_body with the clock replaced by a seed (gd_body.h:102-232):
                  g, r before -> message, r after; gd_r_body (:283-353) in write and add mode
  lcg_*           naive_int_random / naive_real_random draws (naive_random.hpp:15-69)
"""
import os
import sys

import numpy as np


def base_values(n):
    """The decoders' pre-existing output contents: a formula, so that it need not be stored (exact in fp32)."""
    return ((np.arange(n, dtype=np.int64) * 7919) % 1000).astype(np.float32) / np.float32(8) - np.float32(60)


ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import cpu  # noqa: E402


def build_vectors():
    cpu.lib()
    rng = np.random.default_rng(20240607)
    out = {}

    # ---- TBQ ------------------------------------------------------------------------------------
    for k, (n, thr) in enumerate([(10, 2e-3), (2051, 2e-3), (7, 0.5), (1024, 1e-2)]):
        g = rng.normal(0, 1.5 * thr, n).astype(np.float32)
        r0 = rng.normal(0, 0.7 * thr, n).astype(np.float32)
        if n == 10:
            g = np.array([.003, -.003, .001, -.001, .002, -.002, 0, .0041, .5, -.5], np.float32)
            r0 = np.zeros(n, np.float32)
        r = r0.copy()
        packed = cpu.tbq_encode(g.copy(), r, thr)
        base = base_values(n)
        out.update({f"tbq_{k}_g": g, f"tbq_{k}_r0": r0, f"tbq_{k}_thr": np.float32(thr), f"tbq_{k}_packed": packed,
                    f"tbq_{k}_r1": r,
                    f"tbq_{k}_dec_write": cpu.tbq_decode(packed, n, thr, base.copy(), 0),
                    f"tbq_{k}_dec_add": cpu.tbq_decode(packed, n, thr, base.copy(), 1)})
    out["tbq_count"] = np.int32(4)

    # ---- TernGrad, round to nearest (whole body) ------------------------------------------------------
    cases = [(22, 2), (2048, 2), (2051, 2), (1001, 1), (1003, 4), (777, 8), (4097, 1)]
    for k, (n, b) in enumerate(cases):
        x = rng.normal(0, 1e-2, n).astype(np.float32)
        if n == 22:
            x = (np.array([(7 * i % 11) - 5 for i in range(22)], np.float32) * np.float32(0.01)).astype(np.float32)
        rc, msg = cpu.terngrad_encode(x.copy(), b, 0, 0)
        assert rc == 0
        base = base_values(n)
        out.update({f"tgd_{k}_x": x, f"tgd_{k}_bits": np.int32(b), f"tgd_{k}_msg": msg,
                    f"tgd_{k}_dec_write": cpu.terngrad_decode(msg, n, base.copy(), 0)[1],
                    f"tgd_{k}_dec_add": cpu.terngrad_decode(msg, n, base.copy(), 1)[1]})
    out["tgd_count"] = np.int32(len(cases))

    # ---- TernGrad, stochastic rounding (the reference's functor with a fixed seed) -------------------------
    cases = [(40, 2, 12345), (2048, 2, 0), (4000, 1, 2**32 - 3), (2000, 4, 2**40 + 17), (1000, 8, 2**64 - 1)]
    for k, (n, b, seed) in enumerate(cases):
        x = rng.normal(0, 1e-2, n).astype(np.float32)
        if n == 40:
            x = (np.array([(7 * i % 11) - 5 for i in range(40)], np.float32) * np.float32(0.01)).astype(np.float32)
        mn, mx = x.min(), x.max()
        gap = np.float32((mx - mn) / np.float32((1 << b) - 1.0))
        gi = np.float32(1.0 / (float(gap) + 1e-8))
        nbytes = n // (8 // b)
        rc, msg = cpu.terngrad_encode(x.copy(), b, 1, seed)
        assert rc == 0
        pay = msg[10:10 + nbytes].copy()
        out.update({f"tgr_{k}_x": x, f"tgr_{k}_bits": np.int32(b), f"tgr_{k}_seed": np.uint64(seed), f"tgr_{k}_min": mn,
                    f"tgr_{k}_gi": gi, f"tgr_{k}_payload": pay})
    out["tgr_count"] = np.int32(len(cases))

    # ---- GradDrop -------------------------------------------------------------------------------------------
    # (n, sample_rate, drop_ratio, seed, want_cut): the data is redrawn until the case takes the wanted branch
    cases = [(1000, 0.05, 0.99, 0, True), (4097, 0.1, 0.9, 12345, True), (3001, 0.3, 0.9, 2**40 + 5, False),
             (4096, 0.5, 0.5, 2**64 - 2, True), (2500, 0.4, 0.95, 7, False)]
    for k, (n, sr, dr, seed, want_cut) in enumerate(cases):
        for attempt in range(200):
            g = rng.laplace(0, 1e-3, n).astype(np.float32)
            r0 = rng.normal(0, 1e-4, n).astype(np.float32)
            r = r0.copy()
            msg, info = cpu.gd_encode(g.copy(), r, sr, dr, seed)
            if (info["candidates"] > info["kept"]) == want_cut:
                break
        else:
            raise SystemExit(f"no data found for GradDrop case {k}")
        base = base_values(n)
        w, a = base.copy(), base.copy()
        assert cpu.gd_decode(msg, w, 0) == 0 and cpu.gd_decode(msg, a, 1) == 0
        out.update({f"gd_{k}_g": g, f"gd_{k}_r0": r0, f"gd_{k}_sr": np.float64(sr), f"gd_{k}_dr": np.float64(dr),
                    f"gd_{k}_seed": np.uint64(seed), f"gd_{k}_msg": msg, f"gd_{k}_r1": r,
                    f"gd_{k}_candidates": np.int32(info["candidates"]), f"gd_{k}_dec_write": w,
                    f"gd_{k}_dec_add": a})
    out["gd_count"] = np.int32(len(cases))

    # ---- LCG -------------------------------------------------------------------------------------------------
    seeds = np.array([0, 1, 12345, 2**31, 2**32 - 1], np.uint64)
    out["lcg_seeds"] = seeds
    # draw 1 is the one srand() discards (naive_random.hpp:22-25); draws 2..6 are what the codecs use
    out["lcg_draws"] = np.array([[cpu.lcg_kth(int(s), k) for k in range(2, 7)] for s in seeds], np.uint32)
    out["lcg_real01"] = np.array([[cpu.u01_from_u32(cpu.lcg_kth(int(s), k)) for k in range(2, 7)] for s in seeds], np.float32)

    return out


def main():
    out = build_vectors()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hotpath_vectors.npz")
    if "--check" in sys.argv[1:]:
        old = np.load(path)
        assert sorted(old.files) == sorted(out), (sorted(set(old.files) ^ set(out)))
        for k in old.files:
            a, b = old[k], np.asarray(out[k])
            assert a.dtype == b.dtype and a.shape == b.shape and a.tobytes() == b.tobytes(), k
        print(f"{path}: all {len(out)} arrays reproduced")
        return
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
