#!/usr/bin/env python3
"""Benchmark of the gradient-compression hot path on ONE MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one encode + decode pass of the headline workload through the C ABI:
the TernGrad 2-bit quantiser on a ResNet-50-sized fp32 gradient (25,557,032
elements ~N(0,1e-2) with 0.1 % outliers at +-50 sigma, stochastic rounding with a
fixed seed, decode back to fp32).  Inputs are resident in HBM before the clock
starts.  Buffers rotate over several distinct sets so that a step never finds
its input in the 256 MB Infinity Cache from the step before.

Prints ONE JSON line:  value = GB/s of fp32 gradient (4*N bytes per step) over
the whole timed region; "roofline" prices the dominant kernel against the HBM
peak with its duration measured by HIP events on the launch stream;
"cpu_baseline" is the plain-C/OpenMP port of the reference's CPU bodies (the
oracle) timed on the host cores of the same box; "extra" carries the other
codecs of the path at their configuration sizes.
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
FP32_MFMA_PEAK_TF = 157.3   # MI355X dense fp32 matrix, published
N_TERNGRAD = 25_557_032
N_DGC = 138_357_544

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, each scaled by what the same
# counter reads for a plain copy of known size.
MEASURED_TRAFFIC_BYTES = {  # profiles/terngrad_pmc_fetch_write.txt (FETCH x1.99992 + WRITE x1.0, KiB -> bytes)
    "terngrad_resident_kernel": int((52115.5 * 1.99992 + 8303.5) * 1024),  # includes the grid-wide exchange's polls and records
    "terngrad_minmax_kernel": int((49939.6 * 1.99992 + 390.1) * 1024),
    "terngrad_quant_kernel": int((49993.8 * 1.99992 + 6434.5) * 1024),
    "terngrad_decode_kernel": int((3563.9 * 1.99992 + 99879.2) * 1024),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=4, help="distinct buffer sets rotated between steps")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="time budget of the CPU baseline leg")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_SECONDS * 1e3,
                    help="untimed run of each workload before it is measured (0 under a counter-collecting profiler: "
                         "counters do not care, and the trace stays small)")
    ap.add_argument("--no-extra", action="store_true", help="skip the TBQ / DGC / PowerSGD side measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="profiling aid: run just these side measurements (comma-separated names of "
                    "EXTRAS below, e.g. powersgd) and print them; no headline, no CPU leg")
    ap.add_argument("--copy-calibration", type=int, default=0,
                    help="also run this many plain 4*N-byte device copies (a kernel of known traffic for scaling "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


class Call:
    """A C-ABI call with its argument arrays marshalled once."""

    def __init__(self, fn, *args):
        self.fn, self.args = fn, args

    def __call__(self):
        rc = self.fn(*self.args)
        if rc:
            raise RuntimeError(f"{self.fn.__name__} returned {rc}")


SETTLE_SECONDS = 0.04


def settle(torch, fn, seconds=None):
    """Untimed: keeps the GPU busy with the workload itself for `seconds` before a measurement.  A measurement
    that starts within the first milliseconds of a workload reads 2-6 % low on this part (the same kernels get
    faster over the first tens of milliseconds of continuous work, then stay there); a job that runs for hours
    sees the settled rate."""
    t_end = time.perf_counter() + (SETTLE_SECONDS if seconds is None else seconds)
    while time.perf_counter() < t_end:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def timed(torch, fn, steps, warmup, settled=True):
    for _ in range(warmup):
        fn()
    if settled:
        settle(torch, fn)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def event_pairs(torch, fn, steps, warmup=3):
    """Per-step durations (s) from a pair of events recorded on the stream around each step (the launches are on
    torch's current stream): what the GPU spends between the start of a step's first kernel and the end of its last,
    hand-overs between the launches included, host launch time excluded as long as the queue stays ahead."""
    for _ in range(warmup):
        fn()
    settle(torch, fn)
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    for a, b in pairs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) * 1e-3 for a, b in pairs)


def quantiles(xs_sorted, scale=1e3, digits=5):
    n = len(xs_sorted)
    pick = lambda q: xs_sorted[min(n - 1, int(q * n))]
    return {"median": round(pick(0.5) * scale, digits), "p10": round(pick(0.1) * scale, digits),
            "p90": round(pick(0.9) * scale, digits), "min": round(xs_sorted[0] * scale, digits), "n": n}


def terngrad_phases(torch, np, L, fn, workgroups, launches=20):
    """Per-phase breakdown of the resident encode from the four wall-clock stamps each workgroup leaves
    (hpx_terngrad_phase_stamps; 100 MHz, so 0.01 us steps): for each launch, times are taken from the earliest entry
    stamp of the grid; reported are medians over `launches` launches of the min / median / max over workgroups."""
    buf = torch.zeros(4 * workgroups, dtype=torch.int64, device="cuda")
    rows = {k: [] for k in ("entry", "loaded_and_reduced", "exchange_passed", "last_store",
                            "load_phase", "exchange_phase", "quantise_phase")}
    try:
        if L.hpx_terngrad_phase_stamps(buf.data_ptr(), workgroups):
            return None
        for _ in range(3):
            fn()
        for _ in range(launches):
            buf.zero_()
            torch.cuda.synchronize()
            fn()
            torch.cuda.synchronize()
            t = buf.cpu().numpy().reshape(workgroups, 4).astype(np.float64)
            t = t[(t > 0).all(axis=1)]
            if not len(t):
                continue
            t0 = t[:, 0].min()
            rel = (t - t0) / 100.0    # us
            cols = {"entry": rel[:, 0], "loaded_and_reduced": rel[:, 1], "exchange_passed": rel[:, 2], "last_store": rel[:, 3],
                    "load_phase": rel[:, 1] - rel[:, 0], "exchange_phase": rel[:, 2] - rel[:, 1],
                    "quantise_phase": rel[:, 3] - rel[:, 2]}
            for k, v in cols.items():
                rows[k].append((v.min(), np.median(v), v.max()))
    finally:
        L.hpx_terngrad_phase_stamps(None, 0)
        torch.cuda.synchronize()
    if not rows["entry"]:
        return None
    out = {"unit": "us", "clock": "100 MHz wall clock, stamps per workgroup, time 0 = earliest entry of the launch",
           "launches": len(rows["entry"]), "workgroups": workgroups,
           "columns": "median over launches of [min, median, max] over workgroups"}
    for k, v in rows.items():
        a = np.median(np.array(v), axis=0)
        out[k] = [round(float(x), 2) for x in a]
    return out


def kernel_times(torch, capi, fn, names, reps=10):
    """Average duration (s) of each named kernel: HIP events attached to each launch on its stream (begin and end of the kernel itself)."""
    L = capi.load()
    settle(torch, fn)
    torch.cuda.synchronize()
    L.hpx_profile_reset()
    L.hpx_profile_enable(1)
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    L.hpx_profile_enable(0)
    out = {}
    for k in names:
        ms, n = capi.profile_query(k)
        out[k] = (ms / n) * 1e-3 if n else None
    L.hpx_profile_reset()
    return out


def outlier_gradient(torch, n, gen):
    x = torch.randn(n, device="cuda", generator=gen) * 1e-2
    pos = torch.randint(0, n, (n // 1000,), device="cuda", generator=gen)
    x[pos] = torch.where(torch.rand(pos.numel(), device="cuda", generator=gen) < 0.5, 0.5, -0.5)
    return x


def main():
    args = parse()
    global SETTLE_SECONDS
    SETTLE_SECONDS = max(0.0, args.settle_ms) / 1e3
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path has no inter-GPU communication; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    import __graft_entry__
    __graft_entry__.ensure_built()     # loads what is built; builds only if nothing is
    pkg = importlib.import_module("torch-hipress-extension_amd")
    capi = pkg._capi
    L = capi.load()
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(0)
    if args.only:
        names = [w for w in args.only.split(",") if w]
        print(json.dumps({"only": names, "extra": extra(torch, np, capi, L, stream, gen, names)}), flush=True)
        return

    # ---- headline: TernGrad 2-bit encode + decode, N = 25,557,032 --------------------------
    n = N_TERNGRAD
    msg_bytes = 10 + (n + 3) // 4
    sets = []
    for s in range(max(1, args.sets)):
        x = outlier_gradient(torch, n, gen)
        msg = torch.zeros(msg_bytes, dtype=torch.uint8, device="cuda")
        dec = torch.empty(n, device="cuda")
        enc = Call(L.hpx_terngrad_encode, 1, capi.ptr_array([x.data_ptr()]), capi.i32_array([n]),
                   capi.ptr_array([msg.data_ptr()]), capi.i32_array([msg_bytes]), capi.u8_array([2]),
                   capi.i32_array([1]), capi.u64_array([0]), stream)
        dcd = Call(L.hpx_terngrad_decode, 1, capi.ptr_array([dec.data_ptr()]), capi.i32_array([n]),
                   capi.ptr_array([msg.data_ptr()]), capi.i32_array([msg_bytes]), capi.i32_array([0]), stream)
        sets.append((x, msg, dec, enc, dcd))
    state = {"i": 0}

    def step():
        _, _, _, enc, dcd = sets[state["i"] % len(sets)]
        state["i"] += 1
        enc()
        dcd()

    for _ in range(args.copy_calibration):
        sets[0][2].copy_(sets[0][0])  # reads 4*N bytes, writes 4*N bytes
    # the same K steps once more, first, straight after the W warm-up steps of a process that has done nothing yet:
    # reported beside the settled figure (path_roofline.cold_start_ms_per_step), never as `value`
    sec_cold = timed(torch, step, args.steps, args.warmup, settled=False)
    sec = timed(torch, step, args.steps, args.warmup)
    value = 4.0 * n / sec / 1e9

    def warm_step():
        sets[0][3]()
        sets[0][4]()

    sec_warm = timed(torch, warm_step, max(20, args.steps // 4), 5)
    def only(which):
        def f():
            state["i"] += 1
            sets[state["i"] % len(sets)][which]()
        return f

    sec_enc = timed(torch, only(3), max(20, args.steps // 4), 5)
    sec_dec = timed(torch, only(4), max(20, args.steps // 4), 5)
    pairs = event_pairs(torch, step, max(20, min(args.steps, 200)))
    pairs_enc = event_pairs(torch, only(3), 40)
    pairs_dec = event_pairs(torch, only(4), 40)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    phases = terngrad_phases(torch, np, L, only(3), cus)

    kt = kernel_times(torch, capi, step,
                      ["terngrad_resident_kernel", "terngrad_minmax_kernel", "terngrad_quant_kernel", "terngrad_decode_kernel"])
    alg_bytes = {  # algorithmic bytes per launch: every distinct input byte once, every output byte once
        "terngrad_resident_kernel": 4.0 * n + msg_bytes,   # x once in, message out
        "terngrad_minmax_kernel": 4.0 * n,
        "terngrad_quant_kernel": 4.0 * n + msg_bytes,
        "terngrad_decode_kernel": msg_bytes + 4.0 * n,
    }
    dom = max(alg_bytes, key=lambda k: kt[k] or 0.0)
    achieved = alg_bytes[dom] / kt[dom] / 1e9
    roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(dom),
                "traffic_is": "not read in this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by a plain "
                              "copy's readings, from profiles/terngrad_pmc_fetch_write.txt",
                "algorithmic_bytes_per_launch": alg_bytes[dom], "avg_launch_us": round(kt[dom] * 1e6, 2),
                "kernel_us": {k: (round(v * 1e6, 2) if v else None) for k, v in kt.items()}}
    path_alg = 8.5 * n  # x once in, codes out; codes in, fp32 out
    path = {"algorithmic_bytes_per_step": path_alg, "achieved_GBps": round(path_alg / sec / 1e9, 1),
            "frac_of_hbm_peak": round(path_alg / sec / 1e9 / HBM_PEAK_GBS, 4),
            "warm_cache_ms_per_step": round(sec_warm * 1e3, 4), "encode_ms": round(sec_enc * 1e3, 4),
            "decode_ms": round(sec_dec * 1e3, 4), "buffer_sets": len(sets),
            "wall_clock_mean_ms_per_step": round(sec * 1e3, 5),
            "cold_start_ms_per_step": round(sec_cold * 1e3, 5),
            "cold_start_frac_of_hbm_peak": round(path_alg / sec_cold / 1e9 / HBM_PEAK_GBS, 4),
            "event_pair_ms_per_step": quantiles(pairs), "event_pair_encode_ms": quantiles(pairs_enc),
            "event_pair_decode_ms": quantiles(pairs_dec),
            "frac_of_hbm_peak_event_pair_median": round(path_alg / quantiles(pairs, 1.0, 9)["median"] / 1e9 / HBM_PEAK_GBS, 4)}

    result = {
        "metric": "encode+decode GB/s of fp32 gradient (TernGrad 2-bit, 1 GPU)", "value": round(value, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": SETTLE_SECONDS * 1e3,   # untimed: the workload itself, run for this long after the warm-up steps, before every measurement
        "ms_per_step": round(sec * 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "terngrad_2bit_resnet50", "elements": n, "bitwidth": 2, "enable_random": 1, "seed": 0,
                   "outliers": "0.1% at +-50 sigma", "decode": "write"},
        "roofline": roofline, "path_roofline": path,
    }

    del sets
    torch.cuda.empty_cache()
    result["plain_streams"] = plain_streams(torch, stream, n)

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(np, n, args.cpu_seconds)
    if not args.no_extra:
        result["extra"] = extra(torch, np, capi, L, stream, gen)
    if phases:
        result.setdefault("extra", {})["terngrad_phases_us"] = phases
    print(json.dumps(result), flush=True)


def plain_streams(torch, stream, n):
    """What the memory system gives the simplest kernels of the codecs' shapes (bench_probe.hip, built beside this
    file; not part of the product library), measured the way the headline's kernels are: buffers rotate over
    distinct sets, every launch carries a pair of events that take the kernel's own begin and end.  The TernGrad
    step reads 4*n bytes once and writes 4*n bytes once, so read + write of 4*n bytes is the kernel time below which
    no encode+decode of this tensor can go on this part."""
    import __graft_entry__
    probe = C.CDLL(__graft_entry__.BENCH_PROBE)
    probe.bench_probe_stream_timed.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int]
    probe.bench_probe_elapsed_us.restype = C.c_double
    names = {0: "read", 1: "write_streaming", 2: "write_plain", 3: "read_read_write"}
    out = {}
    for label, elems, nsets in (("headline_tensor", n, 6), ("440MB", 110_000_000, 3)):
        nbytes = elems * 4 // 16384 * 16384
        a = [torch.zeros(elems, device="cuda") for _ in range(nsets)]
        b = torch.zeros(elems, device="cuda")
        res = {"bytes": nbytes}
        for kind, name in names.items():
            i = [0]

            def f(slot=-1):
                i[0] += 1
                rc = probe.bench_probe_stream_timed(kind, a[i[0] % nsets].data_ptr(), b.data_ptr(), nbytes, stream, slot)
                assert rc == 0, rc

            for _ in range(2 * nsets):   # untimed: the zero fill's dirty lines out of the caches
                f()
            settle(torch, f)             # the same settling time as every other measurement here gets
            reps = 24
            torch.cuda.synchronize()
            for r in range(reps):        # back to back; every launch carries its own pair of events
                f(r)
            torch.cuda.synchronize()
            us = [probe.bench_probe_elapsed_us(r) for r in range(reps)]
            assert min(us) > 0, us
            kt = sum(us) / reps * 1e-6
            traffic = nbytes * (3 if kind == 3 else 1)
            res[name] = {"us": round(kt * 1e6, 2), "GBps": round(traffic / kt / 1e9, 1),
                         "frac_of_hbm_peak": round(traffic / kt / 1e9 / HBM_PEAK_GBS, 4)}
        out[label] = res
        del a, b
        torch.cuda.empty_cache()
    h = out["headline_tensor"]
    floor_us = h["read"]["us"] + min(h["write_streaming"]["us"], h["write_plain"]["us"])
    out["headline_floor"] = {"read_plus_write_us": round(floor_us, 2),
                             "frac_of_hbm_peak_at_that_floor": round(8.5 * n / (floor_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def cpu_baseline(np, n, budget_s):
    """The plain-C oracle (port of the reference's CPU bodies, OpenMP) on the same workload."""
    from oracle import cpu
    threads = cpu.max_threads()
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1e-2, n).astype(np.float32)
    pos = rng.integers(0, n, n // 1000)
    x[pos] = np.where(rng.random(pos.size) < 0.5, 0.5, -0.5).astype(np.float32)
    out = np.zeros(n, np.float32)

    def one():
        rc, msg = cpu.terngrad_encode(x, 2, 1, 0)
        cpu.terngrad_decode(msg, n, out)

    one()
    one()
    t0 = time.perf_counter()
    reps, laps = 0, []
    while reps < 3 or (time.perf_counter() - t0 < budget_s and reps < 200):
        t1 = time.perf_counter()
        one()
        laps.append(time.perf_counter() - t1)
        reps += 1
    sec = float(np.median(laps))
    res = {"value": round(4.0 * n / sec / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
           "sample": f"median of {reps} full encode+decode passes of the same {n}-element workload, OpenMP over {threads} threads "
                     f"(os.cpu_count()={os.cpu_count()})", "ms_per_step": round(sec * 1e3, 2)}
    # the same port on one thread
    cpu.set_threads(1)
    t0 = time.perf_counter()
    for _ in range(2):
        one()
    sec1 = (time.perf_counter() - t0) / 2
    cpu.set_threads(threads)
    res["one_thread"] = {"value": round(4.0 * n / sec1 / 1e9, 3), "ms_per_step": round(sec1 * 1e3, 2)}
    return res


def kernel_roofline(kt, alg_bytes):
    """The roofline block of a side measurement: its dominant kernel (longest average launch among those with
    algorithmic bytes) priced against the HBM peak, as the headline's is."""
    cand = {k: v for k, v in kt.items() if v and k in alg_bytes}
    if not cand:
        return None
    dom = max(cand, key=cand.get)
    ach = alg_bytes[dom] / cand[dom] / 1e9
    return {"bound": "hbm", "kernel": dom, "avg_launch_us": round(cand[dom] * 1e6, 2), "algorithmic_bytes": alg_bytes[dom],
            "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4)}


def bucket_sizes(np):
    """The 200 tensor sizes of the fused-bucket configuration (110 M elements, log-uniform in [768, 3e7])."""
    rng = np.random.default_rng(0)
    sizes = np.exp(rng.uniform(np.log(768), np.log(3e7), 200))
    sizes = np.clip(np.floor(sizes * 110e6 / sizes.sum()), 768, 3e7).astype(np.int64)
    sizes[np.argmax(sizes)] += 110_000_000 - sizes.sum()
    return [int(x) for x in sizes]


# MFMA utilisation of the PowerSGD kernels from a counter run of `bench.py --only powersgd`
# (profiles/powersgd_mfma_busy.txt): matrix-pipe busy cycles over the cycles on offer, per kernel.
MEASURED_MFMA_BUSY = {
    "from": "profiles/powersgd_mfma_busy.txt (rocprofv3 --pmc run of `bench.py --only powersgd`), not read in this run",
    "busy_is": "SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 XCDs * 1024 SIMDs)",
    "psgd_encode1_kernel": 0.0265, "psgd_mtp_kernel": 0.0749, "psgd_decode_kernel": 0.0195,
    "SQ_INSTS_MFMA_per_launch": 4718592, "SQ_VALU_MFMA_BUSY_CYCLES_per_launch": 37748736}


def x_tbq(torch, np, capi, L, stream, gen, res):
    # ---- TBQ fused bucket: 110M elements in 200 tensors, thr = 2 sigma ----------------------
    sizes = bucket_sizes(np)
    tot = sum(sizes)
    gs = [torch.randn(int(s), device="cuda", generator=gen) * 5e-3 for s in sizes]
    rs = [torch.zeros(int(s), device="cuda") for s in sizes]
    ps = [torch.zeros((int(s) + 3) // 4, dtype=torch.uint8, device="cuda") for s in sizes]
    os_ = [torch.empty(int(s), device="cuda") for s in sizes]
    thr = capi.f32_array([1e-2] * len(sizes))
    szs = capi.i32_array([int(s) for s in sizes])
    enc = Call(L.hpx_tbq_encode, len(sizes), capi.ptr_array([g.data_ptr() for g in gs]), szs,
               capi.ptr_array([r.data_ptr() for r in rs]), capi.ptr_array([p.data_ptr() for p in ps]), thr, stream)
    dec = Call(L.hpx_tbq_decode, len(sizes), capi.ptr_array([o.data_ptr() for o in os_]), szs,
               capi.ptr_array([p.data_ptr() for p in ps]), thr, capi.i32_array([0] * len(sizes)), stream)

    def tbq_step():
        enc()
        dec()

    sec = timed(torch, tbq_step, 30, 5)
    kt = kernel_times(torch, capi, tbq_step, ["tbq_encode_kernel", "tbq_decode_kernel"], reps=5)
    # both kernels run several launches per call when the bucket exceeds one table: total per call = avg * launches
    res["tbq_bucket_110M_200_tensors"] = {
        "ms_per_step": round(sec * 1e3, 4), "GBps_of_gradient": round(4.0 * tot / sec / 1e9, 1),
        "algorithmic_bytes": 16.5 * tot, "frac_of_hbm_peak": round(16.5 * tot / sec / 1e9 / HBM_PEAK_GBS, 4),
        "kernel_us_per_launch": {k: round(v * 1e6, 1) for k, v in kt.items() if v},
        "roofline": kernel_roofline(kt, {"tbq_encode_kernel": 12.25 * tot, "tbq_decode_kernel": 4.25 * tot})}
    # the root's gather-decode: 7 gathered messages per tensor accumulate into the tensor (hp_cuda.cpp:241-259)
    slots = 7
    # the gathered messages of a tensor are the slots of its piece of the communication buffer, one after the other,
    # as the scheduler hands them over (the library then describes a tensor's messages by a base and a distance)
    bufs7 = [torch.randint(0, 255, (slots * ((int(s) + 3) // 4),), dtype=torch.uint8, device="cuda", generator=gen) & 0xA5 for s in sizes]
    outs7, ins7 = [], []
    for k in range(slots):
        outs7 += os_
        ins7 += [b_[k * ((int(s) + 3) // 4):(k + 1) * ((int(s) + 3) // 4)] for b_, s in zip(bufs7, sizes)]
    root = Call(L.hpx_tbq_decode, slots * len(sizes), capi.ptr_array([o.data_ptr() for o in outs7]),
                capi.i32_array([int(s) for s in sizes] * slots), capi.ptr_array([m_.data_ptr() for m_ in ins7]),
                capi.f32_array([1e-2] * (slots * len(sizes))), capi.i32_array([1] * (slots * len(sizes))), stream)
    sec = timed(torch, root, 10, 2)
    kt = kernel_times(torch, capi, root, ["tbq_decode_multi_kernel"], reps=5)
    alg = (8.0 + 0.25 * slots) * tot
    res["tbq_root_decode_add_7_messages_per_tensor"] = {
        "ms": round(sec * 1e3, 4), "algorithmic_bytes": alg, "frac_of_hbm_peak": round(alg / sec / 1e9 / HBM_PEAK_GBS, 4),
        "bytes_if_applied_one_message_at_a_time": 8.25 * slots * tot,
        "roofline": {"bound": "hbm", "kernel": "tbq_decode_multi_kernel (all launches of the call)", "avg_launch_us": round(sec * 1e6, 2),
                     "algorithmic_bytes": alg, "achieved": round(alg / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(alg / sec / 1e9 / HBM_PEAK_GBS, 4),
                     "kernel_us_per_launch": round(kt["tbq_decode_multi_kernel"] * 1e6, 1) if kt["tbq_decode_multi_kernel"] else None}}


def x_terngrad_root(torch, np, capi, L, stream, gen, res):
    # 7 gathered 2-bit messages of the 25.56 M-element gradient accumulate into it (the root's gather-decode)
    slots = 7
    n = N_TERNGRAD
    x = outlier_gradient(torch, n, gen)
    nbytes = 10 + (n + 3) // 4
    msgs = [torch.zeros(nbytes, dtype=torch.uint8, device="cuda") for _ in range(slots)]
    for k in range(slots):
        rc = L.hpx_terngrad_encode(1, capi.ptr_array([x.data_ptr()]), capi.i32_array([n]), capi.ptr_array([msgs[k].data_ptr()]),
                                   capi.i32_array([nbytes]), capi.u8_array([2]), capi.i32_array([1]), capi.u64_array([k + 1]), stream)
        assert rc == 0, capi.last_error()
    acc = torch.zeros(n, device="cuda")
    troot = Call(L.hpx_terngrad_decode, slots, capi.ptr_array([acc.data_ptr()] * slots), capi.i32_array([n] * slots),
                 capi.ptr_array([m_.data_ptr() for m_ in msgs]), capi.i32_array([nbytes] * slots), capi.i32_array([1] * slots), stream)
    sec = timed(torch, troot, 30, 5)
    kt = kernel_times(torch, capi, troot, ["terngrad_decode_multi_kernel"], reps=10)
    alg = (8.0 + 0.25 * slots) * n
    res["terngrad_root_decode_add_7_messages_25M"] = {
        "ms": round(sec * 1e3, 4), "algorithmic_bytes": alg, "frac_of_hbm_peak": round(alg / sec / 1e9 / HBM_PEAK_GBS, 4),
        "bytes_if_applied_one_message_at_a_time": 8.25 * slots * n,
        "roofline": kernel_roofline(kt, {"terngrad_decode_multi_kernel": alg})}


def x_terngrad_resnet50(torch, np, capi, L, stream, gen, res):
    # ---- TernGrad over ResNet-50's own 161 parameter tensors (the same 25,557,032 elements, one call each way) ----
    r50 = [64 * 3 * 7 * 7, 64, 64]
    inp = 64
    for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            r50 += [planes * inp, planes, planes, planes * planes * 9, planes, planes, planes * 4 * planes, planes * 4, planes * 4]
            if b == 0:
                r50 += [planes * 4 * inp, planes * 4, planes * 4]
            inp = planes * 4
    r50 += [1000 * 2048, 1000]
    assert sum(r50) == N_TERNGRAD
    xs = [torch.randn(m_, device="cuda", generator=gen) * 1e-2 for m_ in r50]
    ms_ = [torch.zeros(10 + (m_ + 3) // 4, dtype=torch.uint8, device="cuda") for m_ in r50]
    ds_ = [torch.empty(m_, device="cuda") for m_ in r50]
    k_ = len(r50)
    enc = Call(L.hpx_terngrad_encode, k_, capi.ptr_array([t_.data_ptr() for t_ in xs]), capi.i32_array(r50),
               capi.ptr_array([t_.data_ptr() for t_ in ms_]), capi.i32_array([t_.numel() for t_ in ms_]), capi.u8_array([2] * k_),
               capi.i32_array([1] * k_), capi.u64_array(list(range(k_))), stream)
    dec = Call(L.hpx_terngrad_decode, k_, capi.ptr_array([t_.data_ptr() for t_ in ds_]), capi.i32_array(r50),
               capi.ptr_array([t_.data_ptr() for t_ in ms_]), capi.i32_array([t_.numel() for t_ in ms_]), capi.i32_array([0] * k_), stream)

    def r50_step():
        enc()
        dec()

    sec = timed(torch, r50_step, 50, 10)
    kt = kernel_times(torch, capi, r50_step, ["terngrad_resident_multi_kernel", "terngrad_decode_kernel"], reps=10)
    L.hpx_set_option(b"terngrad_resident_bucket", 0)          # the same call as a min/max launch and a quantise launch
    sec_tiled = timed(torch, r50_step, 50, 10)
    L.hpx_set_option(b"terngrad_resident_bucket", 1)
    msg_bytes = sum(10 + (m_ + 3) // 4 for m_ in r50)
    phases = terngrad_phases(torch, np, L, r50_step, torch.cuda.get_device_properties(0).multi_processor_count)
    res["terngrad_resnet50_161_tensors"] = {
        "phases_us": phases,
        "ms_per_step": round(sec * 1e3, 4), "tensors": k_, "launches_per_step": 2,
        "algorithmic_bytes": 8.5 * N_TERNGRAD, "frac_of_hbm_peak": round(8.5 * N_TERNGRAD / sec / 1e9 / HBM_PEAK_GBS, 4),
        "ms_per_step_with_the_two_launch_encode": round(sec_tiled * 1e3, 4),
        "roofline": kernel_roofline(kt, {"terngrad_resident_multi_kernel": 4.0 * N_TERNGRAD + msg_bytes,
                                         "terngrad_decode_kernel": 4.0 * N_TERNGRAD + msg_bytes})}
    # ---- the root's gather-decode of that bucket: 7 gathered messages per tensor, the slots of the tensor's piece of
    # the communication buffer one after the other (hp_cuda.cpp:421-439), accumulate into the 161 gradients ----
    slots = 7
    bufs = []
    for m_, x_ in zip(ms_, xs):
        nb = m_.numel()
        b_ = torch.zeros(slots * nb, dtype=torch.uint8, device="cuda")
        one = [b_[j * nb:(j + 1) * nb] for j in range(slots)]
        rc = L.hpx_terngrad_encode(slots, capi.ptr_array([x_.data_ptr()] * slots), capi.i32_array([x_.numel()] * slots),
                                   capi.ptr_array([o_.data_ptr() for o_ in one]), capi.i32_array([nb] * slots), capi.u8_array([2] * slots),
                                   capi.i32_array([1] * slots), capi.u64_array(list(range(1, slots + 1))), stream)
        assert rc == 0, capi.last_error()
        bufs.append(one)
    outs_r, ins_r, sizes_r, insz_r = [], [], [], []
    for j in range(slots):
        outs_r += [t_.data_ptr() for t_ in ds_]
        ins_r += [bufs[i_][j].data_ptr() for i_ in range(k_)]
        sizes_r += r50
        insz_r += [t_.numel() for t_ in ms_]
    for t_ in ds_:
        t_.zero_()
    root = Call(L.hpx_terngrad_decode, slots * k_, capi.ptr_array(outs_r), capi.i32_array(sizes_r), capi.ptr_array(ins_r),
                capi.i32_array(insz_r), capi.i32_array([1] * (slots * k_)), stream)
    sec_root = timed(torch, root, 30, 5)
    kt_root = kernel_times(torch, capi, root, ["terngrad_decode_multi_kernel"], reps=10)
    alg_root = (8.0 + 0.25 * slots) * N_TERNGRAD
    res["terngrad_root_decode_add_7_messages_resnet50_161_tensors"] = {
        "ms": round(sec_root * 1e3, 4), "algorithmic_bytes": alg_root, "frac_of_hbm_peak": round(alg_root / sec_root / 1e9 / HBM_PEAK_GBS, 4),
        "launches_per_call": 1,
        "roofline": kernel_roofline(kt_root, {"terngrad_decode_multi_kernel": alg_root})}


def x_terngrad_sizes(torch, np, capi, L, stream, gen, res):
    # ---- TernGrad 2-bit encode + decode over tensor sizes: which encode a size takes (two launches; one launch
    # with the tensor on chip; one launch with the tensor's head on chip and the rest streamed twice), kernel
    # times, step time and fraction of the HBM peak on 8.5 B/elt.  102,760,448 is VGG-16's first fully connected layer.
    kernels = ["terngrad_resident_kernel", "terngrad_resident_streamed_kernel", "terngrad_minmax_kernel",
               "terngrad_quant_kernel", "terngrad_decode_kernel"]
    table = []
    for n in (1_000_000, 2_000_000, 4_000_000, 6_000_000, 8_000_000, 12_000_000, 16_000_000, 20_000_000, N_TERNGRAD,
              30_000_000, 33_500_000, 34_000_000, 40_000_000, 48_000_000, 64_000_000, 80_000_000, 102_760_448,
              128_000_000, 134_000_000, 136_000_000, 160_000_000):
        nsets = 4 if n < 70_000_000 else 2
        sets = []
        for _ in range(nsets):
            x = torch.randn(n, device="cuda", generator=gen) * 1e-2
            msg = torch.zeros(10 + (n + 3) // 4, dtype=torch.uint8, device="cuda")
            dec = torch.empty(n, device="cuda")
            sets.append((x, msg, dec,
                         Call(L.hpx_terngrad_encode, 1, capi.ptr_array([x.data_ptr()]), capi.i32_array([n]), capi.ptr_array([msg.data_ptr()]),
                              capi.i32_array([msg.numel()]), capi.u8_array([2]), capi.i32_array([1]), capi.u64_array([0]), stream),
                         Call(L.hpx_terngrad_decode, 1, capi.ptr_array([dec.data_ptr()]), capi.i32_array([n]), capi.ptr_array([msg.data_ptr()]),
                              capi.i32_array([msg.numel()]), capi.i32_array([0]), stream)))
        state = {"i": 0}

        def step():
            s_ = sets[state["i"] % nsets]
            state["i"] += 1
            s_[3]()
            s_[4]()

        sec = timed(torch, step, 40, 5)
        kt = kernel_times(torch, capi, step, kernels, reps=8)
        path = ("one launch, on chip" if kt["terngrad_resident_kernel"] else
                "one launch, head on chip, rest streamed twice" if kt["terngrad_resident_streamed_kernel"] else "two launches")
        enc_us = sum(v for k, v in kt.items() if v and k != "terngrad_decode_kernel") * 1e6
        table.append({"elements": n, "encode": path, "encode_kernels_us": round(enc_us, 1),
                      "decode_kernel_us": round((kt["terngrad_decode_kernel"] or 0) * 1e6, 1), "step_us": round(sec * 1e6, 1),
                      "frac_of_hbm_peak": round(8.5 * n / sec / 1e9 / HBM_PEAK_GBS, 4)})
        del sets
        torch.cuda.empty_cache()
    res["terngrad_size_sweep"] = table
    big = [r for r in table if r["elements"] == 102_760_448][0]
    res["terngrad_102M"] = dict(big, algorithmic_bytes=8.5 * 102_760_448, workload="VGG-16 fc6, 2-bit, stochastic rounding, encode + decode(write)")


GD_KERNELS = ["gd_sample_kernel", "gd_select_kernel", "gd_threshold_kernel", "gd_presample_kernel", "gd_provisional_kernel", "gd_stream_kernel",
              "gd_resample_kernel", "gd_exact_kernel", "gd_recount_kernel", "gd_scan_kernel",
              "gd_expand_kernel", "gd_sort_count_kernel", "gd_sort_pass_kernel", "gd_gather_kernel"]


def x_dgc(torch, np, capi, L, stream, gen, res):
    # ---- DGC / GradDrop top-0.1 %: 138,357,544 elements --------------------------------------
    n = N_DGC
    # A generator of its own: which seeds below have to sort and cut depends on the gradient drawn here (each does
    # with probability about one half), and the section's mean should not move with what other sections drew before it.
    gen = torch.Generator(device="cuda").manual_seed(138_357_544)
    u = torch.rand(n, device="cuda", generator=gen) - 0.5
    # Laplace(0, 1e-3) by inversion; |u| is kept below 1/2 (a draw of exactly 0 would otherwise become an
    # infinite gradient, which the configuration's float64 Laplace sampler never produces)
    g = (-1e-3 * torch.sign(u) * torch.log1p(-2 * u.abs().clamp_(max=0.5 - 2.0 ** -25))).float()
    del u
    r0 = torch.randn(n, device="cuda", generator=gen) * 1e-4
    r = r0.clone()
    out = torch.zeros(4 + 8 * int(np.ceil(n * (1 - 0.999))), dtype=torch.uint8, device="cuda")
    scrub = torch.empty(160_000_000, device="cuda")  # 640 MB, larger than L2 + Infinity Cache
    # Whether the sampled threshold lets through more than the `expected` entries (and the call has to sort and
    # cut) depends on the sample, i.e. on the seed: time several seeds and report each.
    per_seed = []
    kt = None
    for seed in (0, 1 << 24, 2 << 24, 3 << 24, 4 << 24, 5 << 24, 6 << 24, 7 << 24):  # seeds closer than the sample size share most of their sample
        gd = Call(L.hpx_gd_encode, 1, capi.ptr_array([g.data_ptr()]), capi.i32_array([n]), capi.ptr_array([r.data_ptr()]),
                  capi.ptr_array([out.data_ptr()]), capi.f64_array([0.01]), capi.f64_array([0.999]), capi.u64_array([seed]), stream)
        times = []
        for it in range(7):
            r.copy_(r0)                      # every repetition sees the configuration's residual
            scrub.sum()                      # push the copy's dirty lines out of the caches: inputs are in HBM when the clock starts
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            gd()                             # returns once the counts are known; the tail of the work is still queued
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        k = (int(out[:4].cpu().numpy().view(np.int32)[0]) - 4) // 8
        r.copy_(r0)
        scrub.sum()
        kts = kernel_times(torch, capi, gd, GD_KERNELS, reps=1)
        cut = kts["gd_gather_kernel"] is not None
        per_seed.append({"seed": seed, "encode_ms": round(float(np.median(times[2:])) * 1e3, 4), "selected": k, "cut": cut})
        if kt is None or (cut and kt["gd_gather_kernel"] is None):
            kt = kts
    sec = float(np.mean([p["encode_ms"] for p in per_seed])) * 1e-3
    dout = torch.zeros(n, device="cuda")
    gdr = Call(L.hpx_gd_decode, 1, capi.ptr_array([out.data_ptr()]), capi.i32_array([out.numel()]),
               capi.ptr_array([dout.data_ptr()]), capi.i32_array([n]), capi.i32_array([1]), stream)
    sec_dec = timed(torch, gdr, 20, 3)
    res["dgc_top0.1pct_138M"] = {
        "encode_ms": round(sec * 1e3, 4), "encode_ms_is": "mean over the seeds below", "per_seed": per_seed,
        "encode_GBps_of_gradient": round(4.0 * n / sec / 1e9, 1),
        "algorithmic_bytes": 12.0 * n + 8 * k + 4, "frac_of_hbm_peak": round((12.0 * n + 8 * k + 4) / sec / 1e9 / HBM_PEAK_GBS, 4),
        "stream_kernel_frac_of_hbm_peak": round(12.0 * n / kt["gd_stream_kernel"] / 1e9 / HBM_PEAK_GBS, 4) if kt["gd_stream_kernel"] else None,
        "decode_add_ms": round(sec_dec * 1e3, 4), "kernel_us_per_launch": {k_: round(v * 1e6, 1) for k_, v in kt.items() if v},
        "roofline": kernel_roofline(kt, {"gd_stream_kernel": 12.0 * n})}
    # the same sparsifier without residual (dgc_body.h): reads the gradient once, 4 B/elt
    del r, r0, dout
    g0 = g.clone()
    dgc = Call(L.hpx_dgc_encode, 1, capi.ptr_array([g.data_ptr()]), capi.i32_array([n]), capi.ptr_array([out.data_ptr()]),
               capi.f64_array([0.01]), capi.f64_array([0.001]), capi.u64_array([3 << 24]), stream)
    times = []
    for it in range(7):
        g.copy_(g0)
        scrub.sum()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dgc()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    sec_nr = float(np.median(times[2:]))
    g.copy_(g0)
    scrub.sum()
    kt = kernel_times(torch, capi, dgc, GD_KERNELS, reps=1)
    res["dgc_without_residual_138M"] = {
        "encode_ms": round(sec_nr * 1e3, 4), "algorithmic_bytes": 4.0 * n,
        "frac_of_hbm_peak": round(4.0 * n / sec_nr / 1e9 / HBM_PEAK_GBS, 4),
        "selected": (int(out[:4].cpu().numpy().view(np.int32)[0]) - 4) // 8,
        "roofline": kernel_roofline(kt, {"gd_stream_kernel": 4.0 * n})}


def x_dgc_bucket(torch, np, capi, L, stream, gen, res):
    # ---- GradDrop over the 200-tensor bucket (110 M elements): one call against one call per tensor -------------
    gen = torch.Generator(device="cuda").manual_seed(110_000_000)   # as above: a draw of its own
    sizes = bucket_sizes(np)
    tot = sum(sizes)
    gs = [torch.randn(s, device="cuda", generator=gen) * 5e-3 for s in sizes]
    r0 = [torch.randn(s, device="cuda", generator=gen) * 1e-4 for s in sizes]
    rs = [t.clone() for t in r0]
    outs = [torch.zeros(4 + 8 * int(np.ceil(s * 0.001)) + 64, dtype=torch.uint8, device="cuda") for s in sizes]

    def call(idx):
        return Call(L.hpx_gd_encode, len(idx), capi.ptr_array([gs[i].data_ptr() for i in idx]), capi.i32_array([sizes[i] for i in idx]),
                    capi.ptr_array([rs[i].data_ptr() for i in idx]), capi.ptr_array([outs[i].data_ptr() for i in idx]),
                    capi.f64_array([0.01] * len(idx)), capi.f64_array([0.999] * len(idx)), capi.u64_array([7 + i for i in idx]), stream)

    whole = call(list(range(len(sizes))))
    singles = [call([i]) for i in range(len(sizes))]

    def one_by_one():
        for c_ in singles:
            c_()

    def run(f, reps):
        ts = []
        for it in range(reps):
            for a, b in zip(rs, r0):
                a.copy_(b)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            f()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts[1:]))

    sec = run(whole, 6)
    sec_loop = run(one_by_one, 3)
    for a, b in zip(rs, r0):
        a.copy_(b)
    torch.cuda.synchronize()
    L.hpx_profile_reset()
    L.hpx_profile_enable(1)
    whole()
    torch.cuda.synchronize()
    L.hpx_profile_enable(0)
    per_call = {k_: capi.profile_query(k_) for k_ in GD_KERNELS}      # (total ms, launches) of the one call
    L.hpx_profile_reset()
    kt = {k_: (ms_ / n_) * 1e-3 if n_ else None for k_, (ms_, n_) in per_call.items()}
    stream_s = per_call["gd_stream_kernel"][0] * 1e-3
    cut = sum(1 for o, s in zip(outs, sizes) if (int(o[:4].cpu().numpy().view(np.int32)[0]) - 4) // 8 == int(np.ceil(s * 0.001)))
    res["dgc_bucket_110M_200_tensors"] = {
        "encode_ms_one_call": round(sec * 1e3, 4), "encode_ms_one_call_per_tensor": round(sec_loop * 1e3, 4),
        "tensors": len(sizes), "tensors_filled_to_expected": cut,
        "algorithmic_bytes": 12.0 * tot, "frac_of_hbm_peak": round(12.0 * tot / sec / 1e9 / HBM_PEAK_GBS, 4),
        "kernel_us_per_launch": {k_: round(v * 1e6, 1) for k_, v in kt.items() if v},
        "launches_per_call": {k_: n_ for k_, (ms_, n_) in per_call.items() if n_},
        # the stream pass runs once per table of 256 tensors: all its launches of a call together against all its bytes
        "roofline": {"bound": "hbm", "kernel": "gd_stream_kernel (all launches of the call: one per table of 256 tensors)", "avg_launch_us": round(stream_s * 1e6, 2),
                     "algorithmic_bytes": 12.0 * tot, "achieved": round(12.0 * tot / stream_s / 1e9, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(12.0 * tot / stream_s / 1e9 / HBM_PEAK_GBS, 4)}}


def x_powersgd(torch, np, capi, L, stream, gen, res):
    # ---- PowerSGD rank 4 over the 36-matrix layer set ------------------------------------------
    shapes = [(4096, 4096)] * 12 + [(1024, 4096)] * 12 + [(4096, 1024)] * 12
    rk = 4
    G = [torch.randn(a * b, device="cuda", generator=gen) * 1e-2 for a, b in shapes]
    R = [torch.zeros(a * b, device="cuda") for a, b in shapes]
    Q = [torch.randn(b, rk, device="cuda", generator=gen) for a, b in shapes]
    M = [torch.zeros(a, b, device="cuda") for a, b in shapes]
    P = [torch.zeros(a, rk, device="cuda") for a, b in shapes]
    ns, ms, rs_ = capi.i32_array([a for a, b in shapes]), capi.i32_array([b for a, b in shapes]), capi.i32_array([rk] * 36)
    numels = capi.i64_array([a * b for a, b in shapes])
    pa = lambda ts: capi.ptr_array([t.data_ptr() for t in ts])
    e1 = Call(L.hpx_powersgd_encode1, 36, pa(G), numels, pa(R), pa(Q), pa(M), pa(P), ns, ms, rs_, stream)
    e2 = Call(L.hpx_powersgd_encode2, 36, pa(P), pa(M), pa(Q), ns, ms, rs_, stream)
    dc = Call(L.hpx_powersgd_decode, 36, pa(P), pa(Q), pa(M), pa(R), pa(G), numels, ns, ms, rs_, stream)

    def psgd_step():
        e1()
        e2()
        dc()

    sec = timed(torch, psgd_step, 10, 2)
    names = ["psgd_encode1_kernel", "psgd_orth_kernel", "psgd_mtp_kernel", "psgd_qreduce_kernel", "psgd_decode_kernel"]
    kt = kernel_times(torch, capi, psgd_step, names, reps=3)
    elems = sum(a * b for a, b in shapes)
    flops = 24.0 * elems
    # per kernel: 2 * n*m*r flops each for P = MQ, Q = M^T P and M = P Q^T
    kflops = {"psgd_encode1_kernel": 8.0 * elems, "psgd_mtp_kernel": 8.0 * elems, "psgd_decode_kernel": 8.0 * elems}
    res["powersgd_rank4_36_matrices"] = {
        "ms_per_iteration": round(sec * 1e3, 4), "GBps_of_gradient": round(4.0 * elems / sec / 1e9, 1),
        "algorithmic_bytes": 16.0 * elems, "frac_of_hbm_peak": round(16.0 * elems / sec / 1e9 / HBM_PEAK_GBS, 4),
        "bytes_moved_by_three_phase_api": 32.0 * elems,
        "frac_of_hbm_peak_three_phase_bytes": round(32.0 * elems / sec / 1e9 / HBM_PEAK_GBS, 4),
        "mfma_frac_of_fp32_peak": round(flops / sec / 1e12 / FP32_MFMA_PEAK_TF, 5),
        "mfma_frac_of_fp32_peak_is": "flops / wall time / 157.3 TFLOP/s",
        "mfma_frac_of_fp32_peak_per_kernel": {k_: round(kflops[k_] / kt[k_] / 1e12 / FP32_MFMA_PEAK_TF, 5) for k_ in kflops if kt.get(k_)},
        "mfma_busy_from_counters": MEASURED_MFMA_BUSY,
        "kernel_us_per_launch": {k_: round(v * 1e6, 1) for k_, v in kt.items() if v},
        "roofline": kernel_roofline(kt, {"psgd_encode1_kernel": 12.0 * elems, "psgd_mtp_kernel": 4.0 * elems,
                                         "psgd_decode_kernel": 16.0 * elems})}


def x_scheduler(torch, np, capi, L, stream, gen, res):
    # ---- the scheduler around the path: one COMP task, submit -> name in the finished queue ------------
    # (TernGrad 2-bit, 25.56 M elements; includes the 6.4 MB device-to-host copy of the message into a
    # pinned C buffer and both thread hand-overs; the reference's worker polls its queue every 500 us)
    ext_dir = os.path.join(ROOT, "torch-hipress-extension_amd", "ext")   # the compiled `hp_cuda` extension module
    if ext_dir not in sys.path:
        sys.path.insert(0, ext_dir)
    hp = importlib.import_module("hp_cuda")
    if hp.init("terngrad", {"enable_random": 1, "bitwidth": 2, "seed": 0}, torch.cuda.current_device(), 0, 2):
        n = N_TERNGRAD
        x = outlier_gradient(torch, n, gen)
        nbytes = 10 + (n + 3) // 4
        B = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        Cc = torch.zeros(nbytes, dtype=torch.uint8, pin_memory=True)
        torch.cuda.synchronize()
        lat = []
        for it in range(30):
            t0 = time.perf_counter()
            hp.submit_task("g", x, B, Cc, 0, 10)
            while not hp.getResults(10):
                hp.wait(10, 100)
            lat.append(time.perf_counter() - t0)
        hp.end()
        lat = np.array(lat[5:])
        res["scheduler_terngrad_comp_task_25M"] = {
            "submit_to_finished_ms_median": round(float(np.median(lat)) * 1e3, 4),
            "submit_to_finished_ms_min": round(float(lat.min()) * 1e3, 4), "message_bytes_to_host": nbytes,
            "errors": hp.error_count()}

    # 200 COMP tasks at once (the TBQ bucket, 110 M elements): the worker batches what is queued into
    # multi-tensor encodes; 27.5 MB of messages go to pinned C buffers on the data stream
    if hp.init("tbq", {"threshold": 1e-2}, torch.cuda.current_device(), 0, 2):
        sizes = bucket_sizes(np)
        gs = [torch.randn(int(n_), device="cuda", generator=gen) * 5e-3 for n_ in sizes]
        rs = [torch.zeros(int(n_), device="cuda") for n_ in sizes]
        Bs = [torch.zeros((int(n_) + 3) // 4, dtype=torch.uint8, device="cuda") for n_ in sizes]
        Cs = [torch.zeros((int(n_) + 3) // 4, dtype=torch.uint8, pin_memory=True) for n_ in sizes]
        names = [f"t{i}" for i in range(200)]
        torch.cuda.synchronize()
        lat = []
        for it in range(8):
            t0 = time.perf_counter()
            for nm, g_, r_, B_, C_ in zip(names, gs, rs, Bs, Cs):
                hp.submit_task(nm, g_, r_, B_, C_, 0, 10)
            got = 0
            while got < 200:
                hp.wait(10, 100)
                got += len(hp.getResults(10))
            lat.append(time.perf_counter() - t0)
        hp.end()
        lat = np.array(lat[2:])
        msg_bytes = int(sum((int(n_) + 3) // 4 for n_ in sizes))
        res["scheduler_tbq_bucket_200_comp_tasks"] = {
            "submit_all_to_all_finished_ms_median": round(float(np.median(lat)) * 1e3, 4),
            "elements": int(sum(sizes)), "message_bytes_to_host": msg_bytes,
            "GBps_of_gradient": round(4.0 * float(sum(sizes)) / float(np.median(lat)) / 1e9, 1), "errors": hp.error_count()}


EXTRAS = {"tbq": x_tbq, "terngrad_root": x_terngrad_root, "terngrad_resnet50": x_terngrad_resnet50,
          "terngrad_sizes": x_terngrad_sizes, "dgc": x_dgc,
          "dgc_bucket": x_dgc_bucket, "powersgd": x_powersgd, "scheduler": x_scheduler}


def extra(torch, np, capi, L, stream, gen, only=None):
    """Other codecs of the path at their configuration sizes (GPU only, short runs).  Every entry carries the same
    kind of roofline block as the headline: its dominant kernel, that kernel's average launch time (HIP events on
    the launch stream), its algorithmic bytes and the fraction of the HBM peak."""
    res = {}
    for name, fn in EXTRAS.items():
        if only and name not in only:
            continue
        fn(torch, np, capi, L, stream, gen, res)
        torch.cuda.empty_cache()
    return res


if __name__ == "__main__":
    main()
