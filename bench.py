#!/usr/bin/env python3
"""Benchmark of the HipNx hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-suite] [--no-cpu] [--calibrate]

Headline workload (the configuration the metric is quoted on): `Nx.dot` of bf16 {4096,4096} x
{4096,4096}, f32 accumulation on MFMA, bf16 output -- one step = one `dot` callback through the
C ABI, inputs resident in HBM.  The LAST stdout line is the headline as JSON (under 4 KB); a table of the
suite precedes it and the full record is written to gpurun_out/bench_suite.json.  `value` is TFLOP/s over
K timed steps (wall clock between two device synchronisations).  `roofline` is measured live with HIP events on
the stream the kernels are launched on.  `suite` carries the other configurations (GB/s or
TFLOP/s and their roofline fractions), `cpu_baseline` the CPU restatement of the reference on a
bounded sample of the same workload.  `--calibrate` first launches a streaming kernel of known
traffic (1 GiB read, 1 GiB written) so that a `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` run of this
file carries its own scale for those counters.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK = {"bf16": 2500.0, "f16": 2500.0, "s8": 5000.0, "f32": 157.3, "f64": 78.6}  # dense MFMA TFLOP/s (TOP/s)

# HBM bytes per launch of the headline dot kernel come from two counter runs of this file
# (`rocprofv3 --pmc FETCH_SIZE`, then `--pmc WRITE_SIZE`, with --calibrate); the summary of those runs
# carries the figure in a line `TRAFFIC_BYTES_PER_LAUNCH = <n>`, which is what is reported here.
TRAFFIC_PROFILE = os.path.join("profiles", "dot_bf16_4096_hbm_traffic.md")
TRAFFIC_PROFILE_S8 = os.path.join("profiles", "dot_s8_4096_hbm_traffic.md")
CEILINGS_BIN = os.path.join(ROOT, "nx_amd", "lib", "hipnx_ceilings")
ABI_DRIVER_BIN = os.path.join(ROOT, "nx_amd", "lib", "hipnx_abi_driver")
# suite entries whose roofline fraction is repeated in the headline line (the rest stay in the detail file)
HEADLINE_ALSO = ("dot_s8_4096_s32", "dot_bf16_4096_kinner", "dot_f32_2048", "dot_s8_w8_64x11008x4096_rotated",
                 "dot_qk_bf16_32x512x64_rotated", "softmax_chain_32x512x512_rotated", "config1_chain_f32_1024",
                 "config1_chain_f32_16384", "add_f32_16384", "sum_rows_f32_16384", "argmax_f32_8192x32000",
                 "take_bf16_8192_of_32000x4096_rotated", "config4_chain_rotated", "softmax_1M_f32", "softmax_1M_f32_planned_compiled",
                 "softmax_1M_f64")


def host_transfer_figures(H, B, Nx, template):
    """from_binary / to_binary through the host link (pageable host memory, as a caller has it): never part of
    `value`, reported so that the PCIe-inclusive cost of a round trip is on record."""
    import ctypes
    from nx_amd import _lib as L
    out = {"note": "pageable host memory; uploads return once the source is consumed, downloads wait for the device"}
    for label, nbytes in (("64KiB", 64 << 10), ("256MiB", 256 << 20)):
        host = np.random.default_rng(3).integers(0, 256, size=nbytes, dtype=np.uint8)
        dev = H.from_numpy(template("u8", host.shape), host)
        back = np.zeros(nbytes, dtype=np.uint8)
        B.sync()
        up, down, binary = [], [], []
        for _ in range(5):
            t0 = time.perf_counter()
            dev = H.from_numpy(template("u8", host.shape), host)
            B.sync()
            up.append(time.perf_counter() - t0)
            t0 = time.perf_counter()
            L.check(L.lib.hipnx_d2h(dev.data.ref.ctx, H._handle(dev), 0, back.ctypes.data_as(ctypes.c_void_p), nbytes))
            down.append(time.perf_counter() - t0)
            t0 = time.perf_counter()
            raw = Nx.to_binary(dev)
            binary.append(time.perf_counter() - t0)
            del raw
        assert np.array_equal(back, host)
        out[label] = {"from_binary_us": round(min(up) * 1e6, 1), "from_binary_GBps": round(nbytes / min(up) / 1e9, 2),
                      "d2h_into_touched_memory_us": round(min(down) * 1e6, 1), "d2h_GBps": round(nbytes / min(down) / 1e9, 2),
                      "to_binary_us": round(min(binary) * 1e6, 1), "to_binary_GBps": round(nbytes / min(binary) / 1e9, 2)}
    return out


def c_abi_figures():
    """Configuration 1's callbacks and `take` issued from plain C through libhipnx.so (what a NIF would
    see): host microseconds per call and per chain, without Python or ctypes in the path."""
    import subprocess
    if not os.path.exists(ABI_DRIVER_BIN):
        return None
    try:
        res = subprocess.run([ABI_DRIVER_BIN, "2000"], capture_output=True, text=True, timeout=180)
        out = json.loads(res.stdout.strip().splitlines()[-1])
        out["command"] = "nx_amd/lib/hipnx_abi_driver 2000 (tests/c_abi/abi_driver.c)"
        return out
    except Exception as exc:
        return {"error": str(exc)[:200]}


def headline_traffic(profile):
    """(bytes per launch, source) from the committed counter summary; (None, reason) without it."""
    try:
        with open(os.path.join(ROOT, profile)) as f:
            for line in f:
                if line.startswith("TRAFFIC_BYTES_PER_LAUNCH"):
                    return int(line.split("=")[1].split()[0]), profile
    except OSError:
        pass
    return None, "no counter summary found"


def measured_ceilings(ms=250):
    """What this part sustains: MFMA-only loops (the kernel's own MFMA forms, operands drawn like the
    benchmark's) and streaming kernels, each run by the stand-alone program for `ms` milliseconds."""
    import subprocess
    out = {}
    if not os.path.exists(CEILINGS_BIN):
        return out
    runs = [("mfma_bf16", ["mfma", "bf16", "normal", str(ms)]), ("mfma_f16", ["mfma", "f16", "normal", str(ms)]),
            ("mfma_s8", ["mfma", "s8", "normal", str(ms)]), ("mfma_f32", ["mfma", "f32", "normal", str(ms)]),
            ("mfma_f64", ["mfma", "f64", "normal", str(ms)]),
            # 1 GiB per buffer: the size of the suite's 16384^2 f32 tensors (a 2 GiB stream keeps less of itself in
            # the 256 MB last-level cache and reads a few per cent lower)
            ("stream_read", ["stream", "read", "1024", "100"]), ("stream_write", ["stream", "write", "1024", "100"]),
            ("stream_copy", ["stream", "copy", "1024", "100"])]
    for name, argv in runs:
        try:
            res = subprocess.run([CEILINGS_BIN] + argv, capture_output=True, text=True, timeout=120)
            line = json.loads(res.stdout.strip().splitlines()[-1])
            line["command"] = "nx_amd/lib/hipnx_ceilings " + " ".join(argv)
            out[name] = line
        except Exception as exc:  # an extra: the published peaks stay the denominators of `frac`
            out[name] = {"error": str(exc)[:200]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=30)
    # The clock this part runs a kernel at settles over tens of milliseconds of the same load (a 4096^3
    # dot starts near 112 us, drops to 130-140 us after 2 ms and recovers to ~100 us within 50 ms), so a
    # short run measures the power controller's transient.  Before the warm-up steps of the headline the
    # same call is therefore repeated untimed for this long; `cold_start` in the output is the figure
    # without it.
    ap.add_argument("--settle-ms", type=float, default=400.0)
    ap.add_argument("--no-ceilings", action="store_true")
    ap.add_argument("--no-suite", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate", action="store_true")
    # parts of the suite to run (comma-separated: dots, config1, bf16, config3, config4, config5, misc, random, chains,
    # softmax1m); default all
    ap.add_argument("--only", default=None)
    # which 4096^3 contraction is timed as the headline: bf16 (the metric's configuration, the default) or the
    # int8 one (s8 x s8 -> s32), so that the int8 kernel can be profiled by the same commands
    ap.add_argument("--headline", choices=["bf16", "s8"], default="bf16")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no sharding, no collectives); use --gpus 1")

    from nx_amd import nx as Nx
    from nx_amd import workloads as W
    from nx_amd import backend as B
    from nx_amd.backend import HipNxBackend as H
    from nx_amd.tensor import template

    # what a user does first: `Nx.default_backend(HipNx.Backend)`, so that scalar operands become
    # device constants (a fill kernel) instead of host tensors that are transferred per call
    Nx.default_backend(H)

    def put(arr, ty):
        return H.from_numpy(template(ty, arr.shape), arr)

    def timed(fn, steps, warmup):
        """(wall ms per step, device ms per step): K calls between two synchronisations, with a
        HIP-event pair recorded on the context's stream around the same region."""
        for _ in range(warmup):
            keep = fn()
        B.sync()
        t0 = time.perf_counter()
        B.timer_start()
        for _ in range(steps):
            keep = fn()  # noqa: F841 - results are dropped (returned to the pool) as a caller would
        dev_ms = B.timer_stop()
        B.sync()
        wall_ms = (time.perf_counter() - t0) * 1e3
        return wall_ms / steps, dev_ms / steps

    def laps(fn, steps, warmup):
        """Device ms per step from lap marks on the launch stream: (mean, median, min).  A mark costs a few
        microseconds on the stream, so one is recorded per chunk of steps (at most 20 chunks) and the
        median and the minimum are those of the chunks' per-step means."""
        chunk = max(1, steps // 20)
        chunks = max(1, steps // chunk)
        for _ in range(warmup):
            keep = fn()
        B.timer_mark(0)
        for c in range(chunks):
            for _ in range(chunk):
                keep = fn()  # noqa: F841
            B.timer_mark(c + 1)
        per = sorted(B.timer_between(c, c + 1) / chunk for c in range(chunks))
        return B.timer_between(0, chunks) / (chunks * chunk), per[len(per) // 2], per[0]

    def settle(fn, ms):
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < ms:
            for _ in range(50):
                keep = fn()  # noqa: F841
            B.sync()

    ceilings = {} if args.no_ceilings else measured_ceilings()

    if args.calibrate:
        big = put(np.ones((16384, 16384), dtype=np.float32), "f32")
        for _ in range(5):
            keep = Nx.negate(big)  # noqa: F841 - 2^30 bytes read, 2^30 bytes written per launch
        B.sync()
        del big, keep

    # ---- headline: config 2, dense bf16 GEMM ------------------------------------------------
    n = 4096
    a_np, b_np = W.dense_gemm_bf16(n=n)
    a, b = put(a_np, "bf16"), put(b_np, "bf16")
    flop = 2.0 * n * n * n
    if args.headline == "s8":
        qa, qb = W.dense_gemm_s8()
        qa, qb = put(qa, "s8"), put(qb, "s8")
        head = lambda: Nx.dot(qa, qb, out_type="s32")  # noqa: E731
    else:
        head = lambda: Nx.dot(a, b)  # noqa: E731
    _, cold_ms = timed(head, 20, 5)  # an idle part's first 25 launches
    settle(head, args.settle_ms)
    wall_ms, dev_ms = timed(head, args.steps, args.warmup)
    value = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (dev_ms * 1e-3) / 1e12
    lap_mean, lap_median, lap_min = laps(head, args.steps, 0)
    traffic, traffic_source = headline_traffic(TRAFFIC_PROFILE if args.headline == "bf16" else TRAFFIC_PROFILE_S8)

    hunit = "TFLOP/s" if args.headline == "bf16" else "TOP/s"
    hwork = ("dense GEMM: Nx.dot bf16 {4096,4096} x {4096,4096}, f32 accumulate, bf16 output (BASELINE configs[1])"
             if args.headline == "bf16" else
             "dense GEMM: Nx.dot s8 {4096,4096} x {4096,4096}, s32 accumulate and output (the int8 leg of BASELINE configs[1])")
    result = {
        "metric": "Nx.dot TFLOP/s (bf16, s8->s32) + elementwise/reduce GB/s, % of MI355X peak",
        "value": round(value, 3), "unit": hunit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.headline, "data": "synthetic",
        "config": {"workload": hwork, "seed": 2},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK[args.headline], "unit": hunit,
                     "frac": round(achieved / PEAK[args.headline], 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "dot callback (gemm kernel + operand re-layout, if any), HIP events on the launch stream",
                     "per_step_us": {"mean": round(dev_ms * 1e3, 2), "median": round(lap_median * 1e3, 2),
                                     "min": round(lap_min * 1e3, 2),
                                     "note": "median / min over 20 chunks of a second pass of K steps (one lap mark per chunk)"}},
        "settle_ms": args.settle_ms,
        "cold_start": {"tflops": round(flop / (cold_ms * 1e-3) / 1e12, 1), "steps": 20, "warmup": 5,
                       "note": "the same call on the idle part, before the settling phase"},
    }
    hceil = "mfma_" + args.headline
    if "sustained" in ceilings.get(hceil, {}):
        top = ceilings[hceil]["sustained"]
        result["roofline"]["measured_ceiling"] = {"value": top, "unit": hunit, "frac_of_ceiling": round(achieved / top, 4),
                                                  "source": ceilings[hceil]["command"]}
    if ceilings:
        result["ceilings"] = ceilings

    # ---- the other configurations -----------------------------------------------------------
    # Entries are timed "cache-hot" (the same operands every step).  Where the operands are smaller
    # than the 256 MB Infinity Cache and the kernel is meant to stream from HBM, a second entry
    # `<name>_rotated` walks a ring of operand copies larger than the cache.
    if not args.no_suite:
        suite = {}
        steps, warm = max(args.steps // 2, 10), 5
        from nx_amd import defn

        def section(name):
            """`--only a,b` runs the named parts of the suite alone (for profiles of one configuration)."""
            return args.only is None or name in args.only.split(",")

        def rotating(make, nbytes):
            """A ring of operand sets exceeding 320 MB in total; returns next()."""
            copies = max(2, int(320e6 // nbytes) + 1)
            ring = [make() for _ in range(copies)]
            state = [0]

            def nxt():
                state[0] = (state[0] + 1) % copies
                return ring[state[0]]
            return nxt

        class Ms(float):
            """Mean device ms per step, carrying the median and the minimum of the per-step times."""

        def tstat(fn, steps, warmup, settle_ms=0.0):
            if settle_ms:
                settle(fn, settle_ms)
            mean, median, least = laps(fn, steps, warmup)
            ms = Ms(mean)
            ms.median, ms.least = median, least
            return None, ms

        def entry(name, work, unit, ms, peak, bound, ceil=None, vs=None):
            """`work` = the entry's own algorithmic bytes or flop per step; `ceil` names the measured ceiling
            it is also compared with; `vs` = (label, ms of the formulation it replaces)."""
            scale = 1e12 if unit in ("TFLOP/s", "TOP/s") else 1e9
            rate = work / (ms * 1e-3) / scale
            e = {"ms": round(ms, 5), "ms_median": round(ms.median, 5), "ms_min": round(ms.least, 5),
                 "achieved": round(rate, 2), "unit": unit, "bound": bound, "peak": peak, "frac": round(rate / peak, 4)}
            if ceil is None and bound == "hbm":
                ceil = "stream_copy"
            top = ceilings.get(ceil, {}).get("sustained") if ceil else None
            if top:
                e["measured_ceiling"] = {"value": top, "source": ceilings[ceil]["command"], "frac_of_ceiling": round(rate / top, 4)}
            if vs:
                e["vs_" + vs[0]] = round(vs[1] / ms, 2)
            suite[name] = e

        if section("dots"):
            # K-inner operands: the gemm kernel alone (no re-layout pass)
            bt = Nx.transpose(b)
            msettle = min(args.settle_ms, 150.0)
            _, ms = tstat(lambda: Nx.dot(a, [1], bt, [1]), steps, warm, msettle)
            entry("dot_bf16_4096_kinner", flop, "TFLOP/s", ms, PEAK["bf16"], "mfma", "mfma_bf16")
            nxt = rotating(lambda: (put(a_np, "bf16"), put(b_np, "bf16")), 2 * n * n * 2)

            def dot_rot():
                x, y = nxt()
                return Nx.dot(x, y)
            _, ms = tstat(dot_rot, steps, warm, msettle)
            entry("dot_bf16_4096_rotated", flop, "TFLOP/s", ms, PEAK["bf16"], "mfma", "mfma_bf16")
            del nxt
            fa_np, fb_np = W.dense_gemm_f32()
            fa, fb = put(fa_np, "f32"), put(fb_np, "f32")
            _, ms = tstat(lambda: Nx.dot(fa, fb), steps, warm, msettle)
            entry("dot_f32_2048", 2.0 * 2048 ** 3, "TFLOP/s", ms, PEAK["f32"], "mfma", "mfma_f32")
            da, db = put(fa_np.astype(np.float64), "f64"), put(fb_np.astype(np.float64), "f64")
            _, ms = tstat(lambda: Nx.dot(da, db), steps, warm, msettle)
            entry("dot_f64_2048", 2.0 * 2048 ** 3, "TFLOP/s", ms, PEAK["f64"], "mfma", "mfma_f64")
            del da, db
            sa, sb = W.dense_gemm_s8()
            sa, sb = put(sa, "s8"), put(sb, "s8")
            _, ms = tstat(lambda: Nx.dot(sa, sb, out_type="s32"), steps, warm, msettle)
            entry("dot_s8_4096_s32", flop, "TOP/s", ms, PEAK["s8"], "mfma", "mfma_s8")
            sbt = Nx.transpose(sb)
            _, ms = tstat(lambda: Nx.dot(sa, [1], sbt, [1], out_type="s32"), steps, warm, msettle)
            entry("dot_s8_4096_s32_kinner", flop, "TOP/s", ms, PEAK["s8"], "mfma", "mfma_s8")
            # a serving batch against one weight matrix (bound by the 33.5 MB of weights; K is split over the
            # work-groups of the under-filled grid) and a mid-size square (one 128 x 128 tile per CU)
            xa, wb = put(a_np[:128].copy(), "bf16"), bt
            _, ms = tstat(lambda: Nx.dot(xa, [1], wb, [1]), steps, warm)
            entry("dot_bf16_128x4096x4096", 2.0 * (128 * 4096 * 2) + 4096 * 4096 * 2.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            ma, mb = put(a_np[:2048, :2048].copy(), "bf16"), put(b_np[:2048, :2048].copy(), "bf16")
            _, ms = tstat(lambda: Nx.dot(ma, mb), steps, warm)
            entry("dot_bf16_2048", 2.0 * 2048 ** 3, "TFLOP/s", ms, PEAK["bf16"], "mfma", "mfma_bf16")
            # a prefill-sized batch against the weight matrix (256 tiles of 128 x 128, 64 slabs of K each)
            pa = put(a_np[:1024].copy(), "bf16")
            _, ms = tstat(lambda: Nx.dot(pa, b), steps, warm)
            entry("dot_bf16_1024x4096x4096", 2.0 * 1024 * 4096 * 4096, "TFLOP/s", ms, PEAK["bf16"], "mfma", "mfma_bf16")
            # mid-size int8: both operands K-inner, and the plain layout (right operand K-outer, laid out K-inner first)
            qa, qb = (put(q, "s8") for q in W.dense_gemm_s8(n=2048))
            qbt = Nx.transpose(qb)
            _, ms = tstat(lambda: Nx.dot(qa, [1], qbt, [1], out_type="s32"), steps, warm)
            entry("dot_s8_2048_s32_kinner", 2.0 * 2048 ** 3, "TOP/s", ms, PEAK["s8"], "mfma", "mfma_s8")
            _, ms = tstat(lambda: Nx.dot(qa, qb, out_type="s32"), steps, warm)
            entry("dot_s8_2048_s32", 2.0 * 2048 ** 3, "TOP/s", ms, PEAK["s8"], "mfma", "mfma_s8")
            del xa, wb, ma, mb, pa, qa, qb, qbt
            ha, hb = put(W.bf16_to_f32(a_np).astype(np.float16), "f16"), put(W.bf16_to_f32(b_np).astype(np.float16), "f16")
            _, ms = tstat(lambda: Nx.dot(ha, hb), steps, warm, msettle)
            entry("dot_f16_4096", flop, "TFLOP/s", ms, PEAK["f16"], "mfma", "mfma_f16")
            del fa, fb, sa, sb, bt, sbt, ha, hb

        if section("config1"):
            # config 1 (and a HBM-resident scale of it)
            for nn in (1024, 16384):
                x, y = W.elementwise_reduce(n=nn)
                x, y = put(x, "f32"), put(y, "f32")
                N = nn * nn
                _, ms = tstat(lambda: Nx.add(x, y), steps, warm)
                entry(f"add_f32_{nn}", 12.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
                _, ms = tstat(lambda: Nx.multiply(x, 0.5), steps, warm)
                entry(f"multiply_scalar_f32_{nn}", 8.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
                _, ms = tstat(lambda: Nx.exp(x), steps, warm)
                entry(f"exp_f32_{nn}", 8.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
                _, ms = tstat(lambda: Nx.sum(x, axes=[1]), steps, warm)
                entry(f"sum_rows_f32_{nn}", 4.0 * N + 4.0 * nn, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
                # the whole unfused chain of config 1: add -> multiply 0.5 -> exp -> sum over axis 1
                _, ms = tstat(lambda: Nx.sum(Nx.exp(Nx.multiply(Nx.add(x, y), 0.5)), axes=[1]), steps, warm)
                entry(f"config1_chain_f32_{nn}", 32.0 * N + 4.0 * nn, "GB/s", ms, PEAK_HBM_GBS, "hbm")
                del x, y

        if section("bf16"):
            # the same callbacks on the 2-byte type of most model tensors (bf16, 16384^2), a column sum and a transpose
            rng16 = np.random.default_rng(16)
            bx = put((rng16.standard_normal((16384, 16384)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16), "bf16")
            N = 16384 * 16384
            by = put((rng16.standard_normal((16384, 16384)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16), "bf16")
            _, ms = tstat(lambda: Nx.add(bx, by), steps, warm)
            entry("add_bf16_16384", 6.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del by
            _, ms = tstat(lambda: Nx.exp(bx), steps, warm)
            entry("exp_bf16_16384", 4.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            _, ms = tstat(lambda: Nx.sum(bx, axes=[1]), steps, warm)
            entry("sum_rows_bf16_16384", 2.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            _, ms = tstat(lambda: Nx.sum(bx, axes=[0]), steps, warm)
            entry("sum_columns_bf16_16384", 2.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            _, ms = tstat(lambda: Nx.argmax(bx, axis=1), steps, warm)
            entry("argmax_rows_bf16_16384", 2.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            _, ms = tstat(lambda: Nx.transpose(bx), steps, warm)
            entry("transpose_bf16_16384", 4.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            _, ms = tstat(lambda: Nx.as_type(bx, "f32"), steps, warm)
            entry("as_type_bf16_f32_16384", 6.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del bx

        if section("config3"):
            # config 3: attention scores + softmax chain
            q, k = W.attention_scores()
            q, k = put(q, "bf16"), put(k, "bf16")
            _, ms = tstat(lambda: Nx.dot(q, [2], [0], k, [2], [0]), steps, warm)
            entry("dot_qk_bf16_32x512x64", 20971520.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_write")
            q_np, k_np = W.attention_scores()
            nxt = rotating(lambda: (put(q_np, "bf16"), put(k_np, "bf16")), q_np.nbytes + k_np.nbytes)

            def qk_rot():
                qq, kk = nxt()
                return Nx.dot(qq, [2], [0], kk, [2], [0])
            _, ms = tstat(qk_rot, steps, warm)
            entry("dot_qk_bf16_32x512x64_rotated", 20971520.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_write")
            del nxt
            s = Nx.dot(q, [2], [0], k, [2], [0])

            def softmax():
                z = Nx.multiply(Nx.as_type(s, "f32"), 0.125)
                e = Nx.exp(Nx.subtract(z, Nx.reduce_max(z, axes=[2], keep_axes=True)))
                return Nx.divide(e, Nx.sum(e, axes=[2], keep_axes=True))
            _, ms = tstat(softmax, steps, warm)
            entry("softmax_chain_32x512x512", 386138112.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            nxt = rotating(lambda: Nx.dot(q, [2], [0], k, [2], [0]), 32 * 512 * 512 * 2)

            def softmax_rot():
                z = Nx.multiply(Nx.as_type(nxt(), "f32"), 0.125)
                e = Nx.exp(Nx.subtract(z, Nx.reduce_max(z, axes=[2], keep_axes=True)))
                return Nx.divide(e, Nx.sum(e, axes=[2], keep_axes=True))
            _, ms = tstat(softmax_rot, steps, warm)
            entry("softmax_chain_32x512x512_rotated", 386138112.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del q, k, s, nxt

        if section("config4"):
            # config 4: int8 weight-only linear
            w, xq, sc = W.int8_linear()
            w, xq, sc = put(w, "s8"), put(xq, "s8"), put(sc, "f32")
            _, ms = tstat(lambda: Nx.dot(xq, [1], w, [1], out_type="s32"), steps, warm)
            entry("dot_s8_w8_64x11008x4096", 48168960.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            suite["dot_s8_w8_64x11008x4096"]["tops"] = round(5771362304.0 / (ms * 1e-3) / 1e12, 2)
            w_np = W.int8_linear()[0]
            nxt = rotating(lambda: put(w_np, "s8"), w_np.nbytes)
            _, ms = tstat(lambda: Nx.dot(xq, [1], nxt(), [1], out_type="s32"), steps, warm)
            entry("dot_s8_w8_64x11008x4096_rotated", 48168960.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            # the same layer with its weights stored [K, N], the plain Nx.dot(x, w) of a dense layer (K-outer weights)
            nxt_t = rotating(lambda: put(np.ascontiguousarray(w_np.T), "s8"), w_np.nbytes)
            _, ms = tstat(lambda: Nx.dot(xq, nxt_t(), out_type="s32"), steps, warm)
            del nxt_t
            entry("dot_s8_w8_64x11008x4096_weights_k_outer_rotated", 48168960.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            # the whole config: dot -> as_type f32 -> multiply by the per-column scales
            _, ms = tstat(lambda: Nx.multiply(Nx.as_type(Nx.dot(xq, [1], nxt(), [1], out_type="s32"), "f32"), sc), steps, warm)
            entry("config4_chain_rotated", 48168960.0 + 5636096.0 + 5680128.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del w, xq, sc, nxt

        if section("config5"):
            # config 5: argmax + take
            logits, table, _ = W.logits_and_table()
            logits, table = put(logits, "f32"), put(table, "bf16")
            _, ms = tstat(lambda: Nx.argmax(logits, axis=1, type="u32"), steps, warm)
            entry("argmax_f32_8192x32000", 1048608768.0, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            idx = Nx.argmax(logits, axis=1, type="u32")
            _, ms = tstat(lambda: Nx.take(table, idx), steps, warm)
            entry("take_bf16_8192_of_32000x4096", 134250496.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            suite["take_bf16_8192_of_32000x4096"]["note"] = (
                "per call, not per kernel; the indices are the argmax's own result, which the library knows to lie within "
                "an axis of 32000 entries: the raising bounds policy does not wait for the kernel (the kernel itself "
                "runs ~22 us = ~6.1 TB/s by the rocprofv3 kernel trace)")
            # other rows every step (nine index sets, 600 MB of table rows in all: nothing comes from the cache), each set
            # the argmax over its own {8192, 32000} tensor of random words as in the configuration (indices written by
            # argmax are known to lie within an axis of that length, so the raising policy has nothing to wait for)
            from nx_amd import random as Random
            ring = []
            for part in range(9):
                ring.append(Nx.argmax(Random.random_bits(Random.key(505 + part, backend=H), shape=(8192, 32000)), axis=1, type="u32"))
            pos = [0]

            def next_argmax_indices():
                pos[0] = (pos[0] + 1) % len(ring)
                return ring[pos[0]]
            _, ms = tstat(lambda: Nx.take(table, next_argmax_indices()), steps, warm)
            entry("take_bf16_8192_of_32000x4096_rotated", 134250496.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del ring
            # indices from anywhere else (uploaded from the host): every call waits for its kernel, as the reference's
            # raising bounds check demands
            rng = np.random.default_rng(5)
            nxt = rotating(lambda: put(rng.integers(0, 32000, size=8192, dtype=np.uint32), "u32"), 40e6)
            _, ms = tstat(lambda: Nx.take(table, nxt()), steps, warm)
            entry("take_bf16_8192_of_32000x4096_rotated_foreign_indices", 134250496.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            # the same with the bounds policy that raises late (the kernel records a bad index, the next wait
            # reports it): the call no longer waits for its kernel, so this is the gather kernel's own rate
            previous = B.bounds_policy("defer")
            try:
                _, ms = tstat(lambda: Nx.take(table, nxt()), steps, warm)
            finally:
                B.bounds_policy(previous)
            entry("take_bf16_8192_of_32000x4096_rotated_deferred_bounds", 134250496.0, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del logits, table, idx, nxt

        if section("misc"):
            # selection, windows and creation at the HBM-resident size of config 1
            nn = 16384
            N = nn * nn
            x, y = W.elementwise_reduce(n=nn)
            x, y = put(x, "f32"), put(y, "f32")
            pred = Nx.greater(x, y)
            _, ms = tstat(lambda: Nx.select(pred, x, y), steps, warm)
            entry(f"select_f32_{nn}", 13.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            # take along the last axis (picks within each row: the row goes through LDS), late-raising bounds policy
            cols_idx = put(np.random.default_rng(6).integers(0, nn, size=nn, dtype=np.int32), "s32")
            previous = B.bounds_policy("defer")
            try:
                _, ms = tstat(lambda: Nx.take(x, cols_idx, axis=1), steps, warm)
            finally:
                B.bounds_policy(previous)
            entry(f"take_last_axis_f32_{nn}_deferred_bounds", 8.0 * N + 4.0 * nn, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del cols_idx
            _, ms = tstat(lambda: Nx.clip(x, -0.5, 0.5), steps, warm)
            entry(f"clip_f32_{nn}", 8.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            _, ms = tstat(lambda: Nx.slice(x, [64, 128], [nn - 128, nn - 256]), steps, warm)
            entry(f"slice_f32_{nn}", 8.0 * (nn - 128) * (nn - 256), "GB/s", ms, PEAK_HBM_GBS, "hbm")
            del pred
            _, ms = tstat(lambda: Nx.concatenate([x, y], axis=1), steps, warm)
            entry(f"concatenate_axis1_f32_{nn}", 16.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            _, ms = tstat(lambda: Nx.all(x, axes=[1]), steps, warm)
            entry(f"all_rows_f32_{nn}", 4.0 * N + nn, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read")
            _, ms = tstat(lambda: Nx.iota((nn, nn), type="f32", axis=1, backend=H), steps, warm)
            entry(f"iota_f32_{nn}", 4.0 * N, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_write")
            del x, y

        if section("random"):
            # Nx.Random on the device: 2^28 u32 words from one key (counter-based, write-only), and
            # uniform f32 samples built on them by the reference's chain of element-wise callbacks
            from nx_amd import random as Random
            key = Random.key(1701, backend=H)
            nw = 1 << 28
            _, ms = tstat(lambda: Random.random_bits(key, shape=(nw,)), steps, warm)
            entry("random_bits_u32_2p28", 4.0 * nw, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_write")
            _, ms = tstat(lambda: Random.uniform_split(key, 0.0, 1.0, shape=(nw,)), steps, warm)
            unfused_ms = float(ms)
            # bits out; shift, or, subtract, multiply, add, max each read and write the array once
            entry("uniform_f32_2p28_unfused", 4.0 * nw * 13, "GB/s", ms, PEAK_HBM_GBS, "hbm")
            # the same function traced, its bits-to-floats chain (shift, or, bitcast, subtract, ..., max) planned as
            # one group compiled for the device: the cipher writes the words, one more pass reads them and writes floats
            from nx_amd import defn as _defn
            uniform = _defn.compile(lambda k: Random.uniform_split(k, 0.0, 1.0, shape=(nw,)), key, fuse="compiled")
            _, ms = tstat(lambda: uniform(key), steps, warm)
            # priced at what it moves: the words written, then read once and the floats written
            entry("uniform_f32_2p28_fused_compiled", 4.0 * nw * 3, "GB/s", ms, PEAK_HBM_GBS, "hbm", vs=("unfused", unfused_ms))
            del key, uniform

        if section("chains"):
            # traced chains: one callback per node (the evaluator), and the same chain captured once and
            # replayed as a device graph (one submission for all its kernels)
            from nx_amd import defn
            from nx_amd.backend import fused_mode

            def chain1(a, b):
                return Nx.sum(Nx.exp(Nx.multiply(Nx.add(a, b), 0.5)), axes=[1])

            def chain3(scores):
                z = Nx.multiply(Nx.as_type(scores, "f32"), 0.125)
                e = Nx.exp(Nx.subtract(z, Nx.reduce_max(z, axes=[2], keep_axes=True)))
                return Nx.divide(e, Nx.sum(e, axes=[2], keep_axes=True))

            def chain4(xq_, w_, sc_):
                return Nx.multiply(Nx.as_type(Nx.dot(xq_, [1], w_, [1], out_type="s32"), "f32"), sc_)
            x, y = W.elementwise_reduce(n=1024)
            q, k = W.attention_scores()
            w, xq, sc = W.int8_linear()
            q, k = put(q, "bf16"), put(k, "bf16")
            n1, ns = 1024 * 1024, 32 * 512 * 512
            # name -> (function, arguments, bytes node by node, bytes as fused groups, bytes planned as one kernel)
            cases = {"config1_chain_f32_1024": (chain1, (put(x, "f32"), put(y, "f32")), 32.0 * n1 + 4096.0, 8.0 * n1 + 4096.0, 8.0 * n1 + 4096.0),
                     "softmax_chain_32x512x512": (chain3, (Nx.dot(q, [2], [0], k, [2], [0]),), 386138112.0, 10.0 * ns + 8.0 * 16384, 6.0 * ns),
                     "config4_chain": (chain4, (put(xq, "s8"), put(w, "s8"), put(sc, "f32")), 48168960.0 + 5636096.0 + 5680128.0, 48212992.0, 48212992.0)}
            for name, (fun, targs, nbytes, fbytes, pbytes) in cases.items():
                compiled = defn.compile(fun, *targs)
                _, ms = tstat(lambda: compiled(*targs), steps, warm)
                traced_ms = float(ms)
                entry(name + "_traced", nbytes, "GB/s", ms, PEAK_HBM_GBS, "hbm")
                captured = compiled.capture(*targs)
                held = captured.inputs  # arguments already in the captured buffers: no copies in
                _, ms = tstat(lambda: captured(*held), steps, warm)
                entry(name + "_graph", nbytes, "GB/s", ms, PEAK_HBM_GBS, "hbm", vs=("traced", traced_ms))
                captured.destroy()
                # (for configuration 4 the planner also finishes the layer on the dot's accumulators: dot, as_type and
                # the multiplication by the scales are one kernel)
                # element-wise groups (with the row reduction that follows them) as one kernel each: decoded by
                # the interpreting kernels, then with each group's program compiled for the device on first use.
                # A fused entry is priced at the bytes IT moves; `vs_traced` is its speed-up over node by node.
                fused = defn.compile(fun, *targs, fuse=True)
                for mode, tag in (("interpreted", "_fused"), ("compiled", "_fused_compiled")):
                    fused_mode(mode)
                    _, ms = tstat(lambda: fused(*targs), steps, warm)
                    entry(name + tag, fbytes, "GB/s", ms, PEAK_HBM_GBS, "hbm", vs=("traced", traced_ms))
                fused_mode("interpreted")
                # planned for compiled kernels from the start: groups over the same rows become stages of one program
                # (the softmax: row maximum, sum of exponentials and division in one kernel)
                staged = defn.compile(fun, *targs, fuse="compiled")
                _, ms = tstat(lambda: staged(*targs), steps, warm)
                entry(name + "_planned_compiled", pbytes, "GB/s", ms, PEAK_HBM_GBS, "hbm", vs=("traced", traced_ms))
            x, y = W.elementwise_reduce(n=16384)
            big = (put(x, "f32"), put(y, "f32"))
            node_ms = suite["config1_chain_f32_16384"]["ms"] if "config1_chain_f32_16384" in suite else None
            fused = defn.compile(chain1, *big, fuse=True)
            # priced at what the one pass moves (both operands once, one value per row)
            for mode, tag in (("interpreted", "_fused"), ("compiled", "_fused_compiled")):
                fused_mode(mode)
                _, ms = tstat(lambda: fused(*big), steps, warm)
                entry("config1_chain_f32_16384" + tag, 8.0 * 16384 * 16384 + 4.0 * 16384, "GB/s", ms, PEAK_HBM_GBS, "hbm", "stream_read",
                      vs=("node_by_node", node_ms) if node_ms else None)
            fused_mode("interpreted")
            del big, x, y
            del cases, q, k

        if section("softmax1m"):
            # the one benchmark the reference publishes (nx/README.md:135-146, exla/bench/softmax.exs:1-41):
            # softmax(n) = exp(n) / sum(exp(n)) on 1,000,000 uniform values kept on the device, f32 and f64 --
            # node by node (four callbacks: exp, exp, sum over all axes, divide by the rank-0 sum) and traced with
            # its groups planned for compiled kernels.  Its published figures (hardware unstated) ride along as context.
            published = {"f32": {"exla_gpu_kept_on_device_us": 65.3, "exla_host_jit_us": 2300.0, "binary_backend_us": 311010.0},
                         "f64": {"exla_gpu_kept_on_device_us": 220.0, "exla_host_jit_us": 5940.0, "binary_backend_us": 321700.0}}
            rng1m = np.random.default_rng(1000000)
            vals = rng1m.random(1000000)

            def softmax1m(n_):
                return Nx.divide(Nx.exp(n_), Nx.sum(Nx.exp(n_)))
            for ty, npt, esz in (("f32", np.float32, 4), ("f64", np.float64, 8)):
                t1m = put(vals.astype(npt), ty)
                nel = 1000000.0
                _, ms = tstat(lambda: softmax1m(t1m), steps, warm)
                eager_ms = float(ms)
                # exp, exp: 2 x (read + write); sum: read + one element; divide: read + read of one element + write
                entry(f"softmax_1M_{ty}", esz * nel * 7 + 3 * esz, "GB/s", ms, PEAK_HBM_GBS, "hbm")
                suite[f"softmax_1M_{ty}"]["reference_published_us"] = published[ty]
                suite[f"softmax_1M_{ty}"]["note"] = ("4 MB (8 MB) tensors: launch-bound, not bandwidth-bound; the reference's figures are for unstated "
                                                     "hardware (nx/README.md:135-146)")
                try:
                    planned = defn.compile(softmax1m, t1m, fuse="compiled")
                    _, ms = tstat(lambda: planned(t1m), steps, warm)
                    # priced at what it has to move: the values read (twice: once for the sum, once for the quotient) and written
                    entry(f"softmax_1M_{ty}_planned_compiled", esz * nel * 3, "GB/s", ms, PEAK_HBM_GBS, "hbm", vs=("unfused", eager_ms))
                    del planned
                except Exception as exc:  # a type the planner does not group: the node-by-node figure stands
                    suite[f"softmax_1M_{ty}_planned_compiled"] = {"error": str(exc)[:160]}
                del t1m
        result["suite"] = suite
        if args.only is None:
            result["host_transfers"] = host_transfer_figures(H, B, Nx, template)
        c_abi = c_abi_figures() if args.only is None else None
        if c_abi:
            result["c_abi"] = c_abi
            if "config1_chain_f32_1024_us" in c_abi:
                us = c_abi["config1_chain_f32_1024_us"]
                suite["config1_chain_f32_1024_c_abi"] = {
                    "ms": round(us / 1e3, 5), "achieved": round((32.0 * 1024 * 1024 + 4096.0) / (us * 1e-6) / 1e9, 2), "unit": "GB/s",
                    "bound": "hbm", "peak": PEAK_HBM_GBS, "frac": round((32.0 * 1024 * 1024 + 4096.0) / (us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
                    "note": "the same four callbacks issued from plain C (no Python): per chain, device kept busy"}

    # ---- CPU baseline: the reference-semantics restatement on a bounded sample -----------------
    if not args.no_cpu:
        from oracle import binary_backend as O
        threads = min(os.cpu_count() or 1, 16)
        O.set_threads(threads)
        oa = O.BinaryBackend.from_binary(template("bf16", (n, n)), a_np.tobytes())
        ob = O.BinaryBackend.from_binary(template("bf16", (n, n)), b_np.tobytes())
        passes, t0 = 0, time.perf_counter()
        while passes < 1 or (time.perf_counter() - t0 < 12.0 and passes < 8):
            Nx.dot(oa, ob)
            passes += 1
        dt = time.perf_counter() - t0
        O.set_threads(1)
        rows1 = 64
        oa1 = O.BinaryBackend.from_binary(template("bf16", (rows1, n)), a_np[:rows1].tobytes())
        t1 = time.perf_counter()
        Nx.dot(oa1, ob)
        dt1 = time.perf_counter() - t1
        O.set_threads(threads)
        # an optimised, vectorised CPU GEMM on the same cores (the role a host compiler back end plays
        # upstream): torch's f32 matmul on bf16-representable values, in a child process
        vectorised = None
        probe = ("import time, torch; torch.set_num_threads(%d); g = torch.Generator().manual_seed(2);"
                 "a = (torch.randn(%d, %d, generator=g) / 64).bfloat16().float();"
                 "b = (torch.randn(%d, %d, generator=g) / 64).bfloat16().float();"
                 "torch.matmul(a, b); t = time.perf_counter(); k = 0\n"
                 "while time.perf_counter() - t < 3.0: torch.matmul(a, b); k += 1\n"
                 "print(k, time.perf_counter() - t)") % (threads, n, n, n, n)
        try:
            import subprocess
            out = subprocess.run([sys.executable, "-c", probe], capture_output=True, text=True, timeout=120)
            k, secs = out.stdout.split()[-2:]
            vectorised = {"value": round(int(k) * flop / float(secs) / 1e12, 4), "unit": "TFLOP/s", "cores": threads,
                          "sample": f"{k} passes of torch.matmul f32 4096^3 on bf16-representable values, "
                                    f"{float(secs):.1f} s; not reference semantics (f32 blocked accumulation)"}
        except Exception as exc:  # the figure is an extra; the baseline proper is below
            vectorised = {"value": None, "error": str(exc)[:200]}
        # the other configurations on the same restatement, one pass each at the benchmark's shapes (a quarter of
        # the rows for configuration 5, said in its sample): what the reference's formulation costs on the host cores
        def cpu_pass(fun):
            t = time.perf_counter()
            fun()
            return round((time.perf_counter() - t) * 1e3, 2)

        def oput(arr, ty):
            return O.BinaryBackend.from_binary(template(ty, arr.shape), np.ascontiguousarray(arr).tobytes(), {})
        per_config = {}
        previous = Nx.default_backend(O.BinaryBackend)  # scalar operands of these passes belong on the host too
        cx, cy = (oput(v, "f32") for v in W.elementwise_reduce(n=1024))
        per_config["config1_chain_f32_1024"] = {"ms": cpu_pass(lambda: Nx.sum(Nx.exp(Nx.multiply(Nx.add(cx, cy), 0.5)), axes=[1])),
                                                "sample": "add, multiply, exp, sum at 1024^2, one pass"}
        cq, ck = (oput(v, "bf16") for v in W.attention_scores())
        scores = []
        per_config["dot_qk_bf16_32x512x64"] = {"ms": cpu_pass(lambda: scores.append(Nx.dot(cq, [2], [0], ck, [2], [0]))),
                                               "sample": "the batched dot, one pass"}

        def cpu_softmax():
            z = Nx.multiply(Nx.as_type(scores[0], "f32"), 0.125)
            e = Nx.exp(Nx.subtract(z, Nx.reduce_max(z, axes=[2], keep_axes=True)))
            return Nx.divide(e, Nx.sum(e, axes=[2], keep_axes=True))
        per_config["softmax_chain_32x512x512"] = {"ms": cpu_pass(cpu_softmax), "sample": "the eight callbacks, one pass"}
        cw, cxq, csc = W.int8_linear()
        cw, cxq, csc = oput(cw, "s8"), oput(cxq, "s8"), oput(csc, "f32")
        per_config["config4_chain"] = {"ms": cpu_pass(lambda: Nx.multiply(Nx.as_type(Nx.dot(cxq, [1], cw, [1], out_type="s32"), "f32"), csc)),
                                       "sample": "dot, as_type, multiply at 64 x 11008 x 4096, one pass"}
        clog, ctab, _ = W.logits_and_table(rows=2048)
        clog, ctab = oput(clog, "f32"), oput(ctab, "bf16")
        per_config["argmax_take_2048_of_8192_rows"] = {"ms": cpu_pass(lambda: Nx.take(ctab, Nx.argmax(clog, axis=1, type="u32"))),
                                                       "sample": "argmax over 2048 x 32000 logits and take of 2048 rows of 4096 bf16: a quarter of the benchmark's rows"}
        del cx, cy, cq, ck, scores, cw, cxq, csc, clog, ctab
        Nx.default_backend(*previous)
        result["cpu_baseline"] = {
            "value": round(passes * flop / dt / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{passes} passes of the whole bf16 4096^3 GEMM (f64 sequential accumulation, reference "
                      f"semantics, rows spread over {threads} OpenMP threads), {dt:.1f} s",
            "single_thread": {"value": round(2.0 * rows1 * n * n / dt1 / 1e12, 6), "unit": "TFLOP/s",
                              "sample": f"first {rows1} of 4096 output rows, {dt1:.1f} s"},
            "vectorised_library": vectorised,
            "other_configurations": per_config}

    emit(result)


def emit(result):
    """The full record (suite, ceilings, host transfers, plain-C figures, the CPU baseline's extras) goes to
    `gpurun_out/bench_suite.json` and, as a short table, to stdout; the LAST stdout line is the headline
    alone, a few hundred bytes of JSON that a reader of the output's tail can parse."""
    detail_path = os.path.join(ROOT, "gpurun_out", "bench_suite.json")
    try:
        os.makedirs(os.path.dirname(detail_path), exist_ok=True)
        with open(detail_path, "w") as f:
            json.dump(result, f)
    except OSError as exc:  # a read-only tree: the table below still carries the figures
        detail_path = "not written: " + str(exc)[:80]
    suite = result.get("suite", {})
    if suite:
        print("%-58s %10s %10s %9s %6s %6s" % ("suite entry (device time per call)", "us", "achieved", "unit", "frac", "bound"))
        for name, e in suite.items():
            if "ms" in e:
                print("%-58s %10.2f %10.1f %9s %6.3f %6s" % (name, e["ms"] * 1e3, e["achieved"], e["unit"], e["frac"], e["bound"]))
    for name, c in result.get("ceilings", {}).items():
        if "sustained" in c:
            print("ceiling %-50s %10s sustained" % (name, c["sustained"]))
    head = {k: result[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                                   "scaling", "vs_baseline", "dtype", "data", "config", "roofline")}
    cpu = result.get("cpu_baseline")
    if cpu:
        head["cpu_baseline"] = {k: cpu[k] for k in ("value", "unit", "cores", "kind", "sample")}
    head["cold_start"] = result["cold_start"]["tflops"]
    # the other figures the targets are stated on, one fraction each (full entries in the detail file)
    also = {}
    for name in HEADLINE_ALSO:
        if name in suite:
            also[name] = {"us": round(suite[name]["ms"] * 1e3, 2), "frac": suite[name]["frac"], "of": suite[name]["bound"]}
    if also:
        head["also"] = also
    head["detail"] = "gpurun_out/bench_suite.json" if not detail_path.startswith("not written") else detail_path
    line = json.dumps(head)
    assert len(line) < 4096, "headline JSON line is %d bytes: keep it under 4 KB" % len(line)
    sys.stdout.flush()
    print(line, flush=True)


if __name__ == "__main__":
    main()
