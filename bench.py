#!/usr/bin/env python3
"""Benchmark of the MI355X block-scaled FP8 GEMM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4] [--no-shapes] [--no-cpu]
                    [--no-challenge]

A step is one GEMM call (C ABI, fp8_block_gemm_stream) on one configuration's synthetic
inputs, already resident in HBM.  The headline workload is cfg4 (M=8192, N=4608, K=7168,
the MFMA-utilisation shape); the other four configurations are timed too (shorter runs)
and listed under "shapes" with the geomean latency.  "challenge" holds the 18 shapes of the
reference's own results table (/root/reference/README.md:15-25, measured there on an MI300X)
with this library's latency on each and the geomean of the 18.  One JSON line is printed.

Timing: W untimed warm-up steps -- and as many more as it takes to keep the device under this
load for SETTLE_MS: after any idle gap, however short, the part needs about 30 ms of continuous
work to reach its steady clock (the first launches of the headline shape take 340 us, the
hundredth 240 us, and it stays there) --, then exactly K steps between two device
synchronisations (wall clock -> ms_per_step, value), then a region of at least K steps and at
least 5 ms between two HIP events recorded on the launch stream, entered without an idle gap
(-> roofline.achieved: algorithmic flops or bytes of one launch / average launch duration; the
per-shape latencies are this figure).
cpu_baseline times the CPU oracle (the restatement of the reference's arithmetic) on the whole
headline workload, once, with all host threads (about 15 CPU-seconds).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5033.0   # 256 CU x 2.4 GHz x 8192 flop/CU/clk (dense, v_mfma_f32_16x16x128_f8f6f4)
PEAK_HBM_GBS = 8000.0
SETTLE_MS = 80.0            # continuous load before a timed region (steady device clock)
HBM_BOUND = {"cfg5"}
COLD_TOO = {"cfg1", "cfg3", "cfg5"}   # latency-bound shapes: also timed behind a cache flush

# (k, n, MI300X latency in us for m=1024, for m=6144): the reference's published table,
# /root/reference/README.md:15-25; its geomean over the 18 shapes is 136 us (README.md:13).
CHALLENGE = [(7168, 1536, 147, 341), (1536, 3072, 50.6, 160), (7168, 576, 75.9, 173),
             (256, 7168, 30.9, 88.6), (2048, 7168, 106, 426), (7168, 4608, 193, 948),
             (2304, 7168, 120, 479), (7168, 512, 75.1, 163), (512, 4096, 30.9, 97.7)]
CHALLENGE_REF_GEOMEAN_US = 136.0

# Bytes per launch that crossed the L2 <-> fabric boundary (Infinity Cache / HBM side), from
# rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs (KiB per dispatch, steady-state launches), each
# scaled by what the same counter reads for a 1 GiB copy kernel in the same session: FETCH_SIZE
# reads 0.5 of the bytes copied (factor 2.0), WRITE_SIZE reads them exactly (factor 1.0).
# profiles/counters_cfg1_to_cfg5.md holds the table; the kernels measured are those of the commit
# named here (the kernels of these plans have not changed since).
TRAFFIC_MEASURED_AT_COMMIT = "a37a2c8"
MEASURED_TRAFFIC_BYTES = {
    "cfg1": int((5235 * 2.0 + 3072 * 1.0) * 1024),       # 13.9 MB: C + the mailbox traffic of the K split
    "cfg2": int((115831 * 2.0 + 114688 * 1.0) * 1024),   # 355 MB
    "cfg3": int((28731 * 2.0 + 20315 * 1.0) * 1024),     # 79.6 MB, one kernel (K splits added inside it)
    "cfg4": int((242077 * 2.0 + 73728 * 1.0) * 1024),    # 571 MB: 8 L2s refetch A/B panels
    "cfg5": int((8841 * 2.0 + 3136 * 1.0) * 1024),       # 21.3 MB: B once (1.23 x the reads) + mailbox write-back
}


def max_sclk_mhz():
    """highest "Max Clock Freq. (MHz)" rocminfo lists for a GPU agent, or None"""
    import re
    import subprocess
    try:
        text = subprocess.run(["/opt/rocm/bin/rocminfo"], capture_output=True, text=True, timeout=30).stdout
    except Exception:
        return None
    best = None
    for agent in text.split("*******")[1:]:
        if "Device Type:             GPU" not in agent and not re.search(r"Device Type:\s+GPU", agent):
            continue
        mm = re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", agent)
        if mm:
            best = max(best or 0, int(mm.group(1)))
    return best


def algorithmic_work(m, n, k):
    flops = 2.0 * m * n * k
    sn = (n + 127) // 128
    byts = m * k + n * k + 4 * (k // 128) * m + 4 * (k // 128) * sn + 2 * m * n
    return flops, float(byts)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg4")
    ap.add_argument("--no-shapes", action="store_true", help="time the headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-challenge", action="store_true",
                    help="skip the 18 shapes of the reference's results table")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus above 1 is not supported "
              "(the GEMM shards by rows of A or 128-column blocks of B without exchange, "
              "but no multi-GPU path is built)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import __graft_entry__ as ge
    import oracle

    pkg = ge.load_package()
    pkg.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    sptr = stream.cuda_stream

    def prepare(name):
        if isinstance(name, tuple):
            m, n, k, seed = name
            a, b, sa, sb = oracle.make_inputs(m, n, k, seed)
        else:
            m, n, k, a, b, sa, sb = oracle.make_config_inputs(name)
        dev = [torch.from_numpy(x).cuda() for x in (a, b, sa, sb)]
        dc = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
        return (m, n, k), (a, b, sa, sb), dev, dc

    def step(dev, dc, shape):
        pkg.gemm(dev[0], dev[1], dev[2], dev[3], dc, shape[0], shape[1], shape[2], sptr)

    def parity(host, dc, shape, npts=8192):
        m, n, k = shape
        rs = np.random.RandomState(1234)
        rows = rs.randint(0, m, npts).astype(np.int32)
        cols = rs.randint(0, n, npts).astype(np.int32)
        _, refh = oracle.ref_gemm_points(host[0], host[1], host[2], host[3], rows, cols, m, n, k)
        got = dc.cpu().numpy().view(np.uint16)[rows, cols]
        # bound from the sampled points' own max |ref|: stricter than the whole-matrix rule
        r = oracle.compare_bf16(got, refh, 1e-2, 1e-3)
        return {"points": npts, "max_err": r["max_err"], "bound": r["bound"], "pass": r["bad"] == 0}

    def settle(fn, warmup):
        """warm-up: at least `warmup` calls of fn, and at least SETTLE_MS of continuous load"""
        t0 = time.perf_counter()
        done, batch, per_call_ms = 0, max(warmup, 10), 0.0
        while done < warmup or (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
            tb = time.perf_counter()
            for _ in range(batch):
                fn()
            done += batch
            torch.cuda.synchronize()
            per_call_ms = (time.perf_counter() - tb) * 1e3 / batch
            if per_call_ms * batch < 5.0:
                batch *= 2   # short kernels: fewer synchronisation gaps in the load
        return per_call_ms

    def timed(dev, dc, shape, steps, warmup, exact=False):
        """(wall ms, event ms) per step.  The event figure comes from a region of at least
        `steps` steps and at least 5 ms, entered straight from the warm-up load without a
        host synchronisation: after any idle gap the first launches are slow, which a region of
        thirty 5-us kernels would mostly measure.  With `exact`, the wall figure is taken
        over exactly `steps` steps between two device synchronisations."""
        run = lambda: step(dev, dc, shape)
        per_call_ms = settle(run, warmup)
        wall_ms = None
        if exact:
            t0 = time.perf_counter()
            for _ in range(steps):
                run()
            torch.cuda.synchronize()
            wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        ev_steps = max(steps, int(5.0 / per_call_ms)) if per_call_ms > 0 else steps
        bridge = max(1, min(ev_steps, int(0.5 / per_call_ms))) if per_call_ms > 0 else 1
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        for _ in range(bridge):   # untimed: the queue is busy when the first event is reached
            run()
        e0.record(stream)
        for _ in range(ev_steps):
            run()
        e1.record(stream)
        torch.cuda.synchronize()
        if wall_ms is None:
            wall_ms = (time.perf_counter() - t0) * 1e3 / (bridge + ev_steps)
        return wall_ms, e0.elapsed_time(e1) / ev_steps

    def launch_stats_us(dev, dc, shape, reps=20):
        """median and minimum of single launches, each between its own pair of events"""
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range(reps)]
        for e0, e1 in ev:
            e0.record(stream)
            step(dev, dc, shape)
            e1.record(stream)
        torch.cuda.synchronize()
        ts = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in ev)
        return ts[len(ts) // 2], ts[0]

    def cold_latency_us(dev, dc, shape, reps=10):
        """per-launch latency with caches flushed by a 1 GiB fill between launches"""
        junk = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        ts = []
        for i in range(reps):
            junk.fill_(i)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            step(dev, dc, shape)
            e1.record(stream)
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        del junk
        ts.sort()
        return ts[len(ts) // 2]

    def rotating_operand_us(dev, dc, shape, min_bytes=640 << 20, launches=600):
        """Launches back to back, each on another copy of B: more copies than the part's 256 MB
        Infinity Cache and its L2s hold together (`min_bytes` of B in total), so B comes from HBM every
        time, as the weights of successive layers do in a decode step.  No fill kernel, no idle gap."""
        m_, n_, k_ = shape
        copies = max(2, -(-min_bytes // (n_ * k_)))
        bs = [dev[1]] + [dev[1].clone() for _ in range(copies - 1)]
        call = lambda i: pkg.gemm(dev[0], bs[i % copies], dev[2], dev[3], dc, m_, n_, k_, sptr)
        for i in range(2 * copies):
            call(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        for i in range(copies):          # the queue is busy when the first event is reached
            call(i)
        e0.record(stream)
        for i in range(launches):
            call(i)
        e1.record(stream)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / launches
        del bs
        return us, copies

    def shape_report(name, steps, warmup, exact=False):
        shape, host, dev, dc = prepare(name)
        step(dev, dc, shape)
        torch.cuda.synchronize()
        par = parity(host, dc, shape)
        wall_ms, ev_ms = timed(dev, dc, shape, steps, warmup, exact)
        flops, byts = algorithmic_work(*shape)
        us = ev_ms * 1e3
        rep = {
            "name": name, "m": shape[0], "n": shape[1], "k": shape[2], "kernel": pkg.last_kernel(),
            "latency_us": round(us, 2), "wall_us": round(wall_ms * 1e3, 2),
            "tflops": round(flops / us * 1e-6, 1), "frac_fp8_peak": round(flops / us * 1e-6 / PEAK_FP8_TFLOPS, 4),
            "gbs": round(byts / us * 1e-3, 1), "frac_hbm_peak": round(byts / us * 1e-3 / PEAK_HBM_GBS, 4),
            "bound": "hbm" if name in HBM_BOUND else "mfma", "parity": par,
        }
        med, mn = launch_stats_us(dev, dc, shape)
        rep["single_launch_median_us"] = round(med, 2)
        rep["single_launch_min_us"] = round(mn, 2)
        if name in COLD_TOO:
            cold = cold_latency_us(dev, dc, shape)
            rep["cold_latency_us"] = round(cold, 2)
            rep["cold_gbs"] = round(byts / cold * 1e-3, 1)
        if name in HBM_BOUND:
            # the HBM-side figure: B from HBM on every launch (rotating copies), launches back to back
            rot_us, copies = rotating_operand_us(dev, dc, shape)
            rep["hbm_rotating"] = {"b_copies": copies, "b_bytes_total": copies * shape[1] * shape[2],
                                   "latency_us": round(rot_us, 2), "gbs": round(byts / rot_us * 1e-3, 1),
                                   "frac_hbm_peak": round(byts / rot_us * 1e-3 / PEAK_HBM_GBS, 4)}
        if not args.no_cpu and not isinstance(name, tuple):
            rep["cpu"] = cpu_row(shape, host)
        return rep, (shape, host, wall_ms, ev_ms)

    def cpu_row(shape, host, max_rows=1024):
        """the CPU oracle on the first rows of the same inputs, all host threads, best of up to 3"""
        m_, n_, k_ = shape
        rows = min(m_, max_rows)
        a_s = np.ascontiguousarray(host[0][:, :rows])
        sa_s = np.ascontiguousarray(host[2][:, :rows])
        threads = oracle.max_threads()
        best = None
        for _ in range(3 if 2.0 * rows * n_ * k_ < 5e10 else 1):
            t0 = time.perf_counter()
            oracle.ref_gemm(a_s, host[1], sa_s, host[3], rows, n_, k_, nthreads=threads)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return {"rows": rows, "of_rows": m_, "threads": threads, "us": round(best * 1e6, 1),
                "gflops": round(2.0 * rows * n_ * k_ / best * 1e-9, 1),
                "full_shape_us_extrapolated": round(best * 1e6 * m_ / rows, 1)}

    def challenge_report(steps, warmup):
        rows = []
        for mi, m in enumerate((1024, 6144)):
            for ci, (k, n, ref_1024, ref_6144) in enumerate(CHALLENGE):
                shape, host, dev, dc = prepare((m, n, k, 2000 + 100 * mi + ci))
                step(dev, dc, shape)
                torch.cuda.synchronize()
                par = parity(host, dc, shape, npts=2048)
                _, ev_ms = timed(dev, dc, shape, steps, warmup)
                us = ev_ms * 1e3
                rows.append({"m": m, "n": n, "k": k, "kernel": pkg.last_kernel(),
                             "latency_us": round(us, 2),
                             "tflops": round(2.0 * m * n * k / us * 1e-6, 1),
                             "reference_mi300x_us": ref_1024 if m == 1024 else ref_6144,
                             "parity_pass": par["pass"]})
                del dev, dc
        geo = math.exp(sum(math.log(r["latency_us"]) for r in rows) / len(rows))
        return {"shapes": rows, "geomean_latency_us": round(geo, 2),
                "reference_mi300x_geomean_us": CHALLENGE_REF_GEOMEAN_US,
                "note": "the reference's numbers are the author's MI300X measurements "
                        "(context, different hardware)"}

    def quantiser_report(steps, warmup):
        """the device-side producers of the headline workload's operands (bf16 source)"""
        out = []
        for which, rows in (("a_1x128", m), ("b_128x128", n)):
            x = torch.randn((rows, k), device="cuda", dtype=torch.float32).to(torch.bfloat16)
            q = torch.empty((k, rows), dtype=torch.uint8, device="cuda")
            ncol = rows if which == "a_1x128" else (rows + 127) // 128
            sc = torch.empty((k // 128, ncol), dtype=torch.float32, device="cuda")
            fn = pkg.quantize_a_1x128 if which == "a_1x128" else pkg.quantize_b_128x128
            settle(lambda: fn(x, q, sc, rows, k, pkg.DTYPE_BF16, sptr), warmup)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(steps):
                fn(x, q, sc, rows, k, pkg.DTYPE_BF16, sptr)
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / steps
            nbytes = 3.0 * rows * k + 4.0 * sc.numel()
            out.append({"kernel": "quantize_" + which, "rows": rows, "k": k, "source": "bf16",
                        "latency_us": round(us, 2), "algorithmic_bytes": nbytes,
                        "gbs": round(nbytes / us * 1e-3, 1),
                        "frac_hbm_peak": round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4)})
            del x, q, sc
        return out

    def vendor_plain_fp8_gemm_us(steps, warmup):
        """Context, not a baseline of this metric: torch._scaled_mm (the ROCm library GEMM) on the
        headline shape with one scale per tensor, i.e. WITHOUT the per-128-K-block fold."""
        try:
            xa = torch.randn((m, k), device="cuda").clamp(-3, 3).to(torch.float8_e4m3fn)
            xb = torch.randn((n, k), device="cuda").clamp(-3, 3).to(torch.float8_e4m3fn)
            one = torch.tensor(1.0, device="cuda")
            fn = lambda: torch._scaled_mm(xa, xb.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
            settle(fn, warmup)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(steps):
                fn()
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / steps
            return {"what": "torch._scaled_mm, per-tensor scales (no block-scale fold), same M N K",
                    "latency_us": round(us, 2), "tflops": round(flops / us * 1e-6, 1),
                    "frac_fp8_peak": round(flops / us * 1e-6 / PEAK_FP8_TFLOPS, 4)}
        except Exception as exc:  # library or dtype not available: context only
            return {"what": "torch._scaled_mm unavailable", "error": repr(exc)[:200]}

    def host_boundary_report():
        """fp8_gemm_host on the headline shape: host fp32 values in, bf16 out, device memory
        allocated, filled over PCIe, converted, multiplied, read back and freed inside the call
        (pageable host memory, as the reference's harness uses).  Never `value`."""
        ha, hb, sa, sb = host
        af, bf = oracle.e4m3fn_decode(ha), oracle.e4m3fn_decode(hb)
        ch = np.zeros((m, n), np.uint16)
        L = pkg.lib()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            rc = L.fp8_gemm_host(ch.ctypes.data, af.ctypes.data, bf.ctypes.data, sa.ctypes.data,
                                 sb.ctypes.data, m, n, k, 0)
            dt = time.perf_counter() - t0
            if rc != 0:
                return {"error": rc}
            best = dt if best is None else min(best, dt)
        moved = af.nbytes + bf.nbytes + sa.nbytes + sb.nbytes + ch.nbytes
        return {"what": "fp8_gemm_host, best of 3: alloc + PCIe in (fp32 values) + convert + GEMM + PCIe out + free",
                "ms": round(best * 1e3, 2), "tflops": round(flops / best * 1e-12, 2),
                "host_bytes_moved": moved, "host_gbs": round(moved / best * 1e-9, 1)}

    def grouped_report(steps, warmup, ms=(512, 1024, 768, 1536, 256, 2048, 1024, 1024)):
        """cfg2's problem cut into eight groups of ragged M (an MoE layer's experts): one grouped
        launch against eight launches of fp8_block_gemm_stream, same buffers"""
        ms = list(ms)
        gn, gk = 7168, 2048
        bufs = []
        for g, gm in enumerate(ms):
            a_, b_, sa_, sb_ = oracle.make_inputs(gm, gn, gk, 5000 + g)
            bufs.append([torch.from_numpy(x).cuda() for x in (a_, b_, sa_, sb_)] +
                        [torch.zeros((gm, gn), dtype=torch.int16, device="cuda")])
        cols = lambda i: [bf[i] for bf in bufs]
        grouped = lambda: pkg.gemm_grouped(cols(0), cols(1), cols(2), cols(3), cols(4), ms, gn, gk, sptr)

        def one_by_one():
            for bf, gm in zip(bufs, ms):
                pkg.gemm(bf[0], bf[1], bf[2], bf[3], bf[4], gm, gn, gk, sptr)

        out = {"m": ms, "n": gn, "k": gk}
        gflop = 2.0 * sum(ms) * gn * gk
        for tag, fn in (("grouped", grouped), ("one_by_one", one_by_one)):
            settle(fn, warmup)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(steps):
                fn()
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / steps
            out[tag + "_us"] = round(us, 2)
            out[tag + "_tflops"] = round(gflop / us * 1e-6, 1)
            if tag == "grouped":
                out["kernel"] = pkg.last_kernel()
        return out

    def decode_rows_report(steps, warmup, rows=(1, 8, 16, 24, 32), dn=7168, dk=2048):
        """cfg5's weight matrix against decode batches of other sizes, among them row counts off the 16-byte
        grid (the decode kernel takes those as they are): latency with B in the caches and with B from HBM"""
        out = []
        for m in rows:
            shape, host, dev, dc = prepare((m, dn, dk, 3100 + m))
            step(dev, dc, shape)
            torch.cuda.synchronize()
            par = parity(host, dc, shape, npts=2048)
            _, ev_ms = timed(dev, dc, shape, steps, warmup)
            rot_us, _ = rotating_operand_us(dev, dc, shape)
            _, byts = algorithmic_work(*shape)
            out.append({"m": m, "n": dn, "k": dk, "kernel": pkg.last_kernel(), "latency_us": round(ev_ms * 1e3, 2),
                        "hbm_rotating_us": round(rot_us, 2), "hbm_rotating_gbs": round(byts / rot_us * 1e-3, 1),
                        "parity_pass": par["pass"]})
        return out

    def grouped_decode_report(steps, warmup, experts=64, gn=7168, gk=2048, on_grid=False, rows_hi=64):
        """an MoE layer in a decode step: `experts` problems of 1 to `rows_hi` rows each (seeded), every expert
        with its own weights (14.7 MB each: streamed from HBM on every launch).  One grouped call (one launch
        of the decode kernel on the strips of up to 64 experts) against one call per expert.  Operands are seeded random
        bytes and scales generated on the device (parity of the grouped path is the tests' business)."""
        gen = torch.Generator(device="cuda")
        gen.manual_seed(4242)
        rs = __import__("numpy").random.RandomState(4242)
        ms = [int(v) for v in rs.randint(1, rows_hi + 1, size=experts)]
        if on_grid:
            ms = [max(16, (v + 15) // 16 * 16) for v in ms]
        bufs = []
        for gm in ms:
            a_ = torch.randint(0, 120, (gk, gm), device="cuda", generator=gen, dtype=torch.int16).to(torch.uint8)
            b_ = torch.randint(0, 120, (gk, gn), device="cuda", generator=gen, dtype=torch.int16).to(torch.uint8)
            sa_ = torch.rand((gk // 128, gm), device="cuda", generator=gen) + 0.5
            sb_ = torch.rand((gk // 128, (gn + 127) // 128), device="cuda", generator=gen) + 0.5
            bufs.append([a_, b_, sa_, sb_, torch.zeros((gm, gn), dtype=torch.int16, device="cuda")])
        cols = lambda i: [bf[i] for bf in bufs]
        grouped = lambda: pkg.gemm_grouped(cols(0), cols(1), cols(2), cols(3), cols(4), ms, gn, gk, sptr)

        def one_by_one():
            for bf, gm in zip(bufs, ms):
                pkg.gemm(bf[0], bf[1], bf[2], bf[3], bf[4], gm, gn, gk, sptr)

        byts = sum(algorithmic_work(gm, gn, gk)[1] for gm in ms)
        out = {"experts": experts, "rows_total": sum(ms), "rows_min_max": [min(ms), max(ms)], "n": gn, "k": gk,
               "algorithmic_bytes": byts}
        for tag, fn in (("grouped", grouped), ("one_by_one", one_by_one)):
            settle(fn, warmup)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(steps):
                fn()
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / steps
            out[tag + "_us"] = round(us, 2)
            out[tag + "_gbs"] = round(byts / us * 1e-3, 1)
            out[tag + "_kernel"] = pkg.last_kernel()
        out["grouped_frac_hbm_peak"] = round(out["grouped_gbs"] / PEAK_HBM_GBS, 4)
        pkg.release()
        return out

    def launch_floor_us(reps=200):
        """back-to-back launches of a one-workgroup kernel of this library"""
        x = torch.zeros(256, dtype=torch.float32, device="cuda")
        y = torch.zeros(256, dtype=torch.uint8, device="cuda")
        for _ in range(10):
            pkg.convert_f32_to_e4m3fn(x, y, 256, sptr)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            pkg.convert_f32_to_e4m3fn(x, y, 256, sptr)
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    main_rep, (shape, host, wall_ms, ev_ms) = shape_report(args.workload, args.steps, args.warmup, exact=True)
    m, n, k = shape
    flops, byts = algorithmic_work(m, n, k)

    shapes = [main_rep]
    if not args.no_shapes:
        for name in oracle.CONFIGS:
            if name != args.workload:
                rep, _ = shape_report(name, max(10, args.steps // 2), args.warmup)
                shapes.append(rep)
        shapes.sort(key=lambda r: r["name"])
    geomean_us = math.exp(sum(math.log(r["latency_us"]) for r in shapes) / len(shapes))

    challenge = None
    if not args.no_challenge:
        challenge = challenge_report(max(10, args.steps // 2), args.warmup)
    floor_us = launch_floor_us()
    quantisers = None if args.no_shapes else quantiser_report(max(100, args.steps), args.warmup)
    vendor = None if args.no_shapes else vendor_plain_fp8_gemm_us(max(10, args.steps // 2), args.warmup)
    grouped = None if args.no_shapes else grouped_report(max(30, args.steps), args.warmup)
    if grouped is not None:   # the same token count with group sizes off the 16-row grid: padded copies
        grouped["off_grid"] = grouped_report(max(30, args.steps), args.warmup,
                                             ms=(509, 1027, 771, 1533, 250, 2051, 1023, 1028))
    grouped_decode = None
    if not args.no_shapes:   # 64 experts of 1..64 rows, and the same on the 16-row grid
        grouped_decode = grouped_decode_report(max(20, args.steps), args.warmup)
        grouped_decode["on_grid"] = grouped_decode_report(max(20, args.steps), args.warmup, on_grid=True)
        # every routed expert of a 256-expert layer live, a few tokens each: four launches of 64 experts
        grouped_decode["experts256"] = grouped_decode_report(max(20, args.steps), args.warmup, experts=256, rows_hi=8)
    decode_rows = None if args.no_shapes else decode_rows_report(max(20, args.steps), args.warmup)
    host_boundary = None if args.no_shapes else host_boundary_report()
    props = torch.cuda.get_device_properties(0)
    device = {"name": props.name, "compute_units": props.multi_processor_count,
              "max_sclk_mhz": max_sclk_mhz(),
              "peak_fp8_tflops_assumed": PEAK_FP8_TFLOPS, "peak_hbm_gbs_assumed": PEAK_HBM_GBS,
              "launch_floor_us": round(floor_us, 2)}

    hbm = args.workload in HBM_BOUND
    if hbm:
        achieved = byts / (ev_ms * 1e-3) * 1e-9
        roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBS, 4)}
    else:
        achieved = flops / (ev_ms * 1e-3) * 1e-12
        roof = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP8_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP8_TFLOPS, 4)}
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get(args.workload)
    roof["traffic_measured_at_commit"] = TRAFFIC_MEASURED_AT_COMMIT if roof["traffic"] else None
    roof["kernel"] = main_rep["kernel"]
    roof["launch_us"] = round(ev_ms * 1e3, 2)
    roof["algorithmic_flops"] = flops
    roof["algorithmic_bytes"] = byts

    cpu = None
    if not args.no_cpu:
        rows = m   # the whole workload: about a second of wall time on 16 threads (~15 CPU-seconds)
        a, b, sa, sb = host
        threads = oracle.max_threads()
        t0 = time.perf_counter()
        oracle.ref_gemm(a, b, sa, sb, rows, n, k, nthreads=threads)
        dt = time.perf_counter() - t0
        cpu = {"value": round(2.0 * rows * n * k / dt * 1e-12, 4), "unit": "TFLOP/s", "cores": threads,
               "kind": "port", "seconds": round(dt, 3),
               "sample": f"the whole workload (all {m} rows of A, all {n} columns, K={k}), one run of the "
                         f"CPU oracle oracle_ref_gemm"}
        if not args.no_shapes:
            m1, n1, k1, a1, b1, sa1, sb1 = oracle.make_config_inputs("cfg1")
            t0 = time.perf_counter()
            oracle.ref_gemm(a1, b1, sa1, sb1, m1, n1, k1, nthreads=1)
            dt1 = time.perf_counter() - t0
            cpu["single_thread_cfg1"] = {"seconds": round(dt1, 3),
                                         "gflops": round(2.0 * m1 * n1 * k1 / dt1 * 1e-9, 2)}

    value = flops / (wall_ms * 1e-3) * 1e-12
    out = {
        "metric": "FP8 TFLOPS (block-scaled GEMM, dense) on the headline shape",
        "value": round(value, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3fn x fp8_e4m3fn -> fp32 -> bf16",
        "data": "synthetic (seeded N(0,1) -> bf16 -> 1x128 / 128x128 fp8 quantisation)",
        "config": {"workload": f"{args.workload}: M={m} N={n} K={k}", "kernel": main_rep["kernel"],
                   "frac_fp8_peak": round(value / PEAK_FP8_TFLOPS, 4)},
        "parity": main_rep["parity"],
        "roofline": roof,
        "cpu_baseline": cpu,
        "geomean_latency_us": round(geomean_us, 2),
        "shapes": shapes,
        "challenge": challenge,
        "quantisers": quantisers,
        "vendor_plain_fp8_gemm": vendor,
        "grouped": grouped,
        "grouped_decode": grouped_decode,
        "decode_rows": decode_rows,
        "host_boundary": host_boundary,
        "device": device,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
