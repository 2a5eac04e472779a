#!/usr/bin/env python3
"""Benchmark of the MI355X kernel backend for RefactorGraph's LLM-operator hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops all|headline] [--no-cpu]

Prints ONE JSON line.  The headline metric is AttentionKVCache decode throughput (algorithmic
GB/s, fp16, N=32, 32 query / 8 kv heads, D=128, cache capacity 4096, per-row history lengths
~U{1024..4095}) with all inputs resident in HBM before the timed region.  A "step" is one
decode call (cache append + attention for the whole batch).  The same line carries
  roofline      the decode call against the 8 TB/s HBM peak,
  cpu_baseline  the CPU oracle (a C restatement of the reference's CPU kernels) timed on a
                bounded sample of the same workload on this host,
  ops           the other hot-path kernels at their full-size configurations, each with its own
                roofline entry (MatMulInteger against the 5.0 POP/s dense int8 MFMA peak),
  ceilings      what plain read / write / copy streams and a register-only loop of int8 matrix
                products sustain in the same run (probes of librg_probe.so, a bench-only library),
  targets       (last key) fraction of peak and microseconds per launch of the seven target rows;
                the MatMulInteger half of the metric is also kept under roofline.matmul_integer.
One GPU only: --gpus N with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0        # MI355X dense int8 MFMA, published
FP16_PEAK_TFLOPS = 2500.0      # MI355X dense fp16 MFMA, published
FP32_PEAK_TFLOPS = 157.3       # MI355X fp32 MFMA, published

# HBM-side bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE, one run each,
# KiB per dispatch) on the workloads below and scaled by what the same counters read for a plain
# 256 MiB device copy in the same run (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000).  They are
# properties of the kernels at these shapes, not of a particular run; the counter summaries are
# kept in profiles/.
TRAFFIC_SOURCE = ("profiles/hbm_traffic_pmc.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this bench; "
                  "a constant of the kernel at this shape, not a measurement of the run that prints it")
MEASURED_TRAFFIC = {
    "decode": (2 * 172515 + 2309) * 1024,
    "rms_norm": (2 * 32867 + 65619) * 1024,
    "softmax": (2 * 1048617 + 2097156) * 1024,
    "softmax_causal": (2 * 540713 + 2097158) * 1024,
    "rope": (2 * 131646 + 262167) * 1024,
    "dequantize_linear": (2 * 8292 + 65569) * 1024,
    "matmul_integer": (2 * 50313 + 65560) * 1024,
    "attention_prefill": (2 * 110058 + 196608) * 1024,
    "cast": (2 * 32784 + 32768) * 1024,
    "matmul": (2 * 98778 + 33024) * 1024,
    "matmul_few_rows": (2 * 17456 + 256) * 1024,
    "matmul_eight_rows": (2 * 16661 + 64) * 1024,
    "dequantize_linear_i32": (2 * 32869 + 65611) * 1024,
    "transpose": (2 * 65552 + 131217) * 1024,
    "matmul_integer_dequantize": (2 * 50363 + 65581) * 1024,
    "rms_norm_quantize": (2 * 32883 + 65568 + 2 * 32889 + 16384) * 1024,
    "matmul_integer_few_rows": (2 * 8761 + 8192 + 2 * 10 + 512) * 1024,
    "matmul_one_row": (2 * 16444 + 8) * 1024,
    "matmul_one_row_kn": (2 * 16630 + 273) * 1024,
    "matmul_four_rows_kn": (2 * 17236 + 1065) * 1024,
    "matmul_f32_one_row": (2 * 35255 + 16) * 1024,
    "matmul_few_rows_kn": (2 * 18505 + 4362) * 1024,
    "matmul_integer_one_row": (2 * 8242 + 512 + 2 * 10 + 16) * 1024,
    "dynamic_quantize_linear": (2 * 32798 + 32 + 2 * 32889 + 16384) * 1024,
    "softmax_long_rows": (2 * 32828 + 65602) * 1024,
    "split": (2 * 49176 + 98312) * 1024,
    "concat": (2 * 49181 + 98318) * 1024,
    "where": (2 * 524433 + 1048576) * 1024,
    "expand": (2 * 118 + 262162) * 1024,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=4000)
    ap.add_argument("--ops", default="all", choices=["all", "headline"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the plain read / write / copy streams")
    ap.add_argument("--only", default="", help="comma-separated op names to run besides the headline")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also launch one plain device copy of 256 MiB (a reference point for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters into bytes)")
    ap.add_argument("--calibrate", action="store_true",
                    help="print the issue and copy-rate probes of librg_probe.so (shader clocks per matrix product with "
                         "other instructions behind it; bytes per clock a CU takes from L2) as one JSON line, and exit")
    return ap.parse_args()


class ClockSampler:
    """Samples the shader clock the driver reports (the starred level of pp_dpm_sclk) from a thread
    while a timed region runs; `result()` gives None when the file cannot be read."""

    def __init__(self, period=0.002):
        import glob
        import threading
        paths = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.path = paths[0] if paths else None
        self.period, self.samples, self._stop = period, [], threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _read(self):
        try:
            for line in open(self.path):
                if line.rstrip().endswith("*"):
                    return int(line.split(":")[1].strip().split("M")[0])
        except (OSError, ValueError, IndexError, TypeError):
            pass
        return None

    def _run(self):
        while not self._stop.is_set():
            v = self._read()
            if v is not None:
                self.samples.append(v)
            self._stop.wait(self.period)

    def __enter__(self):
        if self.path:
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self.path:
            self._thread.join()

    def result(self):
        if not self.samples:
            return None
        v = sorted(self.samples)
        return {"median": v[len(v) // 2], "min": v[0], "max": v[-1], "samples": len(v),
                "source": "pp_dpm_sclk sampled during the timed region"}


LAST = {"clock": None, "warmup_ms": None, "warmup_steps": None}   # of the most recent time_steps() call
MIN_WARMUP_S = 0.5    # the GPU leaves its idle clocks only after a few hundred ms of load
CPU_THREADS = min(os.cpu_count() or 1, 16)   # host cores used by the all-cores CPU rows


def time_steps(torch, fn, steps, warmup, n_sets):
    """Times exactly `steps` calls fn(i % n_sets) after at least `warmup` untimed ones and at least
    MIN_WARMUP_S seconds of untimed load (whichever is longer; the time spent is reported as warmup_ms).

    The calls are captured into a HIP graph of `chunk` steps (chunk divides `steps`; plain kernel
    launches on the capture stream) that is replayed steps/chunk times, so the device sees the
    launches back to back and host launch overhead does not enter.  Warm-up replays the same
    graph: the GPU leaves its idle clocks only after a few hundred milliseconds of load, so a
    short warm-up would time the clock ramp, not the kernel.  Two measurements of exactly `steps`
    steps each follow: the wall clock between two device synchronisations, and HIP events on the
    replay stream around replays that follow an untimed one without a gap.  A replay costs a few
    microseconds between its last kernel and the next replay's first one; with fewer than 100 steps
    the events therefore surround a graph that holds the step sequence several times over (at least
    100 launches), so that this gap weighs on a launch as little as it does in a long run.
    Returns (wall ms per step, device ms per step, "graph" | "eager")."""
    steps = max(int(steps), 1)
    chunk = max(d for d in range(1, min(steps, 100) + 1) if steps % d == 0)
    for i in range(min(warmup, 3)):
        fn(i % n_sets)
    torch.cuda.synchronize()
    mode = "graph"
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(chunk):
                fn(i % n_sets)
        run = graph.replay
        run()                      # graph upload
    except Exception as exc:       # capture unavailable: time eager launches instead
        sys.stderr.write(f"bench.py: graph capture failed ({exc}); timing eager launches\n")
        mode = "eager"

        def run():
            for i in range(chunk):
                fn(i % n_sets)
    # warm-up: at least `warmup` steps AND at least MIN_WARMUP_S of back-to-back replays
    t_w = time.perf_counter()
    done = 0
    while done < warmup or time.perf_counter() - t_w < MIN_WARMUP_S:
        for _ in range(4):
            run()
        done += 4 * chunk
        torch.cuda.synchronize()
    LAST["warmup_ms"] = round((time.perf_counter() - t_w) * 1e3, 1)
    LAST["warmup_steps"] = done
    # (a) wall clock around exactly `steps` steps, device idle and synchronised on both sides: this is what
    #     `value` and `ms_per_step` report; it includes the latency of the first launch into an idle queue
    t0 = time.perf_counter()
    for _ in range(steps // chunk):
        run()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # (b) device time of exactly `steps` steps from HIP events on the launch stream.  The timed replays are
    #     queued directly behind one untimed replay, so the events see the kernels back to back, as a
    #     profiler's per-kernel durations do, and not the start-up of a queue that had run dry.
    run_b, reps_b, per_b = run, steps // chunk, chunk
    if mode == "graph" and steps < 100:
        times = -(-100 // steps)                      # whole repetitions of the step sequence
        try:
            graph_b = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph_b):
                for _ in range(times):
                    for i in range(steps):
                        fn(i % n_sets)
            run_b, reps_b, per_b = graph_b.replay, 1, times * steps
            run_b()
        except Exception as exc:
            sys.stderr.write(f"bench.py: second capture failed ({exc}); device time from the short graph\n")
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with ClockSampler() as clock:
        run_b()
        start.record()
        for _ in range(reps_b):
            run_b()
        stop.record()
        torch.cuda.synchronize()
    LAST["clock"] = clock.result()
    dev_ms = start.elapsed_time(stop) / (reps_b * per_b)
    return wall_ms, dev_ms, mode


_POOL = []
_PROBES = []


def probes():
    """librg_probe.so: the benchmark's own measurement aids (ceilings), not part of the boundary library."""
    if not _PROBES:
        import ctypes as C
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "refactorgraph_amd", "lib", "librg_probe.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run `python -m refactorgraph_amd.build`")
        lib = C.CDLL(path)
        vp, sz = C.c_void_p, C.c_size_t
        for name, args in (("rg_probe_mfma_i8", [vp, vp, sz, sz, vp]), ("rg_probe_hbm_read", [vp, vp, sz, sz, vp]),
                           ("rg_probe_hbm_write", [vp, sz, sz, vp]), ("rg_probe_hbm_copy", [vp, vp, sz, sz, vp]),
                           ("rg_probe_issue_shadow", [vp, C.c_int, C.c_int, sz, sz, vp]),
                           ("rg_probe_copy_rate", [vp, vp, C.c_int, sz, sz, sz, sz, vp])):
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = C.c_int, args
        _PROBES.append(lib)
    return _PROBES[0]


def pooled(fn_piece, pieces):
    """Returns a callable that runs fn_piece(piece) for every piece on CPU_THREADS host threads (the oracle's C
    functions are called through ctypes, which releases the interpreter lock, as numpy's conversions do)."""
    if not _POOL:
        from concurrent.futures import ThreadPoolExecutor
        _POOL.append(ThreadPoolExecutor(CPU_THREADS))
    return lambda: list(_POOL[0].map(fn_piece, pieces))


def calibrate(torch):
    """The probes behind the issue budgets that the matrix kernels are written to: clocks per
    v_mfma_i32_32x32x32_i8 (32 when nothing delays it) with `count` instructions of one kind issued behind every
    product by a wavefront alone on its SIMD, and the bytes per clock one CU takes from L2."""
    pr = probes()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.zeros(8192, dtype=torch.int64, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    kinds = ["v_xor_b32", "s_nop", "ds_read_b128", "s_add_u32 (dependent)", "v_exp_f32", "v_cvt_pk_f16_f32",
             "v_dot2c_f32_f16", "v_max3_f32", "v_fma_f32", "ds_read_b64_tr_b16"]
    shadow = {}
    iters = 64
    for kind, name in enumerate(kinds):
        row = {}
        for count in (0, 1, 2, 3, 4, 6, 8, 12):
            for _ in range(2):
                rc = pr.rg_probe_issue_shadow(out.data_ptr(), kind, count, cus, iters, st)
                if rc != 0:
                    raise RuntimeError(f"rg_probe_issue_shadow -> {rc}")
                torch.cuda.synchronize()
            row[str(count)] = round(out[:cus].double().mean().item() / (iters * 16), 1)
        shadow[name] = row
    src = torch.zeros(32 << 20, dtype=torch.uint8, device="cuda")
    copy = {}
    iters = 256
    for to_lds in (1, 0):
        for waves in (4, 8):
            for depth in (4, 8, 16, 32):
                for _ in range(2):
                    rc = pr.rg_probe_copy_rate(out.data_ptr(), src.data_ptr(), to_lds, waves, depth, cus, iters, st)
                    if rc != 0:
                        raise RuntimeError(f"rg_probe_copy_rate -> {rc}")
                    torch.cuda.synchronize()
                clocks = out[:cus].double().mean().item()
                copy[f"{'lds' if to_lds else 'regs'}_{waves}w_x{depth}"] = round(iters * depth * waves * 1024 / clocks, 1)
    return {"clocks_per_mfma_i8_32x32x32_with_n_behind_it": shadow, "l2_bytes_per_clock_per_cu": copy,
            "note": "zero operands and a constant source: the clock stays up, clocks are what is measured; "
                    "key of the copy table: destination, wavefronts, 1 KiB transfers in flight per wavefront"}


CEILINGS = {}   # hbm_read / hbm_write / hbm_copy entries of this run (filled before the first operator)


def hbm_entry(bytes_per_call, dev_ms, traffic_key=None, write_share=None):
    """write_share: written bytes over all algorithmic bytes.  With it the row also states `frac_of_ceiling`: its
    rate over what plain streams with the same mix reach in this run (the read part at the read stream's rate
    plus the written part at the write stream's)."""
    gbs = bytes_per_call / (dev_ms * 1e-3) / 1e9
    e = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get(traffic_key),
         "traffic_source": TRAFFIC_SOURCE if traffic_key in MEASURED_TRAFFIC else None,
         "warmup_ms": LAST["warmup_ms"], "warmup_steps": LAST["warmup_steps"]}
    if write_share is not None and "hbm_read" in CEILINGS:
        r, w = CEILINGS["hbm_read"]["achieved"], CEILINGS["hbm_write"]["achieved"]
        mixed = 1.0 / ((1.0 - write_share) / r + write_share / w)
        e["ceiling_gbs"] = round(mixed, 1)
        e["frac_of_ceiling"] = round(gbs / mixed, 4)
    return e


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the path shards without exchange; "
              "no multi-GPU figure is produced). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from refactorgraph_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = "cuda"
    torch.cuda.set_device(0)
    only = set(filter(None, args.only.split(",")))

    def want(name):
        return args.ops == "all" and (not only or name in only)

    if args.calibrate:
        print(json.dumps(calibrate(torch)))
        return

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------ HBM ceilings of this part, this run
    # Plain streams of 128-bit non-temporal accesses over 1 GiB (four times the memory-side cache): what a kernel
    # that only reads, only writes or copies reaches here.  Every HBM row below states its rate against the stream
    # that matches its mix of reads and writes (`frac_of_ceiling`), beside `frac` against the published 8 TB/s.
    ceilings = CEILINGS
    if args.ops == "all" and not args.no_ceilings:
        pr = probes()
        big = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(5)
        big2 = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        sink = torch.zeros(4, dtype=torch.uint8, device=dev)
        cus = torch.cuda.get_device_properties(0).multi_processor_count

        def stream_of(kind, groups):
            st = lambda: torch.cuda.current_stream().cuda_stream
            if kind == "read":
                return lambda i: pr.rg_probe_hbm_read(sink.data_ptr(), big.data_ptr(), 1 << 30, groups, st()), 1 << 30
            if kind == "write":
                return lambda i: pr.rg_probe_hbm_write(big2.data_ptr(), 1 << 30, groups, st()), 1 << 30
            return lambda i: pr.rg_probe_hbm_copy(big2.data_ptr(), big.data_ptr(), 1 << 30, groups, st()), 2 << 30

        for kind in ("read", "write", "copy"):
            best = None
            for groups in (0, cus * 8):
                fn, nbytes = stream_of(kind, groups)
                wall, dms, mode = time_steps(torch, fn, max(args.steps // 20, 20), 3, 1)
                gbs = nbytes / (dms * 1e-3) / 1e9
                if best is None or gbs > best["achieved"]:
                    best = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": round(gbs / HBM_PEAK_GBS, 4), "device_ms_per_launch": round(dms, 5),
                            "workload": f"plain {kind} stream over 1 GiB ({'one workgroup per 32 KiB' if groups == 0 else str(groups) + ' workgroups, grid stride'})"}
            ceilings[f"hbm_{kind}"] = best
        del big, big2

    # ------------------------------------------------------------ headline: decode
    N, H, Hkv, D, cap = 32, 32, 8, 128, 4096
    scale = 1.0 / math.sqrt(D)
    past_np = np.random.default_rng(14).integers(1024, 4096, N).astype(np.int64)
    sum_past = int(past_np.sum())
    decode_bytes = 4096 * sum_past + 786432  # K,V history read + new rows read/written + Q read + O write
    n_sets = 2                                # 2 x 537 MB of caches: nothing survives in the 256 MB MALL
    gen = torch.Generator(device=dev)

    def randn16(shape, seed):
        gen.manual_seed(seed)
        return torch.randn(shape, generator=gen, device=dev, dtype=torch.float32).half()

    sets = []
    for s in range(n_sets):
        sets.append(dict(
            q=randn16((N, H, 1, D), 9 + 100 * s), k=randn16((N, Hkv, 1, D), 10 + 100 * s),
            v=randn16((N, Hkv, 1, D), 11 + 100 * s), kc=randn16((N, Hkv, cap, D), 12 + 100 * s),
            vc=randn16((N, Hkv, cap, D), 13 + 100 * s), o=torch.empty((N, H, 1, D), device=dev, dtype=torch.float16)))
    past = torch.from_numpy(past_np).to(dev)
    ws = ops.attention_workspace(N, H, Hkv, 1, cap, D, dev)
    state = ops.attention_state(dev)   # persistent ticket counters: the call is a single launch

    def decode(i):
        t = sets[i]
        ops.attention_kvcache(t["q"], t["k"], t["v"], t["kc"], t["vc"], past, scale, out=t["o"], workspace=ws,
                              sync_state=state)

    wall_ms, dev_ms, mode = time_steps(torch, decode, args.steps, args.warmup, n_sets)
    value = decode_bytes / (wall_ms * 1e-3) / 1e9
    roofline = hbm_entry(decode_bytes, dev_ms, "decode", 0.002)
    roofline["kernel"] = "attn_split (one rg_hip_attention_kvcache call = one launch)"
    roofline["algorithmic_bytes"] = decode_bytes
    roofline["device_ms_per_launch"] = round(dev_ms, 5)
    roofline["timing"] = mode
    roofline["observed_sclk_mhz"] = LAST["clock"]

    result = {
        "metric": "AttentionKVCache decode GB/s (% HBM peak); MatMulInteger int8 TOPS (% MFMA)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "AttentionKVCache decode fp16 N=32 H=32 Hkv=8 D=128 cap=4096 "
                               "past~U{1024..4095} (seed 14), scale 1/sqrt(128)",
                   "sum_past": sum_past, "cache_sets_rotated": n_sets},
        "roofline": roofline,
    }

    # ------------------------------------------------------------ CPU baseline (bounded sample)
    if not args.no_cpu:
        import oracle
        t = sets[0]
        rows = [0, 1]                       # two batch rows, all 32 heads each
        f = lambda x: x.float().cpu().numpy()
        q, kc, vc = f(t["q"][rows]), f(t["kc"][rows]), f(t["vc"][rows])
        k, v = f(t["k"][rows]), f(t["v"][rows])
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 10.0:
            oracle.attention_kvcache(q, k, v, kc, vc, past_np[rows], scale)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        sample_bytes = 4096 * int(past_np[rows].sum()) + 786432 * len(rows) // N
        result["cpu_baseline"] = {
            "value": round(sample_bytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"batch rows {rows} of the same workload (all 32 heads, {reps} repetitions, "
                      f"{cpu_s * 1e3:.1f} ms each); composed MatMul/scale/softmax/MatMul oracle in fp32"}

        # the same arithmetic with the batch rows dealt to all host cores (one row per thread)
        rows_all = list(range(min(CPU_THREADS, N)))
        per_row = [(f(t["q"][r:r + 1]), f(t["k"][r:r + 1]), f(t["v"][r:r + 1]), f(t["kc"][r:r + 1]), f(t["vc"][r:r + 1]),
                    past_np[r:r + 1]) for r in rows_all]
        run_all = pooled(lambda a: oracle.attention_kvcache(a[0], a[1], a[2], a[3], a[4], a[5], scale), per_row)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 5.0:
            run_all()
            reps += 1
        all_s = (time.perf_counter() - t0) / reps
        all_bytes = 4096 * int(past_np[rows_all].sum()) + 786432 * len(rows_all) // N
        result["cpu_baseline_all_cores"] = {
            "value": round(all_bytes / all_s / 1e9, 3), "unit": "GB/s", "cores": CPU_THREADS, "kind": "port",
            "sample": f"batch rows {rows_all[0]}..{rows_all[-1]} of the same workload, one row per thread "
                      f"({reps} repetitions, {all_s * 1e3:.1f} ms each)"}
        del per_row

    # ------------------------------------------------------------ the other hot-path kernels
    ops_out = {}
    steps, warmup = args.steps, args.warmup

    def cpu_all(fn, algorithmic_bytes, sample, unit="GB/s", per=1e9):
        """The all-cores row: `fn` runs the same arithmetic as the one-core leg with its rows split over
        CPU_THREADS host threads (the oracle's own `threads=` argument, or pieces dealt to a thread pool)."""
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= 1.0:
                break
        return {"value": round(algorithmic_bytes * reps / dt / per, 5), "unit": unit, "cores": CPU_THREADS, "kind": "port",
                "sample": f"{sample} ({reps} repetitions, {dt / reps * 1e3:.1f} ms each)"}

    def cpu_leg(fn, algorithmic_bytes, sample):
        """Times the oracle on a bounded sample for about a second; the rate is quoted in the algorithmic bytes
        of that sample so that it compares with `achieved`."""
        fn()  # page in
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= 1.0:
                break
        return {"value": round(algorithmic_bytes * reps / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{sample} ({reps} repetitions, {dt / reps * 1e3:.1f} ms each)"}

    if want("rms_norm"):
        nb = 5  # 5 x (134 MB in + 134 MB out): beyond the 256 MB MALL
        xs = [torch.randn((32, 128, 4096), device=dev) for _ in range(nb)]
        ys = [torch.empty_like(xs[0]) for _ in range(nb)]
        w = torch.rand(4096, device=dev) + 0.5
        wall, dms, mode = time_steps(torch, lambda i: ops.rms_norm(xs[i], w, 1e-5, out=ys[i]), steps, warmup, nb)
        e = hbm_entry(134234112, dms, "rms_norm", 0.5)
        e.update(workload="RmsNormalization f32 [32,128,4096]", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn, wn = xs[0][:4].cpu().numpy(), w.cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.rms_norm(xn, wn, 1e-5), 134234112 // 8, "4 of the 32 [128,4096] slabs")
            xa = xs[0][:CPU_THREADS].cpu().numpy()
            e["cpu_baseline_all_cores"] = cpu_all(lambda: oracle.rms_norm(xa, wn, 1e-5, threads=CPU_THREADS),
                                                  134234112 * len(xa) // 32, f"{len(xa)} of the 32 [128,4096] slabs")
        ops_out["rms_norm"] = e
        del xs, ys

    if want("softmax"):
        x = (3 * torch.randn((8, 32, 2048, 2048), device=dev)).half()
        y = torch.empty_like(x)
        for causal, nbytes, name in ((False, 4294967296, "softmax"), (True, 3221749760, "softmax_causal")):
            wall, dms, mode = time_steps(torch, lambda i: ops.softmax(x, causal=causal, out=y), max(steps // 4, 10), max(warmup // 8, 3), 1)
            e = hbm_entry(nbytes, dms, name, 2147483648 / nbytes)
            e.update(workload=f"Softmax fp16 [8,32,2048,2048] causal={causal}", device_ms_per_launch=round(dms, 5), timing=mode)
            if not args.no_cpu:
                import oracle
                xn = x[0, :2].float().cpu().numpy()
                fn = (lambda: oracle.softmax_causal(xn)) if causal else (lambda: oracle.softmax(xn))
                e["cpu_baseline"] = cpu_leg(fn, nbytes // 128, "2 of the 256 [2048,2048] matrices, fp32 on up-cast input")
                n_all = min(CPU_THREADS, 32)
                xa = x[0, :n_all].float().cpu().numpy()
                fa = (lambda: oracle.softmax_causal(xa, threads=CPU_THREADS)) if causal else \
                     (lambda: oracle.softmax(xa, threads=CPU_THREADS))
                e["cpu_baseline_all_cores"] = cpu_all(fa, nbytes * n_all // 256, f"{n_all} of the 256 [2048,2048] matrices")
            ops_out[name] = e
        # the causal mask as data (strict upper triangle = -inf) through the plain kernel: full traffic
        x.masked_fill_(torch.ones((2048, 2048), device=dev, dtype=torch.bool).triu(1), float("-inf"))
        wall, dms, mode = time_steps(torch, lambda i: ops.softmax(x, causal=False, out=y), max(steps // 4, 10), max(warmup // 8, 3), 1)
        e = hbm_entry(4294967296, dms, "softmax", 0.5)
        e.update(workload="Softmax fp16 [8,32,2048,2048], causal mask in the data (-inf above the diagonal), plain kernel",
                 device_ms_per_launch=round(dms, 5), timing=mode)
        ops_out["softmax_causal_data_masked"] = e
        del x, y

    if want("softmax_long_rows"):
        # the scores of one decode step over a long context: [32 x 32 heads, 1, 32768] fp16, 64 KiB a row
        nb = 6  # 6 x 134 MB
        xs = [(3 * torch.randn((1024, 32768), device=dev)).half() for _ in range(nb)]
        ys = [torch.empty_like(xs[0]) for _ in range(nb)]
        wall, dms, mode = time_steps(torch, lambda i: ops.softmax(xs[i], out=ys[i]), steps, warmup, nb)
        sl_bytes = 2 * 1024 * 32768 * 2
        e = hbm_entry(sl_bytes, dms, "softmax_long_rows", 0.5)
        e.update(workload="Softmax fp16 [1024,32768] (one workgroup per row, row kept in LDS between the two sweeps)",
                 device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn = xs[0][:64].float().cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.softmax(xn), sl_bytes // 16, "64 of the 1024 rows, fp32 on up-cast input")
        ops_out["softmax_long_rows"] = e
        del xs, ys

    if want("rope"):
        nb = 2
        xs = [torch.randn((16, 2048, 32, 128), device=dev).half() for _ in range(nb)]
        ys = [torch.empty_like(xs[0]) for _ in range(nb)]
        pos = torch.arange(2048, device=dev, dtype=torch.int64).repeat(16, 1).contiguous()
        wall, dms, mode = time_steps(torch, lambda i: ops.rope(xs[i], pos, 10000.0, out=ys[i]), steps, warmup, nb)
        e = hbm_entry(537133056, dms, "rope", 0.5)
        e.update(workload="RotaryEmbedding fp16 [16,2048,32,128]", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn, pn = xs[0][:1].float().cpu().numpy(), pos[:1].cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.rope(xn, pn, 10000.0), 537133056 // 16,
                                        "batch row 0 of 16, fp32 on up-cast input")
            e["cpu_baseline_all_cores"] = cpu_all(lambda: oracle.rope(xn, pn, 10000.0, threads=CPU_THREADS), 537133056 // 16,
                                                  "batch row 0 of 16")
        ops_out["rope"] = e
        del xs, ys

    if want("dequantize_linear"):
        nb = 8  # 8 x 84 MB
        xs = [torch.randint(-128, 128, (4096, 4096), device=dev, dtype=torch.int8) for _ in range(nb)]
        ys = [torch.empty((4096, 4096), device=dev) for _ in range(nb)]
        sc = torch.rand(4096, device=dev) * 9e-3 + 1e-3
        wall, dms, mode = time_steps(torch, lambda i: ops.dequantize_linear(xs[i], sc, axis=1, out=ys[i]), steps, warmup, nb)
        e = hbm_entry(83902464, dms, "dequantize_linear", 0.8)
        e.update(workload="DequantizeLinear i8->f32 [4096,4096] per-axis scale", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn, sn = xs[0].cpu().numpy(), sc.cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.dequantize_linear(xn, sn, axis=1), 83902464, "the whole tensor once")
            e["cpu_baseline_all_cores"] = cpu_all(lambda: oracle.dequantize_linear(xn, sn, axis=1, threads=CPU_THREADS), 83902464,
                                                  "the whole tensor once")
        ops_out["dequantize_linear"] = e
        del xs, ys

    if want("dequantize_linear_i32"):
        # the same operator on the int32 sums of a MatMulInteger (the quantised layer without the fused epilogue)
        nb = 4  # 4 x 134 MB
        xs = [torch.randint(-(1 << 20), 1 << 20, (4096, 4096), device=dev, dtype=torch.int32) for _ in range(nb)]
        ys = [torch.empty((4096, 4096), device=dev, dtype=torch.float32) for _ in range(nb)]
        sc = torch.rand(4096, device=dev) * 9e-3 + 1e-3
        wall, dms, mode = time_steps(torch, lambda i: ops.dequantize_linear(xs[i], sc, axis=1, out=ys[i]), steps, warmup, nb)
        dq_bytes = 4096 * 4096 * 8 + 4096 * 4
        e = hbm_entry(dq_bytes, dms, "dequantize_linear_i32", 0.5)
        e.update(workload="DequantizeLinear i32->f32 [4096,4096] per-axis scale", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn, sn = xs[0].cpu().numpy(), sc.cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.dequantize_linear(xn, sn, axis=1), dq_bytes, "the whole tensor once")
        ops_out["dequantize_linear_i32"] = e
        del xs, ys

    if want("dynamic_quantize_linear"):
        # producer of MatMulInteger's A operand; rotate inputs so that the first pass (min/max)
        # streams from HBM; the second pass re-reads the 67 MB it has just seen
        nb = 8
        xs = [torch.randn((4096, 4096), device=dev) for _ in range(nb)]
        ys = [torch.empty((4096, 4096), device=dev, dtype=torch.uint8) for _ in range(nb)]
        wsq = torch.empty(ops.lib().rg_hip_dynamic_quantize_linear_workspace(4096 * 4096), dtype=torch.uint8, device=dev)
        wall, dms, mode = time_steps(
            torch, lambda i: ops.dynamic_quantize_linear(xs[i], out=ys[i], workspace=wsq), steps, warmup, nb)
        e = hbm_entry(4096 * 4096 * 5 + 5, dms, "dynamic_quantize_linear", 0.2)
        e.update(workload="DynamicQuantizeLinear f32->u8 [4096,4096] (two launches: min/max, quantize); "
                          "algorithmic bytes count x once",
                 device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn = xs[0].cpu().numpy()
            t0 = time.perf_counter()
            oracle.dynamic_quantize_linear(xn)
            dt = time.perf_counter() - t0
            e["cpu_baseline"] = {"value": round(4096 * 4096 * 5 / dt / 1e9, 3), "unit": "GB/s", "cores": 1,
                                 "kind": "port", "sample": f"the whole [4096,4096] tensor once ({dt:.2f} s)"}
        ops_out["dynamic_quantize_linear"] = e
        del xs, ys

    if want("rms_norm_quantize"):
        # the head of a quantised layer: RmsNormalization then DynamicQuantizeLinear of its output, as the fused pair
        # (two launches, the normalised tensor read once) and as the two operators one after the other (three
        # launches, read twice).  Algorithmic bytes of the pair: x in, y out, y in, yq out.
        nb = 4
        xs = [torch.randn((4096, 4096), device=dev) for _ in range(nb)]
        wg = torch.rand(4096, device=dev) + 0.5
        yn = [torch.empty((4096, 4096), device=dev) for _ in range(nb)]
        yq = [torch.empty((4096, 4096), device=dev, dtype=torch.uint8) for _ in range(nb)]
        sc_, zp_ = torch.empty((), device=dev), torch.empty((), device=dev, dtype=torch.uint8)
        L = ops.lib()
        wsf = torch.empty(L.rg_hip_rms_norm_quantize_workspace(4096, 4096), dtype=torch.uint8, device=dev)
        wsq = torch.empty(L.rg_hip_dynamic_quantize_linear_workspace(4096 * 4096), dtype=torch.uint8, device=dev)
        st = lambda: torch.cuda.current_stream().cuda_stream

        def fused(i):
            rc = L.rg_hip_rms_norm_quantize(yq[i].data_ptr(), sc_.data_ptr(), zp_.data_ptr(), yn[i].data_ptr(), xs[i].data_ptr(),
                                            wg.data_ptr(), 4096, 4096, 1e-5, wsf.data_ptr(), wsf.numel(), st())
            assert rc == 0, rc

        def apart(i):
            ops.rms_norm(xs[i], wg, 1e-5, out=yn[i])
            ops.dynamic_quantize_linear(yn[i], out=yq[i], workspace=wsq)

        wall, dms_f, mode = time_steps(torch, fused, steps, warmup, nb)
        wall, dms_a, mode = time_steps(torch, apart, steps, warmup, nb)
        pair_bytes = 4096 * 4096 * (4 + 4 + 4 + 1) + 4096 * 4
        e = hbm_entry(pair_bytes, dms_f, "rms_norm_quantize", (4 + 1) / 13)
        e.update(workload="RmsNormalization f32 [4096,4096] -> DynamicQuantizeLinear, fused pair (2 launches)",
                 device_ms_per_launch=round(dms_f, 5), timing=mode, two_operators_device_ms=round(dms_a, 5),
                 two_operators_gbs=round(pair_bytes / (dms_a * 1e-3) / 1e9, 1))
        ops_out["rms_norm_quantize"] = e
        del xs, yn, yq

    if want("cast"):
        # the Cast either side of the fp16 operators: f32 -> fp16 of an activation tensor (6 B per element)
        nb = 6  # 6 x 100 MB
        xs = [torch.randn((32, 128, 4096), device=dev) for _ in range(nb)]
        ys = [torch.empty((32, 128, 4096), device=dev, dtype=torch.float16) for _ in range(nb)]
        wall, dms, mode = time_steps(torch, lambda i: ops.cast(xs[i], torch.float16, out=ys[i]), steps, warmup, nb)
        cast_bytes = 32 * 128 * 4096 * 6
        e = hbm_entry(cast_bytes, dms, "cast", 1 / 3)
        e.update(workload="Cast f32->fp16 [32,128,4096]", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn = xs[0].cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.cast(xn, "f32", "fp16"), cast_bytes, "the whole tensor once")
            e["cpu_baseline_all_cores"] = cpu_all(pooled(lambda piece: oracle.cast(piece, "f32", "fp16"), list(xn)), cast_bytes,
                                                  "the whole tensor once, the 32 slabs dealt to the threads")
        ops_out["cast"] = e
        del xs, ys

    if want("transpose"):
        # heads and sequence swap between a projection's output and attention: [32, 512, 32, 128] fp16
        nb = 3  # 3 x 268 MB
        xs = [torch.randn((32, 512, 32, 128), device=dev).half() for _ in range(nb)]
        ys = [torch.empty((32, 32, 512, 128), device=dev, dtype=torch.float16) for _ in range(nb)]
        wall, dms, mode = time_steps(torch, lambda i: ops.transpose(xs[i], (0, 2, 1, 3), out=ys[i]), steps, warmup, nb)
        tr_bytes = 2 * 32 * 512 * 32 * 128 * 2
        e = hbm_entry(tr_bytes, dms, "transpose", 0.5)
        e.update(workload="Transpose fp16 [32,512,32,128] perm (0,2,1,3)", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn = xs[0][:4].cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.transpose(xn, (0, 2, 1, 3)), tr_bytes // 8, "4 of the 32 batch rows")
            xa = xs[0][:CPU_THREADS].cpu().numpy()
            e["cpu_baseline_all_cores"] = cpu_all(
                pooled(lambda piece: oracle.transpose(piece, (0, 2, 1, 3)), [xa[i:i + 1] for i in range(len(xa))]),
                tr_bytes * len(xa) // 32, f"{len(xa)} of the 32 batch rows, one per thread")
        ops_out["transpose"] = e
        del xs, ys

    if want("split") or want("concat"):
        # a fused QKV projection's output taken apart (and put together again): [4096, 12288] fp16 <-> 3 x [4096, 4096];
        # every byte is read once and written once
        nb = 3  # 3 x 201 MB
        xs = [torch.randn((4096, 12288), device=dev).half() for _ in range(nb)]
        parts = [[torch.empty((4096, 4096), device=dev, dtype=torch.float16) for _ in range(3)] for _ in range(nb)]
        mv_bytes = 2 * 4096 * 12288 * 2
        if not args.no_cpu:
            import oracle
            xn = xs[0][:512].cpu().numpy()
            pn = oracle.split(xn, [4096] * 3, 1)
        if want("split"):
            wall, dms, mode = time_steps(torch, lambda i: ops.split(xs[i], [4096] * 3, 1, outs=parts[i]), steps, warmup, nb)
            e = hbm_entry(mv_bytes, dms, "split", 0.5)
            e.update(workload="Split fp16 [4096,12288] -> 3 x [4096,4096] along the last axis",
                     device_ms_per_launch=round(dms, 5), timing=mode)
            if not args.no_cpu:
                e["cpu_baseline"] = cpu_leg(lambda: oracle.split(xn, [4096] * 3, 1), mv_bytes // 8, "512 of the 4096 rows")
            ops_out["split"] = e
        if want("concat"):
            wall, dms, mode = time_steps(torch, lambda i: ops.concat(parts[i], 1, out=xs[i]), steps, warmup, nb)
            e = hbm_entry(mv_bytes, dms, "concat", 0.5)
            e.update(workload="Concat fp16 3 x [4096,4096] -> [4096,12288] along the last axis",
                     device_ms_per_launch=round(dms, 5), timing=mode)
            if not args.no_cpu:
                e["cpu_baseline"] = cpu_leg(lambda: oracle.concat(pn, 1), mv_bytes // 8, "512 of the 4096 rows")
            ops_out["concat"] = e
        del xs, parts

    if want("where"):
        # a mask applied to attention scores: c bool [512, 512] broadcast over [32, 32, 512, 512] f32 x, scalar y
        nb = 3
        c = torch.ones((512, 512), device=dev).tril().bool()
        xs = [torch.randn((32, 32, 512, 512), device=dev) for _ in range(nb)]
        ys = [torch.empty_like(xs[0]) for _ in range(nb)]
        fill = torch.full((1,), -1e9, device=dev)
        wall, dms, mode = time_steps(torch, lambda i: ops.where(c, xs[i], fill, out=ys[i]), steps, warmup, nb)
        wh_bytes = 32 * 32 * 512 * 512 * 8 + 512 * 512 + 4
        e = hbm_entry(wh_bytes, dms, "where", 0.5)
        e.update(workload="Where bool [512,512], f32 [32,32,512,512], f32 [1] -> f32 [32,32,512,512]",
                 device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            cn, xn, fn = c.cpu().numpy(), xs[0][:1, :4].cpu().numpy(), fill.cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.where(cn, xn, fn), wh_bytes // 256, "4 of the 1024 [512,512] slabs")
        ops_out["where"] = e
        del xs, ys

    if want("expand"):
        # a bias row laid out over a batch of activations: fp16 [1, 4096] -> [32768, 4096]; only the output is traffic
        y = torch.empty((32768, 4096), device=dev, dtype=torch.float16)
        x = torch.randn((1, 4096), device=dev).half()
        wall, dms, mode = time_steps(torch, lambda i: ops.expand(x, (32768, 4096), out=y), steps, warmup, 1)
        ex_bytes = 32768 * 4096 * 2 + 4096 * 2
        e = hbm_entry(ex_bytes, dms, "expand", 1.0)
        e.update(workload="Expand fp16 [1,4096] -> [32768,4096]", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            xn = x.cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.expand(xn, (4096, 4096)), ex_bytes // 8, "4096 of the 32768 rows")
        ops_out["expand"] = e
        del x, y

    if any(want(nm) for nm in ("matmul_integer", "matmul_integer_dequantize", "matmul_integer_few_rows", "matmul_integer_one_row",
                               "matmul_integer_zero_operands", "matmul_integer_small_operands", "matmul_integer_8192",
                               "matmul_integer_mfma_ceiling")):
        a = torch.randint(0, 256, (4096, 4096), device=dev, dtype=torch.uint8)
        b = torch.randint(-128, 128, (4096, 4096), device=dev, dtype=torch.int8)
        az = torch.tensor([128], device=dev, dtype=torch.uint8)
        bz = torch.tensor([0], device=dev, dtype=torch.int8)
        y = torch.empty((4096, 4096), device=dev, dtype=torch.int32)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul_integer(a, b, az, bz, out=y), steps, warmup, 1)
        tops = 2 * 4096 ** 3 / (dms * 1e-3) / 1e12
        ops_out["matmul_integer"] = {
            "bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
            "frac": round(tops / INT8_PEAK_TOPS, 4), "traffic": MEASURED_TRAFFIC["matmul_integer"],
            "traffic_source": TRAFFIC_SOURCE,
            "workload": "MatMulInteger u8 x i8 -> i32 4096^3, a_zp=128 b_zp=0 (uniform random bytes)",
            "device_ms_per_launch": round(dms, 5), "timing": mode, "observed_sclk_mhz": LAST["clock"],
            "warmup_ms": LAST["warmup_ms"], "warmup_steps": LAST["warmup_steps"]}
        if LAST["clock"]:
            # the published peak is quoted at 2400 MHz: the same pipe at the clock the run held
            at_clock = INT8_PEAK_TOPS * LAST["clock"]["median"] / 2400.0
            ops_out["matmul_integer"]["peak_at_observed_clock"] = round(at_clock, 1)
            ops_out["matmul_integer"]["frac_at_observed_clock"] = round(tops / at_clock, 4)
        if not args.no_cpu:
            import oracle
            m = 64
            an, bn = a[:m].cpu().numpy(), b.cpu().numpy()
            t0 = time.perf_counter()
            oracle.matmul_integer(an, bn, np.array([128], np.uint8), np.array([0], np.int8), threads=1)
            dt = time.perf_counter() - t0
            ops_out["matmul_integer"]["cpu_baseline"] = {
                "value": round(2 * m * 4096 * 4096 / dt / 1e12, 5), "unit": "TOP/s", "cores": 1, "kind": "port",
                "sample": f"first {m} rows of A against all of B ({dt:.1f} s)"}
            ma = m * CPU_THREADS
            an = a[:ma].cpu().numpy()
            t0 = time.perf_counter()
            oracle.matmul_integer(an, bn, np.array([128], np.uint8), np.array([0], np.int8), threads=CPU_THREADS)
            dt = time.perf_counter() - t0
            ops_out["matmul_integer"]["cpu_baseline_all_cores"] = {
                "value": round(2 * ma * 4096 * 4096 / dt / 1e12, 5), "unit": "TOP/s", "cores": CPU_THREADS, "kind": "port",
                "sample": f"first {ma} rows of A against all of B, rows split over the threads ({dt:.1f} s)"}
        def mmi_entry(name, workload, aa, bb, yy, ops_count):
            """Further MatMulInteger rows through the same kernel: what the matrix pipe sustains depends on the
            operand values (power) and on how many tiles a CU gets (one tile per CU leaves its write-out bare)."""
            wall, d_ms, md = time_steps(torch, lambda i: ops.matmul_integer(aa, bb, az, bz, out=yy), steps, warmup, 1)
            t_ops = ops_count / (d_ms * 1e-3) / 1e12
            ent = {"bound": "mfma", "achieved": round(t_ops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                   "frac": round(t_ops / INT8_PEAK_TOPS, 4), "traffic": None, "workload": workload,
                   "device_ms_per_launch": round(d_ms, 5), "timing": md, "observed_sclk_mhz": LAST["clock"],
                   "warmup_ms": LAST["warmup_ms"], "warmup_steps": LAST["warmup_steps"]}
            if LAST["clock"]:
                at = INT8_PEAK_TOPS * LAST["clock"]["median"] / 2400.0
                ent["peak_at_observed_clock"] = round(at, 1)
                ent["frac_at_observed_clock"] = round(t_ops / at, 4)
            ops_out[name] = ent

        if want("matmul_integer_zero_operands"):
            a0 = torch.full((4096, 4096), 128, device=dev, dtype=torch.uint8)   # a - a_zp = 0
            b0 = torch.zeros((4096, 4096), device=dev, dtype=torch.int8)
            mmi_entry("matmul_integer_zero_operands", "MatMulInteger 4096^3, every operand byte 0 after the zero point "
                      "(same kernel, same launches: what the operand values cost)", a0, b0, y, 2 * 4096 ** 3)
            del a0, b0
        if want("matmul_integer_small_operands"):
            a0 = torch.randint(121, 136, (4096, 4096), device=dev, dtype=torch.uint8)   # |a - a_zp| < 8
            b0 = torch.randint(-7, 8, (4096, 4096), device=dev, dtype=torch.int8)
            mmi_entry("matmul_integer_small_operands", "MatMulInteger 4096^3, operands uniform in -7..7 after the zero point",
                      a0, b0, y, 2 * 4096 ** 3)
            del a0, b0
        if want("matmul_integer_8192"):
            a0 = torch.randint(0, 256, (8192, 4096), device=dev, dtype=torch.uint8)
            b0 = torch.randint(-128, 128, (4096, 8192), device=dev, dtype=torch.int8)
            y0 = torch.empty((8192, 8192), device=dev, dtype=torch.int32)
            mmi_entry("matmul_integer_8192", "MatMulInteger u8 [8192,4096] x i8 [4096,8192] -> i32 (uniform random bytes; four "
                      "256 x 256 tiles per CU instead of one)", a0, b0, y0, 2 * 8192 * 8192 * 4096)
            del a0, b0, y0
        if want("matmul_integer_mfma_ceiling"):
            # what the matrix pipe itself sustains: the same 4 x 4 blocks of products from registers (no LDS,
            # no copies, no write-out), as many per wavefront as the 4096^3 kernel issues, one workgroup per CU
            cus = torch.cuda.get_device_properties(0).multi_processor_count
            outp = torch.empty(cus * 256, device=dev, dtype=torch.int32)
            for nm, opnd, what in (
                    ("matmul_integer_mfma_ceiling", torch.randint(-128, 128, (8192,), device=dev, dtype=torch.int8),
                     "uniform random operand bytes"),
                    ("matmul_integer_mfma_ceiling_zero", torch.zeros(8192, device=dev, dtype=torch.int8), "all-zero operands")):
                def probe(i, opnd=opnd):
                    rc = probes().rg_probe_mfma_i8(outp.data_ptr(), opnd.data_ptr(), cus, 128,
                                                   torch.cuda.current_stream().cuda_stream)
                    assert rc == 0, rc
                wall, d_ms, md = time_steps(torch, probe, steps, warmup, 1)
                t_ops = cus * 4 * 128 * 16 * 2 * 32 ** 3 / (d_ms * 1e-3) / 1e12
                ent = {"bound": "mfma", "achieved": round(t_ops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                       "frac": round(t_ops / INT8_PEAK_TOPS, 4), "traffic": None,
                       "workload": f"register-only loop of 2048 v_mfma_i32_32x32x32_i8 per wavefront, {cus} workgroups of 4 "
                                   f"wavefronts, {what}: the ceiling of any int8 GEMM on this part for such data",
                       "device_ms_per_launch": round(d_ms, 5), "timing": md, "observed_sclk_mhz": LAST["clock"],
                       "warmup_ms": LAST["warmup_ms"]}
                if LAST["clock"]:
                    at = INT8_PEAK_TOPS * LAST["clock"]["median"] / 2400.0
                    ent["peak_at_observed_clock"] = round(at, 1)
                    ent["frac_at_observed_clock"] = round(t_ops / at, 4)
                ops_out[nm] = ent
        if want("matmul_integer_dequantize"):
            # the same product with DequantizeLinear (per-column scale) folded into the epilogue, against
            # the two operators one after the other
            sc = torch.rand(4096, device=dev) * 9e-3 + 1e-3
            yf = torch.empty((4096, 4096), device=dev, dtype=torch.float32)
            wall, dms_f, mode = time_steps(torch, lambda i: ops.matmul_integer(a, b, az, bz, out=yf, dequant_scale=sc),
                                           steps, warmup, 1)
            wall, dms_2, mode = time_steps(
                torch, lambda i: ops.dequantize_linear(ops.matmul_integer(a, b, az, bz, out=y), sc, None, axis=1, out=yf),
                steps, warmup, 1)
            tops = 2 * 4096 ** 3 / (dms_f * 1e-3) / 1e12
            ops_out["matmul_integer_dequantize"] = {
                "bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                "frac": round(tops / INT8_PEAK_TOPS, 4), "traffic": MEASURED_TRAFFIC["matmul_integer_dequantize"],
                "traffic_source": TRAFFIC_SOURCE,
                "workload": "MatMulInteger 4096^3 with DequantizeLinear (scale per column) in its epilogue -> f32",
                "device_ms_per_launch": round(dms_f, 5), "timing": mode,
                "two_operators_device_ms": round(dms_2, 5), "warmup_ms": LAST["warmup_ms"]}
        if want("matmul_integer_few_rows"):
            # the same weights against 32 rows of activations (a decode step of the quantised layer): bound by reading B
            a32 = a[:32].contiguous()
            y32 = torch.empty((32, 4096), device=dev, dtype=torch.int32)
            wall, dms_s, mode = time_steps(torch, lambda i: ops.matmul_integer(a32, b, az, bz, out=y32), steps, warmup, 1)
            e = hbm_entry(4096 * 4096 + 32 * 4096 + 32 * 4096 * 4, dms_s, "matmul_integer_few_rows", 0.0)
            e.update(workload="MatMulInteger u8 [32,4096] x i8 [4096,4096] -> i32, a_zp=128 b_zp=0 (zeroing launch included)",
                     device_ms_per_launch=round(dms_s, 5), timing=mode)
            ops_out["matmul_integer_few_rows"] = e
        if want("matmul_integer_one_row"):
            # a single sequence's decode step (matrix-vector product); 20 weight matrices in turn: beyond the memory-side cache
            nb = 20
            a1 = a[:1].contiguous()
            bs = [torch.randint(-128, 128, (4096, 4096), device=dev, dtype=torch.int8) for _ in range(nb)]
            y1 = torch.empty((1, 4096), device=dev, dtype=torch.int32)
            wall, dms_s, mode = time_steps(torch, lambda i: ops.matmul_integer(a1, bs[i], az, bz, out=y1), steps, warmup, nb)
            e = hbm_entry(4096 * 4096 + 4096 + 4096 * 4, dms_s, "matmul_integer_one_row", 0.0)
            e.update(workload="MatMulInteger u8 [1,4096] x i8 [4096,4096] -> i32, a_zp=128 b_zp=0 (zeroing launch included)",
                     device_ms_per_launch=round(dms_s, 5), timing=mode)
            ops_out["matmul_integer_one_row"] = e
            del bs
        del a, b, y

    if want("matmul"):
        # a decoder layer's projection at 4096 tokens: activations [4096, 4096] x weights [4096, 4096]^T, fp16
        a = torch.randn((4096, 4096), device=dev).half()
        b = (torch.randn((4096, 4096), device=dev) * 0.05).half()
        y = torch.empty((4096, 4096), device=dev, dtype=torch.float16)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a, b, trans_b=True, out=y), steps, warmup, 1)
        tflops = 2 * 4096 ** 3 / (dms * 1e-3) / 1e12
        ops_out["matmul"] = {
            "bound": "mfma", "achieved": round(tflops, 1), "peak": FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tflops / FP16_PEAK_TFLOPS, 4), "traffic": MEASURED_TRAFFIC.get("matmul"),
            "traffic_source": TRAFFIC_SOURCE,
            "workload": "MatMul fp16 [4096,4096] x [4096,4096]^T (trans_b), alpha 1, no bias",
            "device_ms_per_launch": round(dms, 5), "timing": mode, "observed_sclk_mhz": LAST["clock"],
            "warmup_ms": LAST["warmup_ms"], "warmup_steps": LAST["warmup_steps"]}
        if LAST["clock"]:
            at_clock = FP16_PEAK_TFLOPS * LAST["clock"]["median"] / 2400.0
            ops_out["matmul"]["peak_at_observed_clock"] = round(at_clock, 1)
            ops_out["matmul"]["frac_at_observed_clock"] = round(tflops / at_clock, 4)
        if not args.no_cpu:
            import oracle
            rows = 128
            an, bn = a[:rows].cpu().numpy(), b.cpu().numpy()
            t0 = time.perf_counter()
            oracle.matmul(an, bn, None, False, True, dtype="fp16")
            dt = time.perf_counter() - t0
            ops_out["matmul"]["cpu_baseline"] = {
                "value": round(2 * rows * 4096 * 4096 / dt / 1e12, 5), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                "sample": f"first {rows} rows of A against all of B ({dt:.1f} s), float on the up-cast values"}
            an = a[:rows * CPU_THREADS].cpu().numpy()
            run_all = pooled(lambda piece: oracle.matmul(piece, bn, None, False, True, dtype="fp16"),
                             [an[i * rows:(i + 1) * rows] for i in range(CPU_THREADS)])
            t0 = time.perf_counter()
            run_all()
            dt = time.perf_counter() - t0
            ops_out["matmul"]["cpu_baseline_all_cores"] = {
                "value": round(2 * rows * CPU_THREADS * 4096 * 4096 / dt / 1e12, 5), "unit": "TFLOP/s", "cores": CPU_THREADS,
                "kind": "port", "sample": f"first {rows * CPU_THREADS} rows of A, {rows} per thread ({dt:.1f} s)"}
        del a, b, y

    if want("matmul_f32"):
        # the same products in float, as an f32 graph asks for them: 4096^3 with the weights as ONNX MatMul stores
        # them ([k, n]) on 32x32x2 matrix instructions, and one row of activations (bound by reading the weights once)
        a = torch.randn((4096, 4096), device=dev)
        b = torch.randn((4096, 4096), device=dev) * 0.05
        y = torch.empty((4096, 4096), device=dev)
        f32_steps = max(steps // 10, 1)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a, b, out=y), f32_steps, max(warmup // 10, 1), 1)
        tflops = 2 * 4096 ** 3 / (dms * 1e-3) / 1e12
        ops_out["matmul_f32"] = {
            "bound": "mfma", "achieved": round(tflops, 1), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tflops / FP32_PEAK_TFLOPS, 4), "traffic": (2 * 378527 + 65536) * 1024,
            "traffic_source": TRAFFIC_SOURCE,
            "workload": "MatMul f32 [4096,4096] x [4096,4096] (weights as [k,n]), alpha 1, no bias",
            "device_ms_per_launch": round(dms, 5), "timing": mode, "steps": f32_steps, "observed_sclk_mhz": LAST["clock"],
            "warmup_ms": LAST["warmup_ms"], "warmup_steps": LAST["warmup_steps"]}
        del a, y
        nb = 5  # 5 x 67 MB of weights: beyond the memory-side cache
        a1 = torch.randn((1, 4096), device=dev)
        ws = [b] + [torch.randn((4096, 4096), device=dev) * 0.05 for _ in range(nb - 1)]
        y1 = torch.empty((1, 4096), device=dev)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a1, ws[i], out=y1), steps, warmup, nb)
        e = hbm_entry((4096 * 4096 + 2 * 4096) * 4, dms, "matmul_f32_one_row", 0.0)
        e.update(workload="MatMul f32 [1,4096] x [4096,4096] (weights as [k,n])", device_ms_per_launch=round(dms, 5), timing=mode)
        ops_out["matmul_f32_one_row"] = e
        del a1, ws, y1, b

    if want("matmul_few_rows"):
        # the same projection in a decode step: 32 rows of activations; bound by reading the weights once
        nb = 10  # 10 x 33.5 MB of weights: beyond the memory-side cache
        a = torch.randn((32, 4096), device=dev).half()
        ws = [(torch.randn((4096, 4096), device=dev) * 0.05).half() for _ in range(nb)]
        y = torch.empty((32, 4096), device=dev, dtype=torch.float16)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a, ws[i], trans_b=True, out=y), steps, warmup, nb)
        few_bytes = (4096 * 4096 + 2 * 32 * 4096) * 2
        e = hbm_entry(few_bytes, dms, "matmul_few_rows", 0.0)
        e.update(workload="MatMul fp16 [32,4096] x [4096,4096]^T (trans_b)", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            an, bn = a.cpu().numpy(), ws[0][:512].cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.matmul(an, bn, None, False, True, dtype="fp16"),
                                        (512 * 4096 + 32 * 4096 + 32 * 512) * 2, "512 of the 4096 rows of W")
        ops_out["matmul_few_rows"] = e
        del a, ws, y

    if want("matmul_eight_rows"):
        # eight sequences in the decode step: operands straight from memory into block products, no pass through LDS
        nb = 10
        a = torch.randn((8, 4096), device=dev).half()
        ws = [(torch.randn((4096, 4096), device=dev) * 0.05).half() for _ in range(nb)]
        y = torch.empty((8, 4096), device=dev, dtype=torch.float16)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a, ws[i], trans_b=True, out=y), steps, warmup, nb)
        e = hbm_entry((4096 * 4096 + 2 * 8 * 4096) * 2, dms, "matmul_eight_rows", 0.0)
        e.update(workload="MatMul fp16 [8,4096] x [4096,4096]^T (trans_b)", device_ms_per_launch=round(dms, 5), timing=mode)
        ops_out["matmul_eight_rows"] = e
        del a, ws, y

    if want("matmul_one_row"):
        # the projection of a single sequence's decode step: one row of activations (matrix-vector product)
        nb = 10
        a = torch.randn((1, 4096), device=dev).half()
        ws = [(torch.randn((4096, 4096), device=dev) * 0.05).half() for _ in range(nb)]
        y = torch.empty((1, 4096), device=dev, dtype=torch.float16)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a, ws[i], trans_b=True, out=y), steps, warmup, nb)
        e = hbm_entry((4096 * 4096 + 2 * 4096) * 2, dms, "matmul_one_row", 0.0)
        e.update(workload="MatMul fp16 [1,4096] x [4096,4096]^T (trans_b)", device_ms_per_launch=round(dms, 5), timing=mode)
        if not args.no_cpu:
            import oracle
            an, bn = a.cpu().numpy(), ws[0].cpu().numpy()
            e["cpu_baseline"] = cpu_leg(lambda: oracle.matmul(an, bn, None, False, True, dtype="fp16"),
                                        (4096 * 4096 + 2 * 4096) * 2, "the whole product")
        ops_out["matmul_one_row"] = e
        del a, ws, y

    for name, rows in (("matmul_one_row_kn", 1), ("matmul_four_rows_kn", 4), ("matmul_few_rows_kn", 32)):
        if not want(name):
            continue
        # the same decode projections with the weights as ONNX MatMul keeps them, [k, n]
        nb = 10
        a = torch.randn((rows, 4096), device=dev).half()
        ws = [(torch.randn((4096, 4096), device=dev) * 0.05).half() for _ in range(nb)]
        y = torch.empty((rows, 4096), device=dev, dtype=torch.float16)
        # the workspace that the routine's lowering asks the allocator for (0 bytes where none helps)
        need = ops.lib().rg_hip_matmul_workspace(ops._T2CODE[torch.float16], 0, 0, 1, rows, 4096, 4096)
        wsb = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        wall, dms, mode = time_steps(torch, lambda i: ops.matmul(a, ws[i], out=y, workspace=wsb), steps, warmup, nb)
        e = hbm_entry((4096 * 4096 + 2 * rows * 4096) * 2, dms, name, 0.0)
        e["workspace_bytes"] = need
        e.update(workload=f"MatMul fp16 [{rows},4096] x [4096,4096] (weights as [k,n])", device_ms_per_launch=round(dms, 5),
                 timing=mode)
        if not args.no_cpu:
            import oracle
            an, bn = a.cpu().numpy(), ws[0].cpu().numpy()
            if rows <= 4:
                e["cpu_baseline"] = cpu_leg(lambda: oracle.matmul(an, bn, None, False, False, dtype="fp16"),
                                            (4096 * 4096 + 2 * rows * 4096) * 2, "the whole product")
        ops_out[name] = e
        del a, ws, y

    if want("attention_prefill"):
        Np, seq = 32, 512
        q = torch.randn((Np, H, seq, D), device=dev).half()
        k = torch.randn((Np, Hkv, seq, D), device=dev).half()
        v = torch.randn((Np, Hkv, seq, D), device=dev).half()
        kc = torch.zeros((Np, Hkv, cap, D), device=dev, dtype=torch.float16)
        vc = torch.zeros_like(kc)
        o = torch.empty_like(q)
        zero = torch.zeros(Np, device=dev, dtype=torch.int64)
        wsp = ops.attention_workspace(Np, H, Hkv, seq, cap, D, dev)
        wall, dms, mode = time_steps(
            torch, lambda i: ops.attention_kvcache(q, k, v, kc, vc, zero, scale, out=o, workspace=wsp,
                                                   sync_state=state),
            max(steps // 10, 20), max(warmup // 80, 2), 1)
        e = hbm_entry(402653184, dms, "attention_prefill", 0.5)
        flops = 68853694464
        e.update(workload="AttentionKVCache prefill fp16 seq=512 past=0 causal N=32 H=32 Hkv=8 D=128",
                 device_ms_per_launch=round(dms, 5), timing=mode,
                 mfma_tflops=round(flops / (dms * 1e-3) / 1e12, 2),
                 mfma_frac=round(flops / (dms * 1e-3) / 1e12 / FP16_PEAK_TFLOPS, 4))
        if not args.no_cpu:
            import oracle
            f32 = lambda t: t.float().cpu().numpy()
            qn, kn, vn = f32(q[:1]), f32(k[:1]), f32(v[:1])
            kcn, vcn = f32(kc[:1]), f32(vc[:1])
            pairs = [(0, h) for h in range(4)]
            e["cpu_baseline"] = cpu_leg(
                lambda: oracle.attention_kvcache(qn, kn, vn, kcn, vcn, np.zeros(1, np.int64), scale, heads=pairs),
                402653184 * 4 // (Np * H), "4 of the 1024 (batch row, head) pairs; composed oracle in fp32")
            pa = [(0, h) for h in range(min(CPU_THREADS, H))]
            e["cpu_baseline_all_cores"] = cpu_all(
                pooled(lambda pr: oracle.attention_kvcache(qn, kn, vn, kcn, vcn, np.zeros(1, np.int64), scale, heads=[pr]), pa),
                402653184 * len(pa) // (Np * H), f"{len(pa)} of the 1024 (batch row, head) pairs, one per thread")
        ops_out["attention_prefill"] = e

    if want("attention_prefill_d64"):
        # the same prefill for a model with 64-wide heads (the tiled kernel on half rows)
        Np, seq, D64 = 32, 512, 64
        q = torch.randn((Np, H, seq, D64), device=dev).half()
        k = torch.randn((Np, Hkv, seq, D64), device=dev).half()
        v = torch.randn((Np, Hkv, seq, D64), device=dev).half()
        kc = torch.zeros((Np, Hkv, cap, D64), device=dev, dtype=torch.float16)
        vc = torch.zeros_like(kc)
        o = torch.empty_like(q)
        zero = torch.zeros(Np, device=dev, dtype=torch.int64)
        wsp = ops.attention_workspace(Np, H, Hkv, seq, cap, D64, dev)
        wall, dms, mode = time_steps(
            torch, lambda i: ops.attention_kvcache(q, k, v, kc, vc, zero, 1.0 / math.sqrt(D64), out=o, workspace=wsp,
                                                   sync_state=state),
            max(steps // 10, 20), max(warmup // 80, 2), 1)
        e = hbm_entry(402653184 // 2, dms)
        flops = 68853694464 // 2
        e.update(workload="AttentionKVCache prefill fp16 seq=512 past=0 causal N=32 H=32 Hkv=8 D=64",
                 device_ms_per_launch=round(dms, 5), timing=mode,
                 mfma_tflops=round(flops / (dms * 1e-3) / 1e12, 2),
                 mfma_frac=round(flops / (dms * 1e-3) / 1e12 / FP16_PEAK_TFLOPS, 4))
        ops_out["attention_prefill_d64"] = e

    if want("attention_chunk_long_history"):
        # a chunk of a long prompt (or a new turn of a conversation): one sequence, 128 new rows against a history
        # of 16384: the tiled kernel shares an item's keys between workgroups, a second launch merges
        Np, seq, past, Dc = 1, 128, 16384, 128
        capc = past + seq
        q = torch.randn((Np, H, seq, Dc), device=dev).half()
        k = torch.randn((Np, Hkv, seq, Dc), device=dev).half()
        v = torch.randn((Np, Hkv, seq, Dc), device=dev).half()
        kc = torch.randn((Np, Hkv, capc, Dc), device=dev).half()
        vc = torch.randn((Np, Hkv, capc, Dc), device=dev).half()
        o = torch.empty_like(q)
        pl = torch.full((Np,), past, device=dev, dtype=torch.int64)
        wsp = ops.attention_workspace(Np, H, Hkv, seq, capc, Dc, dev)
        wall, dms, mode = time_steps(
            torch, lambda i: ops.attention_kvcache(q, k, v, kc, vc, pl, 1.0 / math.sqrt(Dc), out=o, workspace=wsp,
                                                   sync_state=state),
            max(steps // 10, 20), max(warmup // 80, 2), 1)
        # 128 rows x 4 heads share every key: priced on the matrix cores (34 GFLOP against 68 MB)
        kv_bytes = 2 * Np * Hkv * capc * Dc * 2 + 2 * Np * H * seq * Dc * 2 + 2 * Np * Hkv * seq * Dc * 2
        flops = 4 * Np * H * Dc * (seq * past + seq * (seq + 1) // 2)
        tf = flops / (dms * 1e-3) / 1e12
        ops_out["attention_chunk_long_history"] = {
            "bound": "mfma", "achieved": round(tf, 1), "peak": FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tf / FP16_PEAK_TFLOPS, 4), "traffic": None,
            "workload": "AttentionKVCache fp16 N=1 H=32 Hkv=8 D=128, 128 new rows against a history of 16384 (both launches)",
            "device_ms_per_launch": round(dms, 5), "timing": mode, "hbm_gbs": round(kv_bytes / (dms * 1e-3) / 1e9, 1),
            "warmup_ms": LAST["warmup_ms"], "warmup_steps": LAST["warmup_steps"]}

    if want("attention_short_history_large_cache"):
        # where the host's choice between the two attention kernels is weakest: the history length is device data, so
        # half the capacity stands for it; a conversation that has just begun in a cache sized for 32768 positions
        # (8 new rows, history 100) is sent to the tiled kernel with key ranges and a merging launch, most of whose
        # ranges hold no key.  The same call with the cache nearly full is where that choice pays.
        Np, seq, capc, Dc = 1, 8, 32768, 128
        q = torch.randn((Np, H, seq, Dc), device=dev).half()
        k = torch.randn((Np, Hkv, seq, Dc), device=dev).half()
        v = torch.randn((Np, Hkv, seq, Dc), device=dev).half()
        kc = torch.randn((Np, Hkv, capc, Dc), device=dev).half()
        vc = torch.randn((Np, Hkv, capc, Dc), device=dev).half()
        o = torch.empty_like(q)
        wsp = ops.attention_workspace(Np, H, Hkv, seq, capc, Dc, dev)
        times = {}
        for label, past in (("short", 100), ("full", capc - seq - 8)):
            pl = torch.full((Np,), past, device=dev, dtype=torch.int64)
            wall, dms, mode = time_steps(
                torch, lambda i: ops.attention_kvcache(q, k, v, kc, vc, pl, 1.0 / math.sqrt(Dc), out=o, workspace=wsp,
                                                       sync_state=state),
                max(steps // 10, 20), max(warmup // 80, 2), 1)
            times[label] = dms
        short_bytes = 2 * Np * Hkv * (100 + seq) * Dc * 2 + 2 * Np * H * seq * Dc * 2 + 2 * Np * Hkv * seq * Dc * 2
        e = hbm_entry(short_bytes, times["short"])
        e.update(workload="AttentionKVCache fp16 N=1 H=32 Hkv=8 D=128, 8 new rows, cache capacity 32768, history 100 "
                          "(the kernel is chosen for half the capacity)",
                 device_ms_per_launch=round(times["short"], 5), timing=mode,
                 same_call_history_32752_device_ms=round(times["full"], 5))
        ops_out["attention_short_history_large_cache"] = e

    if want("attention_decode_group8"):
        # a decode step of a model with eight query heads per kv head (64/8): one launch reads K/V once for all eight
        Np, H8, past, Dc = 64, 64, 4096, 128
        capc = past + 1
        q = torch.randn((Np, H8, 1, Dc), device=dev).half()
        k = torch.randn((Np, Hkv, 1, Dc), device=dev).half()
        v = torch.randn((Np, Hkv, 1, Dc), device=dev).half()
        kc = torch.randn((Np, Hkv, capc, Dc), device=dev).half()
        vc = torch.randn((Np, Hkv, capc, Dc), device=dev).half()
        o = torch.empty_like(q)
        pl = torch.full((Np,), past, device=dev, dtype=torch.int64)
        wsp = ops.attention_workspace(Np, H8, Hkv, 1, capc, Dc, dev)
        wall, dms, mode = time_steps(
            torch, lambda i: ops.attention_kvcache(q, k, v, kc, vc, pl, 1.0 / math.sqrt(Dc), out=o, workspace=wsp,
                                                   sync_state=state),
            max(steps // 10, 20), max(warmup // 80, 2), 1)
        e = hbm_entry(2 * Np * Hkv * capc * Dc * 2 + 2 * Np * H8 * Dc * 2 + 2 * Np * Hkv * Dc * 2, dms)
        e.update(workload="AttentionKVCache decode fp16 N=64 H=64 Hkv=8 D=128 history 4096",
                 device_ms_per_launch=round(dms, 5), timing=mode)
        ops_out["attention_decode_group8"] = e

    if ops_out:
        result["ops"] = ops_out
    if CEILINGS or "matmul_integer_mfma_ceiling" in ops_out:
        result["ceilings"] = dict(CEILINGS)
        for nm in ("matmul_integer_mfma_ceiling", "matmul_integer_mfma_ceiling_zero"):
            if nm in ops_out:
                result["ceilings"][nm] = {k: ops_out[nm][k] for k in ("achieved", "unit", "frac", "device_ms_per_launch")}

    # The second half of the metric, where a reader of the headline object finds it, and the seven target rows
    # as the last key of the line (fraction of the published peak, microseconds per launch, and the fraction of
    # this run's own ceiling where one was measured).
    mmi = ops_out.get("matmul_integer")
    if mmi:
        keep = {k: mmi.get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "device_ms_per_launch")}
        clk = mmi.get("observed_sclk_mhz")
        keep["observed_sclk_mhz"] = clk["median"] if clk else None
        ceil = ops_out.get("matmul_integer_mfma_ceiling")
        if ceil:
            keep["mfma_ceiling_frac"] = ceil["frac"]
            keep["frac_of_ceiling"] = round(mmi["frac"] / ceil["frac"], 4)
        roofline["matmul_integer"] = keep
        result["config"]["matmul_integer_workload"] = "u8 [4096,4096] x i8 [4096,4096] -> i32, a_zp=128, b_zp=0"
    targets = {"attention_decode": {"frac": roofline["frac"], "us": round(roofline["device_ms_per_launch"] * 1e3, 2),
                                    "of_ceiling": roofline.get("frac_of_ceiling")}}
    for nm in ("rms_norm", "softmax", "softmax_causal", "rope", "dequantize_linear", "matmul_integer", "attention_prefill"):
        if nm in ops_out:
            e = ops_out[nm]
            of = e.get("frac_of_ceiling")
            if nm == "matmul_integer" and "matmul_integer_mfma_ceiling" in ops_out:
                of = round(e["frac"] / ops_out["matmul_integer_mfma_ceiling"]["frac"], 4)
            targets[nm] = {"frac": e["frac"], "us": round(e["device_ms_per_launch"] * 1e3, 2), "of_ceiling": of}
    roofline["targets"] = {k: v["frac"] for k, v in targets.items()}
    result["targets"] = targets
    for pool in _POOL:
        pool.shutdown()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
