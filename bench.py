#!/usr/bin/env python3
"""Benchmark of the op-kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-extras] [--no-cpu] [--pmc-probe | --mfma-probe]

Prints ONE JSON line.  The headline workload (`config.workload`) is the second of the five
benchmark configurations of this path: ReduceMaxOp_f32_f32 and ReduceSumOp_f32_f32
over axis 0 (column / two-pass split case) and over axis 1 of one [16384, 8192] float tensor; a
"step" is those four op-kernel launches, `value` is the algorithmic bytes of a step divided by the
step time, inputs resident in HBM.  The other listed configurations (row sum, fused softmax,
flash-attention forward and backward) are timed in the same run and reported under `all_configs`,
each with its own roofline fraction, the shader clock sampled while it ran, and CPU figures on
one core and on all cores of this job's share.

Inputs come from the library's counter-based generator (brt_rocm_fill: element i is a function
of (seed, i) only), with one seed per tensor; the CPU side regenerates the same bits with
oracle.fill instead of reading buffers back.  Every configuration passes a parity gate against the
CPU oracle before it is timed; a failed gate ends the run.

Timing: HIP events recorded on the stream the kernels are launched on (through the library's
own C ABI, not torch's event wrapper), plus a host clock around the synchronised region.
`value` and every `us_per_op` come from ONE pair of events around all timed steps; `median_*`
from a second pass with an event pair per step.  Everything is launched through the C ABI
(libbrt_rocm_kernels.so / libflash_attn.so); torch is used for device memory and streams only.
"""
import argparse
import ctypes
import glob
import json
import os
import re
import statistics
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 / fp16 MFMA, published (256 CUs x 4 SIMDs x 1024 FLOP/clk x 2.4 GHz)
PEAK_CLOCK_MHZ = 2400.0

METRIC = "reduce HBM GB/s + flash-attn fwd/bwd TFLOP/s, % of MI355X roofline, 1 GPU"

# seeds of the synthetic tensors: one per tensor; rotating copies add their index << 32
SEED = {"c1": 0xC1, "c2": 0xC2, "c3": 0xC3, "c4q": 0xC41, "c4k": 0xC42, "c4v": 0xC43,
        "c5q": 0xC51, "c5k": 0xC52, "c5v": 0xC53, "c5do": 0xC54, "dec": 0xDC}


class Events:
    """HIP events on a given stream via the C ABI."""

    def __init__(self, K, stream):
        self.K, self.stream = K, stream

    def new(self):
        e = ctypes.c_void_p()
        assert self.K.brt_rocm_event_create(ctypes.byref(e)) == 0
        return e

    def record(self, e):
        assert self.K.brt_rocm_event_record(e, self.stream) == 0

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        assert self.K.brt_rocm_event_synchronize(b) == 0
        assert self.K.brt_rocm_event_elapsed_ms(ctypes.byref(ms), a, b) == 0
        return ms.value

    def free(self, evs):
        for e in evs:
            self.K.brt_rocm_event_destroy(e)


class ClockSampler:
    """Samples the GPU's current shader clock (the starred level of pp_dpm_sclk) from a thread
    while a timed region runs: the attention kernels do not hold the 2.4 GHz the published MFMA
    peak assumes, and how far they fall depends on the data (zeros run faster than random
    numbers), so a TFLOP/s figure is only comparable together with the clock it ran at."""

    def __init__(self):
        files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.path = files[0] if files else None
        self.samples, self._stop, self._t = [], None, None

    def read(self):
        if not self.path:
            return None
        try:
            for line in open(self.path).read().splitlines():
                if "*" in line:
                    m = re.search(r"(\d+)\s*[Mm][Hh]z", line)
                    return float(m.group(1)) if m else None
        except OSError:
            return None
        return None

    def __enter__(self):
        self.samples, self._stop = [], threading.Event()

        def run():
            while not self._stop.is_set():
                v = self.read()
                if v:
                    self.samples.append(v)
                time.sleep(0.002)

        self._t = threading.Thread(target=run, daemon=True)
        self._t.start()
        return self

    def __exit__(self, *a):
        self._stop.set()
        self._t.join()

    def summary(self):
        s = [v for v in self.samples if v > 400]  # drop the idle level seen before the first launch lands
        if not s:
            return None
        return {"mean_mhz": round(sum(s) / len(s), 0), "min_mhz": min(s), "max_mhz": max(s), "samples": len(s)}


def time_ops(ev, fns, steps, warmup, clocks=None):
    """Run `fns` (a list of launch closures = one step) `warmup` + `steps` times.
    -> dict(ms: ms per step from one event pair around all steps, per: [ms per launch of fns[i]],
    host_ms, median_ms: median over per-step event pairs of a second pass, clock: sampled MHz)."""
    import torch
    for _ in range(warmup):
        for f in fns:
            f()
    torch.cuda.synchronize()
    e0, e1 = ev.new(), ev.new()
    sampler = clocks if clocks is not None else ClockSampler()
    with sampler:
        t0 = time.perf_counter()
        ev.record(e0)
        for _ in range(steps):
            for f in fns:
                f()
        ev.record(e1)
        torch.cuda.synchronize()
        host_ms = (time.perf_counter() - t0) * 1e3 / steps
    total = ev.elapsed_ms(e0, e1) / steps
    ev.free([e0, e1])
    # second pass: an event after every launch (each costs a few microseconds of idle GPU, so
    # this pass feeds the per-launch breakdown and the median only)
    marks = [[ev.new() for _ in range(len(fns) + 1)] for _ in range(steps)]
    for s in range(steps):
        ev.record(marks[s][0])
        for i, f in enumerate(fns):
            f()
            ev.record(marks[s][i + 1])
    torch.cuda.synchronize()
    per = [sum(ev.elapsed_ms(marks[s][i], marks[s][i + 1]) for s in range(steps)) / steps for i in range(len(fns))]
    med = statistics.median(ev.elapsed_ms(marks[s][0], marks[s][-1]) for s in range(steps))
    for m in marks:
        ev.free(m)
    return {"ms": total, "per": per, "host_ms": host_ms, "median_ms": med, "clock": sampler.summary()}


def time_regions(ev, fns, iters, warmup, regions=3, clocks=None):
    """`regions` independent timed regions of `iters` steps each (a step = every closure of `fns`
    once), one event pair per region on the launch stream, a synchronisation between regions.
    -> dict(ms: the MEDIAN region's ms per step, min_ms, max_ms, region_ms, host_ms, clock: the
    shader clock sampled over all regions).  A 2-3 % difference between two kernels is of the
    size of the spread between regions; the three figures together say how much a number means."""
    import torch
    for _ in range(warmup):
        for f in fns:
            f()
    torch.cuda.synchronize()
    sampler = clocks if clocks is not None else ClockSampler()
    region_ms, host = [], []
    with sampler:
        for _ in range(regions):
            e0, e1 = ev.new(), ev.new()
            t0 = time.perf_counter()
            ev.record(e0)
            for _ in range(iters):
                for f in fns:
                    f()
            ev.record(e1)
            torch.cuda.synchronize()
            host.append((time.perf_counter() - t0) * 1e3 / iters)
            region_ms.append(ev.elapsed_ms(e0, e1) / iters)
            ev.free([e0, e1])
    return {"ms": statistics.median(region_ms), "min_ms": min(region_ms), "max_ms": max(region_ms),
            "region_ms": region_ms, "host_ms": statistics.median(host), "clock": sampler.summary(),
            "iters": iters, "regions": regions}


def spread(r, ops_per_step=1, digits=2):
    """min / median / max microseconds per op over the timed regions of `r`."""
    k = 1e3 / ops_per_step
    return {"min_us_per_op": round(r["min_ms"] * k, digits), "median_us_per_op": round(r["ms"] * k, digits),
            "max_us_per_op": round(r["max_ms"] * k, digits), "timed_regions": r["regions"], "iterations_per_region": r["iters"]}


def roof(bound, kernel, work, unit_work, ms, peak, source):
    """The roofline entry of one configuration: algorithmic bytes (or FLOP) per op over the
    median time per op, against the published peak."""
    rate = work / (ms * 1e-3) / (1e9 if bound == "hbm" else 1e12)
    return {"bound": bound, "kernel": kernel, "achieved": round(rate, 1), "peak": peak,
            "unit": "GB/s" if bound == "hbm" else "TFLOP/s", "frac": round(rate / peak, 4),
            "algorithmic_" + unit_work: work, "us": round(ms * 1e3, 2), "duration_source": source}


def prewarm(fn, seconds=0.5):
    """Run `fn` back to back for about `seconds` of wall time.  After idle time (the parity gate's
    CPU work) or after memory-bound kernels the matrix-heavy attention kernels run 10-20 % slower
    for some tenths of a second while the clocks settle; the timed region should see the steady
    state."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def cpu_time(fn, repeat=2):
    best = float("inf")
    for _ in range(repeat):
        t = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t)
    return best


def cpu_both(oracle, fn, n_thr, repeat=2):
    """Best-of-`repeat` seconds of `fn` on one core and with OpenMP on `n_thr` threads."""
    oracle.set_threads(1)
    t1 = cpu_time(fn, repeat)
    oracle.set_threads(n_thr)
    tn = cpu_time(fn, repeat)
    oracle.set_threads(1)
    return t1, tn


def gate(ok, what):
    if not ok:
        sys.exit(f"bench.py: parity gate failed before timing: {what}")


def measured_traffic(K, _lib, R, Cc):
    """HBM bytes of one first-pass launch of the axis-0 fold, from the tracked counter profile
    (FETCH_SIZE and WRITE_SIZE per dispatch, each scaled by the same counter's reading for a copy
    kernel of known size).  The profile is only valid for the split it was measured with: the
    workspace size it records must equal what the library plans today."""
    path = os.path.join(ROOT, "profiles", "reduce_c2_hbm_traffic.txt")
    if not os.path.exists(path):
        return None, "profiles/reduce_c2_hbm_traffic.txt not present"
    text = open(path).read()
    vals = {"FETCH_SIZE": [], "WRITE_SIZE": []}
    section = None
    for line in text.splitlines():
        for k in vals:
            if line.startswith(k + ":"):
                section = k
        m = re.search(r"reduce_colwide_kernel<float, float, [01],.*scaled_bytes=\s*(\d+)", line)
        if m and section:
            vals[section].append(int(m.group(1)))
    if not vals["FETCH_SIZE"] or not vals["WRITE_SIZE"]:
        return None, "no reduce_colwide_kernel rows in the profile"
    # the profile must name the very kernel instantiation the library plans today
    buf = ctypes.create_string_buffer(256)
    _lib.check(K.brt_rocm_reduce_plan_describe(_lib.F32, 1, R, Cc, buf, 256))
    plan = buf.value.decode()
    for op in "01":
        name = plan.split(" S=")[0].replace("OP", op)
        if name not in text:
            sys.exit(f"bench.py: profiles/reduce_c2_hbm_traffic.txt was measured with another kernel than today's plan ({name}): re-measure it")
    ws_now = K.brt_rocm_reduce_workspace_bytes(_lib.F32, 1, R, Cc)
    ws_then = sum(vals["WRITE_SIZE"]) // len(vals["WRITE_SIZE"])  # the first pass writes exactly its partials
    if ws_now != ws_then:
        sys.exit(f"bench.py: the axis-0 split has changed (partials {ws_now} B now, {ws_then} B when "
                 "profiles/reduce_c2_hbm_traffic.txt was measured): re-measure the traffic profile")
    fetch = sum(vals["FETCH_SIZE"]) / len(vals["FETCH_SIZE"])
    return int(round(fetch + ws_then)), ("not measured in this run: read from the tracked profile profiles/reduce_c2_hbm_traffic.txt "
                                         "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, copy-kernel scaled), which names the same "
                                         "kernel instantiation and the same split as today's plan: " + plan)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=["c2"])
    ap.add_argument("--no-extras", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter-collection mode: one copy kernel of known size, then two C2 steps, two cache-decode calls and two softmax calls")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="counter-collection mode: only the MFMA rate probe, 40 launches per operand set (fp16 / bf16, zeros / N(0,1))")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is single-GPU (one process, one MI355X); run with --gpus 1")

    import numpy as np
    import torch
    from byteir_amd import _lib, ops

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    K = _lib.kernels()
    _lib.flash_attn()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    sp = ctypes.c_void_p(stream.cuda_stream)
    ev = Events(K, sp)
    import oracle  # the checker: parity gates and the cpu_baseline legs only

    # ---- headline: C2, [16384, 8192] f32 ~ U(-1, 1) --------------------------------------
    R, Cc = 16384, 8192
    NBUF = 3  # rotate inputs: 1.5 GiB between two touches of a buffer, beyond the 256 MB LLC
    xs = [ops.fill(torch.empty((R, Cc), device="cuda"), _lib.FILL_UNIFORM, SEED["c2"] + (i << 32), -1.0, 1.0) for i in range(NBUF)]
    out_col = torch.empty(Cc, device="cuda")
    out_row = torch.empty(R, device="cuda")
    ws_col = torch.empty(max(1, ops.reduce_workspace_bytes(torch.float32, 1, R, Cc)), dtype=torch.uint8, device="cuda")
    ws_row = torch.empty(max(1, ops.reduce_workspace_bytes(torch.float32, R, Cc, 1)), dtype=torch.uint8, device="cuda")
    in_bytes = R * Cc * 4
    bytes_col = in_bytes + Cc * 4   # 536 903 680
    bytes_row = in_bytes + R * 4    # 536 936 448
    step_bytes = 2 * bytes_col + 2 * bytes_row
    rot = [0]

    def nxt():
        rot[0] = (rot[0] + 1) % NBUF
        return xs[rot[0]]

    c2_fns = [
        lambda: ops.reduce_abc(_lib.REDUCE_MAX, nxt(), out_col, 1, R, Cc, workspace=ws_col),
        lambda: ops.reduce_abc(_lib.REDUCE_SUM, nxt(), out_col, 1, R, Cc, workspace=ws_col),
        lambda: ops.reduce_abc(_lib.REDUCE_MAX, nxt(), out_row, R, Cc, 1, workspace=ws_row),
        lambda: ops.reduce_abc(_lib.REDUCE_SUM, nxt(), out_row, R, Cc, 1, workspace=ws_row),
    ]

    if args.mfma_probe:
        # for `rocprofv3 --pmc GRBM_GUI_ACTIVE --kernel-trace`: busy cycles over duration = the clock the
        # chip held during each launch
        del xs
        blocks, iters = torch.cuda.get_device_properties(0).multi_processor_count, 8000
        opnd = torch.empty(blocks * 512 * 256, dtype=torch.uint8, device="cuda")
        sink = torch.empty(blocks * 512, dtype=torch.float32, device="cuda")
        flop = blocks * 8 * iters * 16 * 32768
        rates = {}
        for name, code, dt in (("f16", 1, torch.float16), ("bf16", 2, torch.bfloat16)):
            for what in ("zeros", "normal"):
                if what == "zeros":
                    opnd.zero_()
                else:
                    ops.fill(opnd.view(dt), _lib.FILL_NORMAL, SEED["c4q"], 0.0, 1.0)
                probe = lambda: _lib.check(K.brt_rocm_mfma_rate_probe(code, opnd.data_ptr(), opnd.numel(), sink.data_ptr(), sink.numel() * 4, blocks, iters, sp))
                r = time_regions(ev, [probe], 10, 10)
                rates[f"{name}_{what}"] = round(flop / (r["ms"] * 1e-3) / 1e12, 1)
        print(json.dumps({"mfma_probe": True, "TFLOPs": rates, "flop_per_launch": flop, "launches_per_operand_set": 40}))
        return

    if args.pmc_probe:
        dst = torch.empty_like(xs[0])
        _lib.check(K.brt_rocm_copy_kernel(dst.data_ptr(), xs[0].data_ptr(), in_bytes, sp))
        for _ in range(2):
            for f in c2_fns:
                f()
        torch.cuda.synchronize()
        # two calls of the cache-decode configuration (64 sequences x 8192 cached keys, 32 query
        # heads on 8 key/value heads of 128, fp16): 2 GiB of cache rows per call
        del dst
        b_, h_, hk_, sk_, d_ = 64, 32, 8, 8192, 128
        mk = lambda shape, j: ops.fill(torch.empty(shape, dtype=torch.float16, device="cuda"), _lib.FILL_NORMAL, SEED["dec"] + (j << 32), 0.0, 1.0)
        qd, kc, vc, kn, vn = mk((b_, 1, h_, d_), 0), mk((b_, sk_, hk_, d_), 1), mk((b_, sk_, hk_, d_), 2), mk((b_, 1, hk_, d_), 3), mk((b_, 1, hk_, d_), 4)
        lens = torch.full((b_,), sk_ - 1, dtype=torch.int32, device="cuda")
        for _ in range(2):
            ops.flash_attn_kvcache(qd, kc, vc, kn, vn, lens, 1.0 / np.sqrt(d_), (-1, -1))
        torch.cuda.synchronize()
        # two calls of the fused softmax configuration ([32768, 4096] bf16: 256 MiB in, 256 MiB out)
        del qd, kc, vc, kn, vn
        x3 = ops.fill(torch.empty((32768, 4096), dtype=torch.bfloat16, device="cuda"), _lib.FILL_NORMAL, SEED["c3"], 0.0, 2.0)
        y3 = torch.empty_like(x3)
        for _ in range(2):
            ops.softmax(x3, out=y3)
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": True, "copy_bytes_read": in_bytes, "copy_bytes_written": in_bytes,
                          "decode_cache_bytes": 2 * b_ * sk_ * hk_ * d_ * 2, "softmax_bytes_each_way": 32768 * 4096 * 2}))
        return

    # parity gate (and the CPU baseline's input): the host regenerates buffer 0 from its seed
    n_thr = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
    xh = oracle.fill(0, oracle.UNIFORM, SEED["c2"], R * Cc, -1.0, 1.0).reshape(R, Cc)
    gate(np.array_equal(xs[0][:64].cpu().numpy(), xh[:64]) and np.array_equal(xs[0][-1].cpu().numpy(), xh[-1]),
         "GPU fill and host fill disagree")
    oracle.set_threads(n_thr)
    for dims, (A, B, C), o in (((0,), (1, R, Cc), out_col), ((1,), (R, Cc, 1), out_row)):
        ops.reduce_abc(_lib.REDUCE_MAX, xs[0], o, A, B, C, workspace=ws_col if C > 1 else ws_row)
        gate(np.array_equal(o.cpu().numpy(), oracle.reduce_abc(oracle.MAX, xh, A, B, C)), f"c2 ReduceMax dims={dims}")
        ops.reduce_abc(_lib.REDUCE_SUM, xs[0], o, A, B, C, workspace=ws_col if C > 1 else ws_row)
        s64, sabs = oracle.reduce_sum_f64(xh, A, B, C)
        gate(np.all(np.abs(o.cpu().numpy().astype(np.float64) - s64) <= 1e-5 * np.maximum(np.abs(s64), 1e-2 * sabs)),
             f"c2 ReduceSum dims={dims} (1e-5 relative against the float64 fold)")
    oracle.set_threads(1)

    # `value`: three timed regions of exactly `steps` steps each (after `warmup` untimed steps),
    # the median region counts; the per-launch breakdown comes from a marked pass of time_ops
    r2 = time_regions(ev, c2_fns, args.steps, args.warmup)
    r2m = time_ops(ev, c2_fns, args.steps, 0)
    ms_step, per, host_ms = r2["ms"], r2m["per"], r2["host_ms"]
    value = step_bytes / (ms_step * 1e-3) / 1e9
    # The same step as the runtime runs it: a ByRE module with the four Reduce{Max,Sum}Op_f32_f32
    # ops, loaded by the C++ session (workspace from the frame's allocator), one `run` per step
    # over the same three rotating inputs (one request context per input buffer).
    from byteir_amd import brt
    t_in, t_c, t_r = f'memref<{R}x{Cc}xf32, "cuda">', f'memref<{Cc}xf32, "cuda">', f'memref<{R}xf32, "cuda">'
    mod = ("module attributes {byre.container_module} {\n  func.func @c2(\n"
           f'    %x : {t_in} {{byre.argname = "X", byre.argtype = 1: i32}},\n'
           f'    %cmax : {t_c} {{byre.argname = "CMAX", byre.argtype = 2: i32}},\n'
           f'    %csum : {t_c} {{byre.argname = "CSUM", byre.argtype = 2: i32}},\n'
           f'    %rmax : {t_r} {{byre.argname = "RMAX", byre.argtype = 2: i32}},\n'
           f'    %rsum : {t_r} {{byre.argname = "RSUM", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{\n'
           + "".join(f'    byre.compute @Reduce{op}Op_f32_f32(%x, %{o}) {{dimensions = dense<[{d}]> : tensor<1xi64>, '
                     f'memory_effects = [1 : i32, 2 : i32]}} : {t_in}, {t}\n'
                     for op, o, d, t in (("Max", "cmax", 0, t_c), ("Sum", "csum", 0, t_c), ("Max", "rmax", 1, t_r), ("Sum", "rsum", 1, t_r)))
           + "    return\n  }\n}\n")
    sess = brt.Session(device="ROCM", device_id=0)
    sess.load_from_memory(mod)
    s_outs = [torch.empty(n, device="cuda") for n in (Cc, Cc, R, R)]
    reqs = []
    for x in xs:
        rq = sess.new_request_context(torch.cuda.current_stream().cuda_stream)
        rq.bind_arg(0, x.data_ptr())
        for j, o in enumerate(s_outs):
            rq.bind_arg(1 + j, o.data_ptr())
        rq.finish_io_binding()
        reqs.append(rq)
    reqs[0].run()
    reqs[0].sync()
    ops.reduce_abc(_lib.REDUCE_SUM, xs[0], out_col, 1, R, Cc, workspace=ws_col)
    ops.reduce_abc(_lib.REDUCE_MAX, xs[0], out_row, R, Cc, 1, workspace=ws_row)
    gate(torch.equal(s_outs[1], out_col) and torch.equal(s_outs[2], out_row), "c2 through the session differs from the direct calls")
    rq_i = [0]

    def session_step():
        rq_i[0] = (rq_i[0] + 1) % len(reqs)
        reqs[rq_i[0]].run()

    r_sess = time_regions(ev, [session_step], args.steps, args.warmup)
    # per-op figures: each pair of launches timed back to back on its own, one event pair around
    # all repeats (an event after every launch, as in `per`, leaves the GPU idle for a few
    # microseconds per launch and is kept only as a secondary figure)
    r_col = time_regions(ev, c2_fns[:2], max(args.steps, 25), max(2, args.warmup // 2))
    r_row = time_regions(ev, c2_fns[2:], max(args.steps, 25), max(2, args.warmup // 2))
    col_ms, row_ms = r_col["ms"] / 2, r_row["ms"] / 2
    col_ms_marked, row_ms_marked = (per[0] + per[1]) / 2, (per[2] + per[3]) / 2
    # The axis-0 op is two launches: the split first pass (the dominant kernel) and a small
    # combine over the [S, 8192] partials.  A second timed region records an event between the
    # two (brt_rocm_reduce_ex), so `avg_launch_us` is the first pass alone (compare with
    # rocprofv3's figure for reduce_colwide_kernel).
    n_mid = max(args.steps, 10)
    triples = [(ev.new(), ev.new(), ev.new()) for _ in range(2 * n_mid)]
    for i, (e0, e1, e2) in enumerate(triples):
        ev.record(e0)
        _lib.check(K.brt_rocm_reduce_ex(_lib.REDUCE_MAX if i % 2 == 0 else _lib.REDUCE_SUM, _lib.F32, nxt().data_ptr(),
                                        out_col.data_ptr(), 1, R, Cc, ws_col.data_ptr(), ws_col.numel(), sp, e1))
        ev.record(e2)
    torch.cuda.synchronize()
    pass1_ms = sum(ev.elapsed_ms(e0, e1) for e0, e1, _ in triples) / len(triples)
    p2_ms = sum(ev.elapsed_ms(e1, e2) for _, e1, e2 in triples) / len(triples)
    for t in triples:
        ev.free(t)
    col_gbs = bytes_col / (pass1_ms * 1e-3) / 1e9
    traffic, traffic_src = measured_traffic(K, _lib, R, Cc)
    roofline = {
        "bound": "hbm", "kernel": "reduce_colwide_kernel<float, float, OP, 4, 4, 2> (first pass of the axis-0 split reduction)",
        "achieved": round(col_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(col_gbs / HBM_PEAK_GBS, 4),
        "algorithmic_bytes_per_launch": bytes_col, "avg_launch_us": round(pass1_ms * 1e3, 2),
        "op_us_including_combine_pass": round(col_ms * 1e3, 2), "combine_pass_us": round(p2_ms * 1e3, 2),
        "traffic": traffic, "traffic_source": traffic_src,
    }
    col_op_gbs = bytes_col / (col_ms * 1e-3) / 1e9

    props = torch.cuda.get_device_properties(0)
    max_sclk = None
    try:
        levels = [float(m) for m in re.findall(r"(\d+)\s*[Mm][Hh]z", open(ClockSampler().path).read())]
        max_sclk = max(levels) if levels else None
    except (OSError, TypeError):
        pass
    result = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "ms_per_step_regions": {"min": round(r2["min_ms"], 4), "median": round(r2["ms"], 4), "max": round(r2["max_ms"], 4),
                                "timed_regions": r2["regions"], "steps_per_region": args.steps},
        "ms_per_step_with_an_event_after_every_launch": round(r2m["median_ms"], 4),
        "host_ms_per_step": round(host_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "c2: ReduceMaxOp_f32_f32 + ReduceSumOp_f32_f32 over axis 0 and over axis 1 "
                               "of [16384, 8192] f32 ~ U(-1,1) (4 op-kernel launches per step, "
                               f"{NBUF} rotating input buffers)",
                   "algorithmic_bytes_per_step": step_bytes,
                   "generator": "brt_rocm_fill / oracle_fill: splitmix64 counter stream per tensor (uniform: 24 bits; "
                                "normal: sum of twelve 16-bit fields), seeds " + json.dumps({k: hex(v) for k, v in SEED.items()})},
        "roofline": roofline,
        "through_brt_session": {"ms_per_step": round(r_sess["ms"], 4), "value": round(step_bytes / (r_sess["ms"] * 1e-3) / 1e9, 1),
                                "unit": "GB/s", "what": "the same four ops as one ByRE module run by the C++ session"},
        "device": {"name": props.name, "compute_units": props.multi_processor_count,
                   "max_shader_clock_mhz": max_sclk, "hbm_bytes": props.total_memory,
                   "memory_clock_mhz": (getattr(props, "memory_clock_rate", 0) or 0) / 1e3 or None,
                   "memory_bus_bits": getattr(props, "memory_bus_width", None),
                   "published_peaks": {"hbm_GBs": HBM_PEAK_GBS, "mfma_f16_bf16_dense_TFLOPs": MFMA_PEAK_TFLOPS,
                                       "at_shader_clock_mhz": PEAK_CLOCK_MHZ},
                   # compute units x 4 SIMDs x 1024 FLOP per clock (one 32x32x16 MFMA per 32 clocks) x the top clock level
                   "mfma_peak_from_device_TFLOPs": round(props.multi_processor_count * 4 * 1024 * max_sclk * 1e6 / 1e12, 1) if max_sclk else None,
                   "shader_clock_during_c2": r2["clock"]},
    }

    all_cfg = {
        "c2a_col_max_sum_axis0": {"value": round(col_op_gbs, 1), "unit": "GB/s", "us_per_op": round(col_ms * 1e3, 2),
                                  "frac_of_hbm_peak": round(col_op_gbs / HBM_PEAK_GBS, 4),
                                  "first_pass_kernel_GBs": round(col_gbs, 1),
                                  "us_per_op_with_an_event_after_every_launch": round(col_ms_marked * 1e3, 2),
                                  **spread(r_col, 2),
                                  "roofline": roof("hbm", "reduce_colwide_kernel<float, float, OP, 4, 4, 2> + reduce_col_kernel<float, float, OP, 4, 8> (combine pass)",
                                                   bytes_col, "bytes", col_ms, HBM_PEAK_GBS, "event pair around back-to-back ops (both launches of an op), median of three regions")},
        "c2b_row_max_sum_axis1": {"value": round(bytes_row / (row_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                                  "us_per_op": round(row_ms * 1e3, 2),
                                  "frac_of_hbm_peak": round(bytes_row / (row_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                  "us_per_op_with_an_event_after_every_launch": round(row_ms_marked * 1e3, 2),
                                  **spread(r_row, 2),
                                  "roofline": roof("hbm", "reduce_row_kernel<float, float, OP, 4, 256, false>", bytes_row, "bytes", row_ms, HBM_PEAK_GBS,
                                                   "event pair around back-to-back launches, median of three regions")},
    }

    # ---- CPU baseline for the headline workload --------------------------------------------
    if not args.no_cpu:
        step = lambda: (oracle.reduce_abc(oracle.MAX, xh, 1, R, Cc), oracle.reduce_abc(oracle.SUM, xh, 1, R, Cc),
                        oracle.reduce_abc(oracle.MAX, xh, R, Cc, 1), oracle.reduce_abc(oracle.SUM, xh, R, Cc, 1))
        t_cpu, t_par = cpu_both(oracle, step, n_thr, 60)
        result["cpu_baseline"] = {
            "value": round(step_bytes / t_cpu / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "the full step (4 reductions of the [16384, 8192] tensor) run once per repeat, best of 60 (about 10 s of CPU work on one core), "
                      "by the scalar loop-nest oracle (the reference's CPU path is single-threaded LLVM-JIT'ed "
                      "loop nests, which cannot be built here)",
            "seconds": round(t_cpu, 3), "host_cores_available": os.cpu_count(),
            # the same loop nests with OpenMP over the independent outputs, on this job's CPU share
            "openmp": {"value": round(step_bytes / t_par / 1e9, 3), "unit": "GB/s", "cores": n_thr, "seconds": round(t_par, 3)},
        }
        for key, (A, B, C), byt in (("c2a_col_max_sum_axis0", (1, R, Cc), bytes_col), ("c2b_row_max_sum_axis1", (R, Cc, 1), bytes_row)):
            t1, tn = cpu_both(oracle, lambda: (oracle.reduce_abc(oracle.MAX, xh, A, B, C), oracle.reduce_abc(oracle.SUM, xh, A, B, C)), n_thr, 1)
            all_cfg[key]["cpu_1core_GBs"] = round(2 * byt / t1 / 1e9, 3)
            all_cfg[key]["cpu_allcore_GBs"] = round(2 * byt / tn / 1e9, 3)
            all_cfg[key]["cpu_cores"] = n_thr
    del xh

    if not args.no_extras:
        extras(all_cfg, ev, ops, _lib, oracle, args, np, torch, n_thr)
    result["all_configs"] = all_cfg
    print(json.dumps(result))


def with_clock(entry, r, peak, key):
    """Adds the spread over the timed regions, the sampled shader clock and the fraction of the
    peak scaled to that clock."""
    c = r["clock"]
    entry.update(spread(r, r.get("ops_per_step", 1), 1))
    if c:
        entry["shader_clock_mhz"] = c
        entry[key + "_at_sampled_clock"] = round(entry["value"] / (peak * c["mean_mhz"] / PEAK_CLOCK_MHZ), 4)
    return entry


def extras(all_cfg, ev, ops, _lib, oracle, args, np, torch, n_thr):
    """The remaining benchmark configurations: parity gate, timing, CPU figures."""
    steps, warm = max(5, args.steps // 2), max(2, args.warmup // 2)
    do_cpu = not args.no_cpu
    F, H, B16 = torch.float32, torch.float16, torch.bfloat16

    def mk(shape, dtype, dist, seed, a, b):
        return ops.fill(torch.empty(shape, dtype=dtype, device="cuda"), dist, seed, a, b)

    # c1: row ReduceSum f32 [4096, 1024] ~ N(0,1).  16 MiB: launch-bound; rotating 40 buffers
    # (640 MiB) keeps the input out of the 256 MB LLC ("cold"), one buffer gives the warm figure.
    bufs = [mk((4096, 1024), F, _lib.FILL_NORMAL, SEED["c1"] + (i << 32), 0.0, 1.0) for i in range(40)]
    o1 = torch.empty(4096, device="cuda")
    b1 = 4096 * 1024 * 4 + 4096 * 4
    xh = oracle.fill(0, oracle.NORMAL, SEED["c1"], 4096 * 1024, 0.0, 1.0).reshape(4096, 1024)
    ops.reduce_abc(_lib.REDUCE_SUM, bufs[0], o1, 4096, 1024, 1)
    s64, sabs = oracle.reduce_sum_f64(xh, 4096, 1024, 1)
    gate(np.all(np.abs(o1.cpu().numpy().astype(np.float64) - s64) <= 1e-5 * np.maximum(np.abs(s64), 1e-2 * sabs)), "c1 row ReduceSum")
    i = [0]

    def c1_cold():
        i[0] = (i[0] + 1) % len(bufs)
        ops.reduce_abc(_lib.REDUCE_SUM, bufs[i[0]], o1, 4096, 1024, 1)

    rc = time_regions(ev, [c1_cold] * 10, 50, warm)
    # the same launches through the C ABI itself with the arguments marshalled once (what a
    # compiled host pays per launch), instead of through the Python mirror of the op interface
    import functools
    K1 = _lib.kernels()
    sp1 = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    direct = [functools.partial(K1.brt_rocm_reduce, _lib.REDUCE_SUM, _lib.F32, ctypes.c_void_p(b.data_ptr()),
                                ctypes.c_void_p(o1.data_ptr()), 4096, 1024, 1, None, 0, sp1) for b in bufs]
    rd = time_regions(ev, direct, 50, warm)  # 50 x 40 launches per region
    rw = time_regions(ev, [lambda: ops.reduce_abc(_lib.REDUCE_SUM, bufs[0], o1, 4096, 1024, 1)] * 10, 50, warm)
    ms_cold, ms_warm = rc["ms"], rw["ms"]
    # the same 40 cold launches captured once in a HIP graph: launch cost leaves the host
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for b in bufs:
            ops.reduce_abc(_lib.REDUCE_SUM, b, o1, 4096, 1024, 1, stream=side)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for b in bufs:
                ops.reduce_abc(_lib.REDUCE_SUM, b, o1, 4096, 1024, 1, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    ms_graph = time_regions(ev, [graph.replay], 50, warm)["ms"]
    # and through the runtime itself: one ByRE module with 40 ReduceSumOp_f32_f32 ops, one per
    # buffer, run by the C++ session (one `run` = 40 op-kernel launches on the request's stream)
    from byteir_amd import brt
    tin, tout = 'memref<4096x1024xf32, "cuda">', 'memref<4096xf32, "cuda">'
    margs = ",\n".join(f'    %arg{j} : {tin} {{byre.argname = "A{j}", byre.argtype = 1: i32}}' for j in range(len(bufs)))
    mops = "\n".join(f'    byre.compute @ReduceSumOp_f32_f32(%arg{j}, %out) {{dimensions = dense<[1]> : tensor<1xi64>, '
                      f'memory_effects = [1 : i32, 2 : i32]}} : {tin}, {tout}' for j in range(len(bufs)))
    module = ("module attributes {byre.container_module} {\n  func.func @c1(\n" + margs +
              f',\n    %out : {tout} {{byre.argname = "B", byre.argtype = 2: i32}}) attributes {{byre.entry_point}} {{\n' +
              mops + "\n    return\n  }\n}\n")
    sess = brt.Session(device="ROCM", device_id=0)
    sess.load_from_memory(module)
    req = sess.new_request_context(torch.cuda.current_stream().cuda_stream)
    for j, b in enumerate(bufs):
        req.bind_arg(j, b.data_ptr())
    o_sess = torch.zeros(4096, device="cuda")
    req.bind_arg(len(bufs), o_sess.data_ptr())
    req.finish_io_binding()
    req.run()
    req.sync()
    gate(torch.equal(o_sess, ops.reduce_abc(_lib.REDUCE_SUM, bufs[-1], torch.empty_like(o_sess), 4096, 1024, 1)),
         "c1 through the session differs from the direct call")
    rs = time_regions(ev, [req.run], 50, warm)
    ms_direct = rd["ms"] / len(bufs)
    c1 = {"value": round(b1 / (ms_direct * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_op": round(ms_direct * 1e3, 2),
          "frac_of_hbm_peak": round(b1 / (ms_direct * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
          **spread(rd, len(bufs)),
          "roofline": roof("hbm", "reduce_row_kernel<float, float, 1, 4, 64, false>", b1, "bytes", ms_direct, HBM_PEAK_GBS,
                           "event pair around 2000 back-to-back launches over 40 rotating buffers (launch gaps included), median of three regions"),
          "python_mirror_GBs": round(b1 / (ms_cold / 10 * 1e-3) / 1e9, 1), "python_mirror_us_per_op": round(ms_cold / 10 * 1e3, 2),
          "python_mirror_warm_cache_us_per_op": round(ms_warm / 10 * 1e3, 2),
          "brt_session_us_per_op": round(rs["ms"] / len(bufs) * 1e3, 2),
          "graph_replay_GBs": round(b1 / (ms_graph / len(bufs) * 1e-3) / 1e9, 1),
          "graph_replay_us_per_op": round(ms_graph / len(bufs) * 1e3, 2),
          "note": "16 MiB per launch: bound by launch latency, not by HBM (an empty kernel costs 2.4 us back to back); "
                  "value = back-to-back launches through the C ABI over 40 rotating buffers (beyond the last-level cache) "
                  "with the arguments marshalled once, python_mirror = the same through the Python mirror of the op "
                  "interface (host-bound), brt_session = a ByRE module of 40 ReduceSumOp_f32_f32 ops run by the C++ session, "
                  "graph_replay = the same 40 launches replayed from one HIP graph"}
    if do_cpu:
        t1, tn = cpu_both(oracle, lambda: oracle.reduce_abc(oracle.SUM, xh, 4096, 1024, 1), n_thr, 3)
        c1.update(cpu_1core_GBs=round(b1 / t1 / 1e9, 3), cpu_allcore_GBs=round(b1 / tn / 1e9, 3), cpu_cores=n_thr)
    all_cfg["c1_row_sum"] = c1
    del bufs, xh

    # c3: fused softmax bf16 [32768, 4096] ~ N(0, 4)
    xs = [mk((32768, 4096), B16, _lib.FILL_NORMAL, SEED["c3"] + (i << 32), 0.0, 2.0) for i in range(3)]
    ys = torch.empty_like(xs[0])
    b3 = 2 * 32768 * 4096 * 2
    rows = 1024  # the oracle's share: 1024 of the 32768 rows (gate and CPU sample)
    xh = oracle.fill(2, oracle.NORMAL, SEED["c3"], rows * 4096, 0.0, 2.0).reshape(rows, 4096)
    ops.softmax(xs[0], out=ys)
    got = oracle.from_bf16_bits(ys[:rows].view(torch.int16).cpu().numpy().view(np.uint16))
    want = oracle.from_bf16_bits(oracle.softmax(xh))
    gate(np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + 1e-38), "c3 softmax (1 bf16 ulp against the float oracle)")
    j = [0]

    def c3():
        j[0] = (j[0] + 1) % 3
        ops.softmax(xs[j[0]], out=ys)

    # The copy ceiling is measured here, interleaved with the softmax: a plain copy kernel (one
    # 128-bit load and store per lane) of the same tensors, region by region in alternation, so
    # that both see the same box, clock and memory state.
    K3 = _lib.kernels()
    sp3 = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def cp():
        j[0] = (j[0] + 1) % 3
        _lib.check(K3.brt_rocm_copy_kernel(ys.data_ptr(), xs[j[0]].data_ptr(), b3 // 2, sp3))

    r3s, rcs = [], []
    for _ in range(3):
        r3s.append(time_regions(ev, [c3], 100, warm, regions=1))
        rcs.append(time_regions(ev, [cp], 100, warm, regions=1))
    ops.softmax(xs[0], out=ys)  # leave ys holding the softmax again
    merge = lambda rs: {"ms": statistics.median(r["ms"] for r in rs), "min_ms": min(r["ms"] for r in rs), "max_ms": max(r["ms"] for r in rs),
                        "regions": len(rs), "iters": rs[0]["iters"], "clock": rs[0]["clock"]}
    r3, rcp = merge(r3s), merge(rcs)
    ms3, msc = r3["ms"], rcp["ms"]
    copy_gbs = b3 / (msc * 1e-3) / 1e9
    c3r = {"value": round(b3 / (ms3 * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_op": round(ms3 * 1e3, 2),
           "frac_of_hbm_peak": round(b3 / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           **spread(r3),
           "copy_kernel_same_tensors": {"value": round(copy_gbs, 1), "unit": "GB/s", **spread(rcp)},
           "frac_of_copy_kernel_ceiling": round(msc / ms3, 4),
           "roofline": roof("hbm", "softmax_split_kernel<__bf16, 4, true>", b3, "bytes", ms3, HBM_PEAK_GBS,
                            "event pair around 100 back-to-back launches over 3 rotating inputs, median of three regions"),
           "note": "copy_kernel_same_tensors is a plain 256 MiB -> 256 MiB copy (one 128-bit load and store per lane) timed in "
                   "alternation with the softmax in this run: equal parts of reads and writes do not reach the 7.0 TB/s of a pure read stream"}
    if do_cpu:
        t1, tn = cpu_both(oracle, lambda: oracle.softmax(xh), n_thr)
        c3r.update(cpu_1core_GBs=round(2 * rows * 4096 * 2 / t1 / 1e9, 3), cpu_allcore_GBs=round(2 * rows * 4096 * 2 / tn / 1e9, 3),
                   cpu_cores=n_thr, cpu_sample="1024 rows")
    all_cfg["c3_softmax_bf16"] = c3r
    del xs, ys, xh

    def head_slice(code, seed, b, s, h, d, rows=None):
        """Host copy of batch 0, head 0 of a [b, s, h, d] tensor (storage bits), rows = slice."""
        t = oracle.fill(code, oracle.NORMAL, seed, s * h * d, 0.0, 1.0).reshape(1, s, h, d)[:, :, :1]
        t = t.view(np.float16) if code == 1 else t
        return np.ascontiguousarray(t if rows is None else t[:, rows])

    # What a matrix-instruction stream reaches on this box: nothing but v_mfma_f32_32x32x16 on
    # operands held in registers, once on zeros (the issue peak at the boost clock) and once on
    # N(0,1) operands like the attention inputs (the chip lowers its clock under the toggling
    # operand bits).  The second is the ceiling for any kernel that is fed such data.
    mf_blocks, mf_iters = torch.cuda.get_device_properties(0).multi_processor_count, 8000
    mf_ops = torch.empty(mf_blocks * 512 * 256, dtype=torch.uint8, device="cuda")
    mf_sink = torch.empty(mf_blocks * 512, dtype=F, device="cuda")
    mf_flop = mf_blocks * 8 * mf_iters * 16 * 32768
    sp_m = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    mfma_rate = {}
    for name, code, dt in (("f16", 1, H), ("bf16", 2, B16)):
        view = mf_ops.view(dt)
        probe = lambda: _lib.check(K3.brt_rocm_mfma_rate_probe(code, mf_ops.data_ptr(), mf_ops.numel(), mf_sink.data_ptr(),
                                                                mf_sink.numel() * 4, mf_blocks, mf_iters, sp_m))
        for what in ("zeros", "normal"):
            if what == "zeros":
                view.zero_()
            else:
                ops.fill(view, _lib.FILL_NORMAL, SEED["c4q"], 0.0, 1.0)
            prewarm(probe, 0.3)
            r = time_regions(ev, [probe], 5, 1)
            mfma_rate[f"{name}_{what}"] = with_clock({"value": round(mf_flop / (r["ms"] * 1e-3) / 1e12, 1), "unit": "TFLOP/s"}, r, MFMA_PEAK_TFLOPS, "frac_of_mfma_peak")
    mfma_rate["note"] = ("brt_rocm_mfma_rate_probe: 16 independent v_mfma_f32_32x32x16 per iteration and wave, 2 waves per SIMD, operands in registers, "
                         f"{mf_blocks} workgroups x {mf_iters} iterations per launch; 'normal' = operands ~ N(0,1) as the attention inputs are")
    all_cfg["mfma_rate_probe"] = mfma_rate
    del mf_ops, mf_sink

    def of_probe(entry, key):
        entry["frac_of_mfma_rate_on_normal_operands"] = round(entry["value"] / mfma_rate[key]["value"], 4)
        return entry

    # c4: flash-attention forward fp16 causal b4 h32 s2048 d128
    q, k, v = (mk((4, 2048, 32, 128), H, _lib.FILL_NORMAL, SEED[n], 0.0, 1.0) for n in ("c4q", "c4k", "c4v"))
    sc4 = 1.0 / np.sqrt(128.0)
    fl4 = 4 * 4 * 32 * 2048 * 2048 * 128 // 2  # 137 438 953 472
    fwd_out = (torch.empty_like(q), torch.empty((4, 32, 2048), device="cuda"), torch.zeros(2, dtype=torch.int64, device="cuda"))
    c4_fwd = lambda: ops.flash_attn_fwd(q, k, v, sc4, (-1, 0), out=fwd_out)
    # gate: batch 0, head 0, the last 64 query rows against the float oracle (2e-2 absolute)
    c4_fwd()
    qs, ks_, vs_ = (head_slice(1, SEED[n], 4, 2048, 32, 128) for n in ("c4q", "c4k", "c4v"))
    oracle.set_threads(n_thr)
    _, lse_ref, o32 = oracle.flash_fwd(qs[:, -64:], ks_, vs_, sc4, (-1, 0), round_p=False)
    oracle.set_threads(1)
    gate(np.abs(fwd_out[0][0, -64:, 0].float().cpu().numpy() - o32[0, :, 0]).max() <= 2e-2 and
         np.abs(fwd_out[1][0, 0, -64:].cpu().numpy() - lse_ref[0, 0]).max() <= 2e-2, "c4 flash forward O / LSE (2e-2 absolute)")
    prewarm(c4_fwd)
    r4 = time_regions(ev, [c4_fwd], 100, warm)
    ms4 = r4["ms"]
    c4 = with_clock({"value": round(fl4 / (ms4 * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "us_per_op": round(ms4 * 1e3, 1),
                     "frac_of_mfma_peak": round(fl4 / (ms4 * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "flop": fl4,
                     "roofline": roof("mfma", "flash_fwd_kernel<_Float16, 128, 1, 8, false>", fl4, "flop", ms4, MFMA_PEAK_TFLOPS,
                                      "event pair around 100 back-to-back calls, median of three regions")},
                    r4, MFMA_PEAK_TFLOPS, "frac_of_mfma_peak")
    if do_cpu:
        # the reference has no CPU attention; the naive oracle on one (batch, head) with 256
        # query rows, scaled by the flop ratio
        fl_s = 4 * 256 * (2048 - 128) * 128  # rows 1792..2047 see ~1920 keys on average
        t1, tn = cpu_both(oracle, lambda: oracle.flash_fwd(qs[:, -256:], ks_, vs_, sc4, (-1, 0)), n_thr, 1)
        c4.update(cpu_1core_TFLOPs=round(fl_s / t1 / 1e12, 6), cpu_allcore_TFLOPs=round(fl_s / tn / 1e12, 6), cpu_cores=n_thr,
                  cpu_sample="naive oracle, 1 batch x 1 head x last 256 query rows, by flop count")
    all_cfg["c4_flash_fwd_fp16_causal"] = of_probe(c4, "f16_normal")
    del q, k, v, qs, ks_, vs_

    # c5: flash-attention forward + backward bf16 non-causal b2 h16 s8192 d64
    q, k, v, do = (mk((2, 8192, 16, 64), B16, _lib.FILL_NORMAL, SEED[n], 0.0, 1.0) for n in ("c5q", "c5k", "c5v", "c5do"))
    fl5 = 4 * 2 * 16 * 8192 * 8192 * 64  # 549 755 813 888
    fwd_out = (torch.empty_like(q), torch.empty((2, 16, 8192), device="cuda"), torch.zeros(2, dtype=torch.int64, device="cuda"))
    c5_fwd = lambda: ops.flash_attn_fwd(q, k, v, 0.125, (-1, -1), out=fwd_out)
    c5_fwd()
    qs, ks_, vs_, dos = (head_slice(2, SEED[n], 2, 8192, 16, 64) for n in ("c5q", "c5k", "c5v", "c5do"))
    rows5 = slice(4096, 4096 + 32)
    oracle.set_threads(n_thr)
    _, lse_ref, o32 = oracle.flash_fwd(qs[:, rows5], ks_, vs_, 0.125, (-1, -1), round_p=False)
    gate(np.abs(fwd_out[0][0, rows5, 0].float().cpu().numpy() - o32[0, :, 0]).max() <= 2e-2 and
         np.abs(fwd_out[1][0, 0, rows5].cpu().numpy() - lse_ref[0, 0]).max() <= 2e-2, "c5 flash forward O / LSE (2e-2 absolute)")
    prewarm(c5_fwd)
    rf = time_regions(ev, [c5_fwd], 50, warm)
    msf = rf["ms"]
    o, lse = ops.flash_attn_fwd(q, k, v, 0.125, (-1, -1))
    bwd_out = ops.flash_attn_bwd_buffers(q, k, v)
    c5_bwd = lambda: ops.flash_attn_bwd(do, q, k, v, o, lse, 0.125, (-1, -1), out=bwd_out)
    # gate for the backward kernels: the first 1024 positions of batch 0, head 0 as a problem of
    # its own (same kernels, same head_dim and dtype; the full-size oracle would take minutes)
    n5 = 1024
    tq, tk, tv, tdo = (torch.from_numpy(np.ascontiguousarray(t[:, :n5]).view(np.int16)).cuda().view(torch.bfloat16) for t in (qs, ks_, vs_, dos))
    to_, tlse = ops.flash_attn_fwd(tq, tk, tv, 0.125, (-1, -1))
    gq, gk, gv = ops.flash_attn_bwd(tdo, tq, tk, tv, to_, tlse, 0.125, (-1, -1))
    rq, rk, rv, _ = oracle.flash_bwd(dos[:, :n5], qs[:, :n5], ks_[:, :n5], vs_[:, :n5], to_.view(torch.int16).cpu().numpy().view(np.uint16),
                                     tlse.cpu().numpy(), 0.125, (-1, -1), round_p=False)
    oracle.set_threads(1)
    worst, ok = {}, True
    for n, g, r in (("dq", gq, rq), ("dk", gk, rk), ("dv", gv, rv)):
        ref = oracle.to_f32(r)
        worst[n] = float(np.abs(g.float().cpu().numpy() - ref).max())
        ok = ok and worst[n] <= 2e-2 + 2.0 ** -8 * float(np.abs(ref).max())  # + 1 bf16 ulp of the largest value stored
    gate(ok, f"c5 flash backward dq/dk/dv (2e-2 absolute + 1 bf16 ulp of the largest value): {worst}")
    prewarm(c5_bwd)
    rb = time_regions(ev, [c5_bwd], 50, 2)
    msb = rb["ms"]
    all_cfg["c5_flash_fwd_bf16"] = with_clock({
        "value": round(fl5 / (msf * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "us_per_op": round(msf * 1e3, 1),
        "frac_of_mfma_peak": round(fl5 / (msf * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "flop": fl5,
        "roofline": roof("mfma", "flash_fwd_kernel<__bf16, 64, 1, 8, false>", fl5, "flop", msf, MFMA_PEAK_TFLOPS,
                         "event pair around 50 back-to-back calls, median of three regions")}, rf, MFMA_PEAK_TFLOPS, "frac_of_mfma_peak")
    flb = fl5 * 5 // 2
    all_cfg["c5_flash_bwd_bf16"] = with_clock({
        "value": round(flb / (msb * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "us_per_op": round(msb * 1e3, 1),
        "frac_of_mfma_peak": round(flb / (msb * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "flop": flb,
        "gate_worst_abs_error": {n: round(e, 5) for n, e in worst.items()},
        "roofline": roof("mfma", "dkdv_kernel<__bf16, 64, 1> + dq_kernel<__bf16, 64> + dot_do_o_kernel<__bf16, 64> (three launches per call)",
                         fl5 * 5 // 2, "flop", msb, MFMA_PEAK_TFLOPS, "event pair around 50 back-to-back calls, median of three regions"),
        "note": "flop = 2.5 x forward (5 GEMMs); the kernels execute 7 (S and dP are recomputed by the dQ pass)"},
        rb, MFMA_PEAK_TFLOPS, "frac_of_mfma_peak")
    of_probe(all_cfg["c5_flash_fwd_bf16"], "bf16_normal")
    of_probe(all_cfg["c5_flash_bwd_bf16"], "bf16_normal")
    all_cfg["c5_flash_fwd_bwd_bf16"] = {
        "value": round((fl5 + flb) / ((msf + msb) * 1e-3) / 1e12, 1), "unit": "TFLOP/s",
        "frac_of_mfma_peak": round((fl5 + flb) / ((msf + msb) * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)}
    if do_cpu:
        # naive oracle on batch 0, head 0: 128 query rows against all 8192 keys, scaled by flops
        r128 = slice(0, 128)
        fl_s = 4 * 128 * 8192 * 64
        t1, tn = cpu_both(oracle, lambda: oracle.flash_fwd(qs[:, r128], ks_, vs_, 0.125, (-1, -1)), n_thr, 1)
        all_cfg["c5_flash_fwd_bf16"].update(cpu_1core_TFLOPs=round(fl_s / t1 / 1e12, 6), cpu_allcore_TFLOPs=round(fl_s / tn / 1e12, 6),
                                            cpu_cores=n_thr, cpu_sample="naive oracle, 1 batch x 1 head x 128 query rows x 8192 keys, by flop count")
        o_s = fwd_out[0][:1, r128, :1].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        lse_s = fwd_out[1][:1, :1, r128].contiguous().cpu().numpy()
        bw = lambda: oracle.flash_bwd(dos[:, r128], qs[:, r128], ks_, vs_, o_s, lse_s, 0.125, (-1, -1))
        t1, tn = cpu_both(oracle, bw, n_thr, 1)
        all_cfg["c5_flash_bwd_bf16"].update(cpu_1core_TFLOPs=round(2.5 * fl_s / t1 / 1e12, 6), cpu_allcore_TFLOPs=round(2.5 * fl_s / tn / 1e12, 6),
                                            cpu_cores=n_thr, cpu_sample="naive oracle backward, 1 batch x 1 head x 128 query rows x 8192 keys, by flop count")
    del q, k, v, do, o, lse, bwd_out, fwd_out

    # decode against a key/value cache (not a BASELINE configuration; the serving-side call of the
    # same library): one new token per sequence, fp16, 64 sequences x 8192 cached keys,
    # 32 query heads on 8 key/value heads of 128: the 2 GiB cache is read once per call
    b_, h_, hk_, sk_, d_ = 64, 32, 8, 8192, 128
    mkd = lambda shape, jj: mk(shape, H, _lib.FILL_NORMAL, SEED["dec"] + (jj << 32), 0.0, 1.0)
    qd, kc, vc, kn, vn = mkd((b_, 1, h_, d_), 0), mkd((b_, sk_, hk_, d_), 1), mkd((b_, sk_, hk_, d_), 2), mkd((b_, 1, hk_, d_), 3), mkd((b_, 1, hk_, d_), 4)
    lens = torch.full((b_,), sk_ - 1, dtype=torch.int32, device="cuda")
    dec = lambda: ops.flash_attn_kvcache(qd, kc, vc, kn, vn, lens, 1.0 / np.sqrt(d_), (-1, -1))
    rd = time_regions(ev, [dec], 50, warm)
    msd = rd["ms"]
    byt = 2 * b_ * sk_ * hk_ * d_ * 2
    all_cfg["kvcache_decode_fp16"] = {
        "value": round(byt / (msd * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_op": round(msd * 1e3, 1),
        "frac_of_hbm_peak": round(byt / (msd * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "algorithmic_bytes": byt,
        **spread(rd, 1, 1),
        "roofline": roof("hbm", "decode_kernel<_Float16, 128> (+ decode_merge_kernel)", byt, "bytes", msd, HBM_PEAK_GBS,
                         "event pair around 50 back-to-back calls, median of three regions"),
        "note": "append kernel + decode kernel per call; bytes = K and V cache rows read once"}


if __name__ == "__main__":
    main()
