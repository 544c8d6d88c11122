#!/usr/bin/env python3
"""Benchmark of the op-kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-extras] [--pmc-probe]

Prints ONE JSON line.  The headline workload (`config.workload`) is the second of the benchmark configurations the repository's BASELINE.json lists:
ReduceMaxOp_f32_f32 and ReduceSumOp_f32_f32 over axis 0 (column / two-pass split case) and over
axis 1 of one [16384, 8192] float tensor; a "step" is those four op-kernel launches, `value` is
the algorithmic bytes of a step divided by the step time, inputs resident in HBM.  The other
listed configurations (row sum, fused softmax, flash-attention forward and backward) are
timed in the same run and reported under `all_configs`, each with its own roofline fraction and
a CPU figure.

Timing: HIP events recorded on the stream the kernels are launched on (through the library's
own C ABI, not torch's event wrapper), plus a host clock around the synchronised region.
Everything is launched through the C ABI (libbrt_rocm_kernels.so / libflash_attn.so); torch is
used for device memory, streams and random input only.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 / fp16 MFMA, published

# measured HBM bytes of one first-pass launch: 536 894 846 fetched + 4 194 304 written
TRAFFIC_COL_FIRST_PASS = 541089150

METRIC = "reduce HBM GB/s + flash-attn fwd/bwd TFLOP/s, % of MI355X roofline, 1 GPU"


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


def time_ops(ev, fns, steps, warmup):
    """Run `fns` (a list of launch closures = one step) `warmup` + `steps` times.
    -> (ms per step by events, [ms per launch of fns[i]], ms per step by host clock).
    The step time comes from ONE pair of events around all `steps` steps (an event between every
    two launches costs a few microseconds of idle GPU each); the per-launch breakdown is taken
    in a second pass of the same length with an event after every launch."""
    import torch
    for _ in range(warmup):
        for f in fns:
            f()
    torch.cuda.synchronize()
    e0, e1 = ev.new(), ev.new()
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
    if len(fns) == 1:
        return total, [total], host_ms
    marks = [[ev.new() for _ in range(len(fns) + 1)] for _ in range(steps)]
    for s in range(steps):
        ev.record(marks[s][0])
        for i, f in enumerate(fns):
            f()
            ev.record(marks[s][i + 1])
    torch.cuda.synchronize()
    per = [sum(ev.elapsed_ms(marks[s][i], marks[s][i + 1]) for s in range(steps)) / steps
           for i in range(len(fns))]
    for m in marks:
        ev.free(m)
    return total, per, host_ms


def prewarm(fn, seconds=0.08):
    """Run `fn` back to back for about `seconds` of wall time.  After idle time (or after
    memory-bound kernels) the matrix-heavy attention kernels run 15-20 % slower for their first
    ~100 launches (~30 ms) while the clocks ramp; the timed region should see the steady state."""
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=["c2"])
    ap.add_argument("--no-extras", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter-collection mode: one copy kernel of known size, then two steps")
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
    gen = torch.Generator(device="cuda")

    # ---- headline: C2, [16384, 8192] f32 ~ U(-1, 1) --------------------------------------
    R, Cc = 16384, 8192
    NBUF = 3  # rotate inputs: 1.5 GiB between two touches of a buffer, beyond the 256 MB LLC
    gen.manual_seed(0xC2)
    xs = [torch.rand((R, Cc), generator=gen, device="cuda") * 2 - 1 for _ in range(NBUF)]
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
        qd = torch.randn((b_, 1, h_, d_), generator=gen, device="cuda").half()
        kc, vc = (torch.randn((b_, sk_, hk_, d_), generator=gen, device="cuda").half() for _ in range(2))
        kn, vn = (torch.randn((b_, 1, hk_, d_), generator=gen, device="cuda").half() for _ in range(2))
        lens = torch.full((b_,), sk_ - 1, dtype=torch.int32, device="cuda")
        for _ in range(2):
            ops.flash_attn_kvcache(qd, kc, vc, kn, vn, lens, 1.0 / np.sqrt(d_), (-1, -1))
        torch.cuda.synchronize()
        print(json.dumps({"pmc_probe": True, "copy_bytes_read": in_bytes, "copy_bytes_written": in_bytes,
                          "decode_cache_bytes": 2 * b_ * sk_ * hk_ * d_ * 2}))
        return

    ms_step, per, host_ms = time_ops(ev, c2_fns, args.steps, args.warmup)
    value = step_bytes / (ms_step * 1e-3) / 1e9
    col_ms = (per[0] + per[1]) / 2
    row_ms = (per[2] + per[3]) / 2
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
    roofline = {
        "bound": "hbm", "kernel": "reduce_colwide_kernel<float, float, OP, 4, 2, 2> (first pass of the axis-0 split reduction)",
        "achieved": round(col_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(col_gbs / HBM_PEAK_GBS, 4),
        "algorithmic_bytes_per_launch": bytes_col, "avg_launch_us": round(pass1_ms * 1e3, 2),
        "op_us_including_combine_pass": round(col_ms * 1e3, 2), "combine_pass_us": round(p2_ms * 1e3, 2),
        # FETCH_SIZE + WRITE_SIZE per first-pass dispatch from two rocprofv3 --pmc runs, each
        # scaled by the same counter's reading for a 512 MiB copy kernel (profiles/)
        "traffic": TRAFFIC_COL_FIRST_PASS,
    }
    col_op_gbs = bytes_col / (col_ms * 1e-3) / 1e9

    result = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "host_ms_per_step": round(host_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "c2: ReduceMaxOp_f32_f32 + ReduceSumOp_f32_f32 over axis 0 and over axis 1 "
                               "of [16384, 8192] f32 ~ U(-1,1) (4 op-kernel launches per step, "
                               f"{NBUF} rotating input buffers)",
                   "algorithmic_bytes_per_step": step_bytes},
        "roofline": roofline,
    }

    all_cfg = {
        "c2a_col_max_sum_axis0": {"value": round(col_op_gbs, 1), "unit": "GB/s", "us_per_op": round(col_ms * 1e3, 2),
                                  "frac_of_hbm_peak": round(col_op_gbs / HBM_PEAK_GBS, 4),
                                  "first_pass_kernel_GBs": round(col_gbs, 1)},
        "c2b_row_max_sum_axis1": {"value": round(bytes_row / (row_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                                  "us_per_op": round(row_ms * 1e3, 2),
                                  "frac_of_hbm_peak": round(bytes_row / (row_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
    }

    # ---- CPU baseline for the headline workload --------------------------------------------
    if not args.no_cpu:
        import oracle
        oracle.set_threads(1)
        xh = xs[0].cpu().numpy()
        t_cpu = cpu_time(lambda: (oracle.reduce_abc(oracle.MAX, xh, 1, R, Cc), oracle.reduce_abc(oracle.SUM, xh, 1, R, Cc),
                                  oracle.reduce_abc(oracle.MAX, xh, R, Cc, 1), oracle.reduce_abc(oracle.SUM, xh, R, Cc, 1)),
                         repeat=2)
        result["cpu_baseline"] = {
            "value": round(step_bytes / t_cpu / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "the full step (4 reductions of the [16384, 8192] tensor) run once per repeat, best of 2, "
                      "by the scalar loop-nest oracle (the reference's CPU path is single-threaded LLVM-JIT'ed "
                      "loop nests, which cannot be built here)",
            "seconds": round(t_cpu, 3), "host_cores_available": os.cpu_count(),
        }
        # the same loop nests with OpenMP over the independent outputs, on this job's CPU share
        n_thr = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        oracle.set_threads(n_thr)
        t_par = cpu_time(lambda: (oracle.reduce_abc(oracle.MAX, xh, 1, R, Cc), oracle.reduce_abc(oracle.SUM, xh, 1, R, Cc),
                                  oracle.reduce_abc(oracle.MAX, xh, R, Cc, 1), oracle.reduce_abc(oracle.SUM, xh, R, Cc, 1)),
                         repeat=2)
        oracle.set_threads(1)
        result["cpu_baseline"]["openmp"] = {"value": round(step_bytes / t_par / 1e9, 3), "unit": "GB/s", "cores": n_thr,
                                            "seconds": round(t_par, 3)}
        del xh

    if not args.no_extras:
        extras(all_cfg, ev, ops, _lib, gen, args, np, torch)
    result["all_configs"] = all_cfg
    print(json.dumps(result))


def extras(all_cfg, ev, ops, _lib, gen, args, np, torch):
    """The remaining benchmark configurations, timed with the same event machinery."""
    import oracle
    steps, warm = max(5, args.steps // 2), max(2, args.warmup // 2)
    do_cpu = not args.no_cpu

    # c1: row ReduceSum f32 [4096, 1024] ~ N(0,1).  16 MiB: launch-bound; rotating 40 buffers
    # (640 MiB) keeps the input out of the 256 MB LLC ("cold"), one buffer gives the warm figure.
    gen.manual_seed(0xC1)
    bufs = [torch.randn((4096, 1024), generator=gen, device="cuda") for _ in range(40)]
    o1 = torch.empty(4096, device="cuda")
    b1 = 4096 * 1024 * 4 + 4096 * 4
    i = [0]

    def c1_cold():
        i[0] = (i[0] + 1) % len(bufs)
        ops.reduce_abc(_lib.REDUCE_SUM, bufs[i[0]], o1, 4096, 1024, 1)

    ms_cold, _, _ = time_ops(ev, [c1_cold] * 10, steps, warm)
    ms_warm, _, _ = time_ops(ev, [lambda: ops.reduce_abc(_lib.REDUCE_SUM, bufs[0], o1, 4096, 1024, 1)] * 10, steps, warm)
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
    ms_graph, _, _ = time_ops(ev, [graph.replay], steps, warm)
    c1 = {"value": round(b1 / (ms_cold / 10 * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_op": round(ms_cold / 10 * 1e3, 2),
          "frac_of_hbm_peak": round(b1 / (ms_cold / 10 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
          "warm_cache_GBs": round(b1 / (ms_warm / 10 * 1e-3) / 1e9, 1), "warm_us_per_op": round(ms_warm / 10 * 1e3, 2),
          "graph_replay_GBs": round(b1 / (ms_graph / len(bufs) * 1e-3) / 1e9, 1),
          "graph_replay_us_per_op": round(ms_graph / len(bufs) * 1e3, 2),
          "note": "16 MiB per launch: bound by launch latency, not by HBM; value = back-to-back launches from the "
                  "host over 40 rotating buffers, graph_replay = the same 40 launches replayed from one HIP graph"}
    if do_cpu:
        xh = bufs[0].cpu().numpy()
        t = cpu_time(lambda: oracle.reduce_abc(oracle.SUM, xh, 4096, 1024, 1), 3)
        c1["cpu_1core_GBs"] = round(b1 / t / 1e9, 3)
    all_cfg["c1_row_sum"] = c1
    del bufs

    # c3: fused softmax bf16 [32768, 4096] ~ N(0, 4)
    gen.manual_seed(0xC3)
    xs = [(torch.randn((32768, 4096), generator=gen, device="cuda") * 2).bfloat16() for _ in range(3)]
    ys = torch.empty_like(xs[0])
    b3 = 2 * 32768 * 4096 * 2
    j = [0]

    def c3():
        j[0] = (j[0] + 1) % 3
        ops.softmax(xs[j[0]], out=ys)

    ms3, _, _ = time_ops(ev, [c3], steps, warm)
    c3r = {"value": round(b3 / (ms3 * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_op": round(ms3 * 1e3, 2),
           "frac_of_hbm_peak": round(b3 / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if do_cpu:
        rows = 1024  # bounded sample: 1024 of the 32768 rows, scaled
        xh = xs[0][:rows].view(torch.int16).cpu().numpy().view(np.uint16)
        t = cpu_time(lambda: oracle.softmax(xh), 2)
        c3r["cpu_1core_GBs"] = round(2 * rows * 4096 * 2 / t / 1e9, 3)
        c3r["cpu_sample"] = "1024 rows"
    all_cfg["c3_softmax_bf16"] = c3r
    del xs, ys

    # c4: flash-attention forward fp16 causal b4 h32 s2048 d128
    gen.manual_seed(0xC4)
    q, k, v = (torch.randn((4, 2048, 32, 128), generator=gen, device="cuda").half() for _ in range(3))
    sc4 = 1.0 / np.sqrt(128.0)
    fl4 = 4 * 4 * 32 * 2048 * 2048 * 128 // 2  # 137 438 953 472
    fwd_out = (torch.empty_like(q), torch.empty((4, 32, 2048), device="cuda"), torch.zeros(2, dtype=torch.int64, device="cuda"))
    c4_fwd = lambda: ops.flash_attn_fwd(q, k, v, sc4, (-1, 0), out=fwd_out)
    prewarm(c4_fwd)
    ms4, _, _ = time_ops(ev, [c4_fwd], steps, warm)
    c4 = {"value": round(fl4 / (ms4 * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "us_per_op": round(ms4 * 1e3, 1),
          "frac_of_mfma_peak": round(fl4 / (ms4 * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "flop": fl4}
    if do_cpu:
        # the reference has no CPU attention; the naive oracle on one (batch, head) with 256
        # query rows, scaled by the flop ratio
        qs, ks_, vs_ = (t[:1, :, :1].cpu().numpy() for t in (q, k, v))
        t = cpu_time(lambda: oracle.flash_fwd(qs[:, -256:], ks_, vs_, sc4, (-1, 0)), 1)
        fl_s = 4 * 256 * (2048 - 128) * 128  # rows 1792..2047 see ~1920 keys on average
        c4["cpu_1core_TFLOPs"] = round(fl_s / t / 1e12, 6)
        c4["cpu_sample"] = "1 batch x 1 head x last 256 query rows"
    all_cfg["c4_flash_fwd_fp16_causal"] = c4
    del q, k, v

    # c5: flash-attention forward + backward bf16 non-causal b2 h16 s8192 d64
    gen.manual_seed(0xC5)
    q, k, v, do = (torch.randn((2, 8192, 16, 64), generator=gen, device="cuda").bfloat16() for _ in range(4))
    fl5 = 4 * 2 * 16 * 8192 * 8192 * 64  # 549 755 813 888
    fwd_out = (torch.empty_like(q), torch.empty((2, 16, 8192), device="cuda"), torch.zeros(2, dtype=torch.int64, device="cuda"))
    c5_fwd = lambda: ops.flash_attn_fwd(q, k, v, 0.125, (-1, -1), out=fwd_out)
    prewarm(c5_fwd)
    msf, _, _ = time_ops(ev, [c5_fwd], steps, warm)
    o, lse = ops.flash_attn_fwd(q, k, v, 0.125, (-1, -1))
    bwd_out = ops.flash_attn_bwd_buffers(q, k, v)
    c5_bwd = lambda: ops.flash_attn_bwd(do, q, k, v, o, lse, 0.125, (-1, -1), out=bwd_out)
    prewarm(c5_bwd)
    msb, _, _ = time_ops(ev, [c5_bwd], max(3, steps // 3), 2)
    all_cfg["c5_flash_fwd_bf16"] = {
        "value": round(fl5 / (msf * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "us_per_op": round(msf * 1e3, 1),
        "frac_of_mfma_peak": round(fl5 / (msf * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "flop": fl5}
    flb = fl5 * 5 // 2
    all_cfg["c5_flash_bwd_bf16"] = {
        "value": round(flb / (msb * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "us_per_op": round(msb * 1e3, 1),
        "frac_of_mfma_peak": round(flb / (msb * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4), "flop": flb,
        "note": "flop = 2.5 x forward (5 GEMMs); the kernels execute 7 (S and dP are recomputed by the dQ pass)"}
    all_cfg["c5_flash_fwd_bwd_bf16"] = {
        "value": round((fl5 + flb) / ((msf + msb) * 1e-3) / 1e12, 1), "unit": "TFLOP/s",
        "frac_of_mfma_peak": round((fl5 + flb) / ((msf + msb) * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)}
    del q, k, v, do, o, lse, bwd_out, fwd_out

    # decode against a key/value cache (not a BASELINE configuration; the serving-side call of the
    # same library): one new token per sequence, fp16, 64 sequences x 8192 cached keys,
    # 32 query heads on 8 key/value heads of 128: the 2 GiB cache is read once per call
    b_, h_, hk_, sk_, d_ = 64, 32, 8, 8192, 128
    gen.manual_seed(0xDC)
    qd = torch.randn((b_, 1, h_, d_), generator=gen, device="cuda").half()
    kc, vc = (torch.randn((b_, sk_, hk_, d_), generator=gen, device="cuda").half() for _ in range(2))
    kn, vn = (torch.randn((b_, 1, hk_, d_), generator=gen, device="cuda").half() for _ in range(2))
    lens = torch.full((b_,), sk_ - 1, dtype=torch.int32, device="cuda")
    dec = lambda: ops.flash_attn_kvcache(qd, kc, vc, kn, vn, lens, 1.0 / np.sqrt(d_), (-1, -1))
    msd, _, _ = time_ops(ev, [dec], steps, warm)
    byt = 2 * b_ * sk_ * hk_ * d_ * 2
    all_cfg["kvcache_decode_fp16"] = {
        "value": round(byt / (msd * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_op": round(msd * 1e3, 1),
        "frac_of_hbm_peak": round(byt / (msd * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "algorithmic_bytes": byt,
        "note": "append kernel + decode kernel per call; bytes = K and V cache rows read once"}


if __name__ == "__main__":
    main()
