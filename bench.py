#!/usr/bin/env python3
"""Benchmark of the apply-node kernel path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c5|llama|build|all]

The headline workload is the fused elementwise + reduce configuration (f16, 8192 x 8192):
one "step" runs its four apply nodes through the C-ABI kernel manager on buffers that are
already resident in HBM:
    (i)   ij,ij->ij   max(x,0) * y
    (ii)  ij->i       row max of x
    (iii) ij,i->ij    exp(x - rowmax)
    (iv)  ij->i       row sum of (iii)
`value` is algorithmic bytes per step / wall time per step (host launch cost included).
`roofline` is the dominant kernel -- node (i) -- timed with events on the launch stream.
`cpu_baseline` times the reference CPU executor's loops, ported as -O3 C with OpenMP
(oracle/es_cpu_loops.c), over the same workload on all host cores; the same loops on one
thread, the scalar interpreter and the other configurations' baselines are under
"others.cpu_baselines".  Other workloads are reported under "others", and "others.targets"
lists every numeric target with the worst measurement that answers it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
# c64 products run as fp32 products of twice the depth: real flops against the fp32 peak
PEAK_TFLOPS = {"f16": 2500.0, "f32": 157.3, "f64": 78.6, "c64": 157.3}

# HBM bytes per launch of the dominant kernel (C2 node (i)) from two rocprofv3 --pmc runs:
# FETCH_SIZE 131084.4 KiB x 1.9999 + WRITE_SIZE 131075.3 KiB x 1.0000, the factors being what
# the same counters read for a 512 MiB copy of known size.
DOMINANT_KERNEL_TRAFFIC_BYTES = 402662523

RELU_MUL = "*[ite_>=[constant{f16|0},hole|f16@0,constant{f16|0},hole|f16@0],hole|f16@1]"
EXP_SUB = "exp[+[hole|f16@0,*[constant{f16|-1},hole|f16@1]]]"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    choices=["c2", "c1", "c3", "c4", "c5", "c5opt", "llama", "copy", "mfma_peak",
                             "build", "colred", "all"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    return ap.parse_args()


class Timed:
    """Average duration of one launch site, from events recorded on the launch stream."""

    def __init__(self):
        self.pairs = []

    def record(self, fn):
        import torch

        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        self.pairs.append((a, b))

    def mean_ms(self):
        return sum(a.elapsed_time(b) for a, b in self.pairs) / max(len(self.pairs), 1)


SETTLE_MS = 40.0


def back_to_back_ms(fn, steps):
    """Average duration of `steps` launches issued one behind the other between two events.
    A pair of events around every single launch (Timed) charges each launch the idle moment
    in which the queue turns from the event packet to the kernel, some microseconds that
    weigh on a kernel of 30 or 50 us; rows that carry both say so."""
    import torch

    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / max(steps, 1)


def with_back_to_back(row, fn, steps, nbytes):
    ms = back_to_back_ms(fn, steps)
    row["ms_back_to_back"] = round(ms, 5)
    row["hbm_frac_back_to_back"] = round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)
    return row


def warm(fn, steps):
    """Untimed warm-up of the workloads reported under "others": `steps` calls, then more
    until SETTLE_MS of wall time have gone by.  The device's clocks need some tens of
    milliseconds of load to settle: the f32 2048^3 product runs at 105 TFLOP/s over its first
    60 launches after an idle moment and at 127 TFLOP/s from about the 150th on."""
    import torch

    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def c2_nodes(n):
    import einsummable_amd as ea

    E = ea.Einsummable
    return [
        ("relu_mul ij,ij->ij", E([n, n], [[0, 1], [0, 1]], 2, RELU_MUL), 3 * n * n * 2),
        ("rowmax ij->i", E([n, n], [[0, 1]], 1, "hole|f16@0", "^"), n * n * 2 + n * 2),
        ("exp_sub ij,i->ij", E([n, n], [[0, 1], [0]], 2, EXP_SUB), 2 * n * n * 2 + n * 2),
        ("rowsum ij->i", E([n, n], [[0, 1]], 1, "hole|f16@0", "+"), n * n * 2 + n * 2),
    ]


def run_c2(km, steps, warmup):
    import torch

    n = 8192
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(n, n, device="cuda", dtype=torch.float16, generator=g)
    y = torch.randn(n, n, device="cuda", dtype=torch.float16, generator=g)
    z = torch.empty_like(x)
    ex = torch.empty_like(x)
    m = torch.empty(n, device="cuda", dtype=torch.float16)
    s = torch.empty(n, device="cuda", dtype=torch.float16)
    nodes = c2_nodes(n)
    for _, e, _ in nodes:
        assert km.build(e) == 0
    stream = torch.cuda.current_stream().cuda_stream
    calls = [
        lambda: km(nodes[0][1], stream, z.data_ptr(), [x.data_ptr(), y.data_ptr()]),
        lambda: km(nodes[1][1], stream, m.data_ptr(), [x.data_ptr()]),
        lambda: km(nodes[2][1], stream, ex.data_ptr(), [x.data_ptr(), m.data_ptr()]),
        lambda: km(nodes[3][1], stream, s.data_ptr(), [ex.data_ptr()]),
    ]
    timers = [Timed() for _ in calls]

    for _ in range(warmup):
        for c in calls:
            c()
    # The timed region carries events around the dominant kernel only (the first node): every
    # event pair is two more packets between dependent kernels, and the step is what is timed.
    # The other three nodes get their events in a second pass of the same steps.
    # An event recorded straight after a launch is stamped when the stream reaches it, so the
    # step closes with one more event: without it the dominant kernel's start stamp falls into
    # the tail of the step before.
    torch.cuda.synchronize()
    step_end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    for _ in range(steps):
        timers[0].record(calls[0])
        for c in calls[1:]:
            c()
        step_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    for _ in range(steps):
        calls[0]()
        for c, t in zip(calls[1:], timers[1:]):
            t.record(c)
    torch.cuda.synchronize()

    # nodes (iii) and (iv) as the one fused einsummable ab,a->a: sum_b exp(x[a,b] - m[a])
    import einsummable_amd as ea

    fused = ea.Einsummable([n, n], [[0, 1], [0]], 1, EXP_SUB, "+")
    assert km.build(fused) == 0
    t_fused = Timed()
    warm(lambda: km(fused, stream, s.data_ptr(), [x.data_ptr(), m.data_ptr()]), warmup)
    for _ in range(steps):
        t_fused.record(lambda: km(fused, stream, s.data_ptr(), [x.data_ptr(), m.data_ptr()]))
    torch.cuda.synchronize()

    total_bytes = sum(b for _, _, b in nodes)
    per_node = []
    for (name, e, nbytes), t in zip(nodes, timers):
        ms = t.mean_ms()
        per_node.append({"node": name, "kernel": km.describe(e), "bytes": nbytes,
                         "ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1),
                         "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)})
    fb, fms = n * n * 2 + 2 * n * 2, t_fused.mean_ms()
    per_node.append({"node": "(iii)+(iv) fused ij,i->i sum exp(x-rowmax) [not part of the step]",
                     "kernel": km.describe(fused), "bytes": fb, "ms": round(fms, 5),
                     "GBps": round(fb / fms / 1e6, 1),
                     "hbm_frac": round(fb / fms / 1e6 / HBM_PEAK_GBPS, 4)})
    return {"wall_s": wall, "bytes_per_step": total_bytes, "per_node": per_node,
            "tensors": (x, y, m)}


def cpu_loops_c2(threads, reps):
    """The four C2 nodes through the -O3 / AVX2 / OpenMP loops of oracle/es_cpu_loops.c (a port
    of the reference CPU executor's loops, kernel_executor.cc:786-914, 1163-1253) over the
    whole 8192 x 8192 configuration: seconds per step."""
    import numpy as np

    import oracle

    n = 8192
    r = np.random.default_rng(0)
    x = r.standard_normal((n, n), dtype=np.float32).astype(np.float16)
    y = r.standard_normal((n, n), dtype=np.float32).astype(np.float16)

    def step():
        oracle.loops_relu_mul(x, y, threads)
        m = oracle.loops_rowmax(x, threads)
        ex = oracle.loops_exp_sub(x, m, threads)
        oracle.loops_rowsum(ex, threads)

    step()
    t0 = time.perf_counter()
    for _ in range(reps):
        step()
    return (time.perf_counter() - t0) / reps


def cpu_baseline_c2():
    """The reported CPU baseline of the headline configuration: the reference CPU executor's
    loops as -O3 C (kind "port") on all host cores, whole workload."""
    import oracle

    n = 8192
    cores = oracle.cpu_loops().es_cpu_max_threads()
    dt = cpu_loops_c2(0, 3)
    nbytes = n * n * 2 * (3 + 1 + 2 + 1) + 3 * n * 2
    return {"value": round(nbytes / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "all four nodes over all 8192 rows, -O3 AVX2/F16C loops with OpenMP over "
                      "rows, mean of 3 steps of %.3f s" % dt}


def cpu_interpreter_c2(rows=512):
    """The CPU oracle (a single-threaded C restatement of the reference's scalar interpreter,
    every fp16 operation rounded in software) on the first `rows` rows of the same four nodes."""
    import numpy as np

    import oracle

    n = 8192
    r = np.random.RandomState(0)
    x = r.normal(0, 1, (rows, n)).astype(np.float16)
    y = r.normal(0, 1, (rows, n)).astype(np.float16)
    t0 = time.perf_counter()
    oracle.einsummable([rows, n], [[0, 1], [0, 1]], 2, RELU_MUL, None, [x, y], oracle.EXACT)
    m = oracle.einsummable([rows, n], [[0, 1]], 1, "hole|f16@0", "^", [x], oracle.EXACT)
    ex = oracle.einsummable([rows, n], [[0, 1], [0]], 2, EXP_SUB, None, [x, m], oracle.EXACT)
    oracle.einsummable([rows, n], [[0, 1]], 1, "hole|f16@0", "+", [ex], oracle.EXACT)
    dt = time.perf_counter() - t0
    nbytes = rows * n * 2 * (3 + 1 + 2 + 1) + 3 * rows * 2
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "first %d of 8192 rows of the four nodes through the scalar interpreter, "
                      "%.1f s" % (rows, dt)}


def cpu_baselines_other_configs():
    """Bounded samples of the other configurations on the host: the CPU oracle on one core
    (kind "port") and, for the f32 matmul, the host BLAS behind torch.matmul on all the
    threads torch uses (the reference's CPU manager calls MKL's sgemm there,
    kernel_executor.cc:1293-1449).  A few seconds in all."""
    import numpy as np
    import torch

    import oracle

    out = {}
    r = np.random.RandomState(1)
    cores = oracle.cpu_loops().es_cpu_max_threads()
    # C2 again: the loops on one thread (what one apply node of the reference gets), and the
    # scalar interpreter
    n2 = 8192
    c2_bytes = n2 * n2 * 2 * (3 + 1 + 2 + 1) + 3 * n2 * 2
    dt = cpu_loops_c2(1, 1)
    out["c2_loops_1_thread"] = {"value": round(c2_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": 1,
                                "kind": "port", "sample": "all four nodes, all rows, %.2f s" % dt}
    out["c2_interpreter"] = cpu_interpreter_c2()
    # C3a through the row-copy loop, whole tensor, one thread and all cores
    rg = np.random.default_rng(1)
    xa = rg.standard_normal((32, 2048, 32, 128), dtype=np.float32).astype(np.float16)
    for label, threads in (("1_thread", 1), ("all_cores", 0)):
        oracle.loops_permute_acbd(xa[:2], threads)
        t0 = time.perf_counter()
        oracle.loops_permute_acbd(xa, threads)
        dt = time.perf_counter() - t0
        out["c3a_loops_" + label] = {"value": round(2 * xa.nbytes / dt / 1e9, 2), "unit": "GB/s",
                                     "cores": threads or cores, "kind": "port",
                                     "sample": "whole 32x2048x32x128 permute, %.3f s" % dt}
    del xa
    # C3b: all 64 touches through the row loop
    accl = np.zeros((4096, 4096), np.float16)
    blks = [rg.standard_normal((512, 512), dtype=np.float32).astype(np.float16) for _ in range(8)]
    offl = [(int(r.randint(0, 3585)), int(r.randint(0, 3585))) for _ in range(64)]
    for label, threads in (("1_thread", 1), ("all_cores", 0)):
        t0 = time.perf_counter()
        for _ in range(5):
            for k, (ro, co) in enumerate(offl):
                oracle.loops_touch_add(accl, blks[k % 8], ro, co, threads)
        dt = (time.perf_counter() - t0) / 5
        out["c3b_loops_" + label] = {"value": round(64 * 3 * 512 * 512 * 2 / dt / 1e9, 2),
                                     "unit": "GB/s", "cores": threads or cores, "kind": "port",
                                     "sample": "all 64 touches, mean of 5, %.4f s" % dt}
    # f16 contractions on the host: fp32 GEMM on up-converted inputs (the reference's
    # cblas_hgemm path is not available here), LLaMA projection 2048 x 4096 x 4096
    pa = torch.from_numpy(rg.standard_normal((2048, 4096), dtype=np.float32))
    pb = torch.from_numpy(rg.standard_normal((4096, 4096), dtype=np.float32))
    torch.matmul(pa, pb.t())
    t0 = time.perf_counter()
    for _ in range(3):
        torch.matmul(pa, pb.t())
    dt = (time.perf_counter() - t0) / 3
    out["f16_projection_host_blas_fp32"] = {
        "value": round(2 * 2048 * 4096 * 4096 / dt / 1e12, 4), "unit": "TFLOP/s",
        "cores": torch.get_num_threads(), "kind": "host_blas",
        "sample": "2048x4096x4096 ij,kj->ik as fp32 on the host BLAS, %.3f s" % dt}
    del pa, pb
    # C1: 64 of the 2048 rows of A through the oracle; the whole product through the BLAS
    n, rows = 2048, 64
    A = r.uniform(-1, 1, (n, n)).astype(np.float32)
    B = r.uniform(-1, 1, (n, n)).astype(np.float32)
    t0 = time.perf_counter()
    oracle.einsummable([rows, n, n], [[0, 2], [2, 1]], 2, "*[hole|f32@0,hole|f32@1]", "+",
                       [A[:rows].copy(), B], oracle.EXACT)
    dt = time.perf_counter() - t0
    out["c1_oracle"] = {"value": round(2 * rows * n * n / dt / 1e12, 5), "unit": "TFLOP/s",
                        "cores": 1, "kind": "port",
                        "sample": "%d of 2048 rows of A, %.1f s" % (rows, dt)}
    ta, tb = torch.from_numpy(A), torch.from_numpy(B)
    torch.matmul(ta, tb)
    t0 = time.perf_counter()
    for _ in range(3):
        torch.matmul(ta, tb)
    dt = (time.perf_counter() - t0) / 3
    out["c1_host_blas"] = {"value": round(2 * n ** 3 / dt / 1e12, 4), "unit": "TFLOP/s",
                           "cores": torch.get_num_threads(), "kind": "host_blas",
                           "sample": "whole 2048^3 product, torch.matmul on the host, %.3f s" % dt}
    # C3a: 2 of the 32 outer slices of the permute
    a, b, c, d = 2, 2048, 32, 128
    x = r.normal(0, 1, a * b * c * d).astype(np.float16)
    t0 = time.perf_counter()
    oracle.einsummable([a, c, b, d], [[0, 2, 1, 3]], 4, "hole|f16@0", None, [x], oracle.EXACT)
    dt = time.perf_counter() - t0
    out["c3a_oracle"] = {"value": round(2 * x.nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": 1,
                         "kind": "port", "sample": "2 of 32 outer slices, %.1f s" % dt}
    # C3b: all 64 touches
    nn, blk = 4096, 512
    acc = np.zeros((nn, nn), np.float16)
    blocks = [r.normal(0, 1, (blk, blk)).astype(np.float16) for _ in range(8)]
    offs = [(int(r.randint(0, nn - blk + 1)), int(r.randint(0, nn - blk + 1))) for _ in range(64)]
    t0 = time.perf_counter()
    for k, (ro, co) in enumerate(offs):
        oracle.touch([(blk, nn, 0, ro, blk), (blk, nn, 0, co, blk)], "+", acc, blocks[k % 8])
    dt = time.perf_counter() - t0
    out["c3b_oracle"] = {"value": round(64 * 3 * blk * blk * 2 / dt / 1e9, 4), "unit": "GB/s",
                         "cores": 1, "kind": "port", "sample": "all 64 touches, %.2f s" % dt}
    # C4: the scores contraction of one of the 128 (batch, head) pairs, 128 of its 2048 rows
    s, dd, si = 2048, 128, 128
    Q = r.normal(0, 1, (si, dd)).astype(np.float16)
    K = r.normal(0, 1, (s, dd)).astype(np.float16)
    t0 = time.perf_counter()
    oracle.einsummable([si, s, dd], [[0, 2], [1, 2]], 2, "*[hole|f16@0,hole|f16@1]", "+", [Q, K],
                       oracle.EXACT)
    dt = time.perf_counter() - t0
    out["c4_scores_oracle"] = {"value": round(2 * si * s * dd / dt / 1e12, 6), "unit": "TFLOP/s",
                               "cores": 1, "kind": "port",
                               "sample": "128 of 2048 rows of one of 128 heads, %.1f s" % dt}
    return out


def run_contraction(km, name, e, shapes, dtype, flops, steps, warmup, yardstick=None):
    import torch

    tdt = {"f16": torch.float16, "f32": torch.float32, "f64": torch.float64,
           "c64": torch.complex64}[dtype]
    g = torch.Generator(device="cuda").manual_seed(1)
    ins = [torch.randn(*s, device="cuda", dtype=tdt, generator=g) for s in shapes[:-1]]
    out = torch.empty(*shapes[-1], device="cuda", dtype=tdt)
    ws = km.build(e)
    if ws is None:
        return {"node": name, "error": "unsupported"}
    wbuf = torch.empty(max(ws, 1), device="cuda", dtype=torch.uint8)
    if not km.describe(e).startswith("contraction"):
        # generated fallback kernel (no matrix-core path for this form): keep the run short
        if flops > 5e10:
            return {"node": name, "kernel": km.describe(e), "skipped": "fallback kernel"}
        steps, warmup = min(steps, 2), 1
    stream = torch.cuda.current_stream().cuda_stream
    call = lambda: km(e, stream, out.data_ptr(), [t.data_ptr() for t in ins],
                      (wbuf.data_ptr(), ws) if ws else None)
    warm(call, warmup)
    t = Timed()
    for _ in range(steps):
        t.record(call)
    torch.cuda.synchronize()
    ms = t.mean_ms()
    tf = flops / ms / 1e9
    row = {"node": name, "kernel": km.describe(e), "flop": flops, "ms": round(ms, 5),
           "TFLOPs": round(tf, 2), "mfma_frac": round(tf / PEAK_TFLOPS[dtype], 4)}
    nbytes = sum(t_.numel() * t_.element_size() for t_ in ins) + out.numel() * out.element_size()
    row["hbm_frac"] = round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)
    if yardstick is not None:
        # the vendor library's GEMM (torch.matmul -> hipBLASLt) on the same operands, as a
        # yardstick only: nothing here calls it outside this measurement
        fn = lambda: yardstick(*ins)
        warm(fn, warmup)
        t = Timed()
        for _ in range(steps):
            t.record(fn)
        torch.cuda.synchronize()
        row["torch_matmul_TFLOPs"] = round(flops / t.mean_ms() / 1e9, 2)
    return row


def run_c1(km, steps, warmup):
    import einsummable_amd as ea

    n = 2048
    e = ea.Einsummable([n, n, n], [[0, 2], [2, 1]], 2, "*[hole|f32@0,hole|f32@1]", "+")
    return run_contraction(km, "c1 ij,jk->ik f32 2048^3", e, [(n, n), (n, n), (n, n)], "f32",
                           2 * n ** 3, steps, warmup)


def run_c3(km, steps, warmup):
    import numpy as np
    import torch

    import einsummable_amd as ea

    out = []
    # (a) abcd->acbd of a [32, 2048, 32, 128] f16 tensor
    a, b, c, d = 32, 2048, 32, 128
    e = ea.Einsummable([a, c, b, d], [[0, 2, 1, 3]], 4, "hole|f16@0")
    x = torch.randn(a, b, c, d, device="cuda", dtype=torch.float16)
    y = torch.empty(a, c, b, d, device="cuda", dtype=torch.float16)
    assert km.build(e) == 0
    stream = torch.cuda.current_stream().cuda_stream
    call = lambda: km(e, stream, y.data_ptr(), [x.data_ptr()])
    warm(call, warmup)
    t = Timed()
    for _ in range(steps):
        t.record(call)
    torch.cuda.synchronize()
    nbytes = 2 * x.numel() * 2
    ms = t.mean_ms()
    out.append(with_back_to_back(
        {"node": "c3a permute abcd->acbd f16 32x2048x32x128", "kernel": km.describe(e),
         "bytes": nbytes, "ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1),
         "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}, call, steps, nbytes))
    del x, y
    # (a') a permute that changes the innermost mode (not part of the configuration; shows the
    # LDS-tiled transpose): ba->ab of an 8192 x 8192 f16 matrix
    n2 = 8192
    e = ea.Einsummable([n2, n2], [[1, 0]], 2, "hole|f16@0")
    x = torch.randn(n2, n2, device="cuda", dtype=torch.float16)
    y = torch.empty_like(x)
    assert km.build(e) == 0
    call = lambda: km(e, stream, y.data_ptr(), [x.data_ptr()])
    warm(call, warmup)
    t = Timed()
    for _ in range(steps):
        t.record(call)
    torch.cuda.synchronize()
    nbytes = 2 * x.numel() * 2
    ms = t.mean_ms()
    out.append(with_back_to_back(
        {"node": "transpose ba->ab f16 8192x8192", "kernel": km.describe(e),
         "bytes": nbytes, "ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1),
         "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}, call, steps, nbytes))
    del x, y
    # (b) 64 accumulate touches of 512x512 into random windows of a zeroed 4096x4096 matrix
    n, blk, count = 4096, 512, 64
    r = np.random.RandomState(0)
    acc = torch.zeros(n, n, device="cuda", dtype=torch.float16)
    blocks = [torch.randn(blk, blk, device="cuda", dtype=torch.float16) for _ in range(count)]
    touches = []
    for _ in range(count):
        ro, co = int(r.randint(0, n - blk + 1)), int(r.randint(0, n - blk + 1))
        touches.append(ea.Touch([(blk, n, 0, ro, blk), (blk, n, 0, co, blk)], "+", ea.F16))

    def all_touches():
        for tch, bl in zip(touches, blocks):
            km.touch(tch, stream, acc.data_ptr(), bl.data_ptr())

    warm(all_touches, warmup)
    t = Timed()
    for _ in range(steps):
        t.record(all_touches)
    torch.cuda.synchronize()
    nbytes = count * 3 * blk * blk * 2
    ms = t.mean_ms()
    out.append({"node": "c3b 64 touch(add) 512x512 into 4096x4096 f16", "bytes": nbytes,
                "ms": round(ms, 5), "GBps": round(nbytes / ms / 1e6, 1),
                "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
                "note": "one launch per touch, as the reference's engine issues them"})
    # the same 64 touches handed over as one group (one launch per 32 touches, same bits)
    batch = ea.TouchBatch(touches)
    ptrs = [bl.data_ptr() for bl in blocks]
    call = lambda: km.touch_batch(batch, stream, acc.data_ptr(), ptrs)
    warm(call, warmup)
    t = Timed()
    for _ in range(steps):
        t.record(call)
    torch.cuda.synchronize()
    ms = t.mean_ms()
    out.append(with_back_to_back(
        {"node": "c3b same 64 touches as one batch", "bytes": nbytes, "ms": round(ms, 5),
         "GBps": round(nbytes / ms / 1e6, 1),
         "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}, call, steps, nbytes))
    return out


def c4_nodes(b, h, s, d):
    """Batched attention as the apply nodes the reference's graph would hold: scores, the
    1/sqrt(d) scale with the constant as the reference writes it (6 significant digits, then
    fp16), the row softmax as four scalarop / reduce nodes, and P.V.  Returns
    (name, einsummable, out buffer, input buffers, work, unit)."""
    import einsummable_amd as ea

    E = ea.Einsummable
    mul = "*[hole|f16@0,hole|f16@1]"
    rows, flops = b * h * s, 2 * b * h * s * s * d
    mat = rows * s * 2
    return [
        ("scores bhid,bhjd->bhij", E([b, h, s, s, d], [[0, 1, 2, 4], [0, 1, 3, 4]], 4, mul, "+"),
         "S", ["Q", "K"], flops, "flop"),
        ("scale a->a", E([rows * s], [[0]], 1, "*[constant{f16|0.0883789},hole|f16@0]"),
         "S", ["S"], 2 * mat, "B"),
        ("rowmax ab->a", E([rows, s], [[0, 1]], 1, "hole|f16@0", "^"), "m", ["S"],
         mat + rows * 2, "B"),
        ("exp_sub ab,a->ab", E([rows, s], [[0, 1], [0]], 2, EXP_SUB), "S", ["S", "m"],
         2 * mat + rows * 2, "B"),
        ("rowsum ab->a", E([rows, s], [[0, 1]], 1, "hole|f16@0", "+"), "l", ["S"],
         mat + rows * 2, "B"),
        ("div ab,a->ab", E([rows, s], [[0, 1], [0]], 2, "*[hole|f16@0,power{-1}[hole|f16@1]]"),
         "S", ["S", "l"], 2 * mat + rows * 2, "B"),
        ("values bhij,bhjd->bhid", E([b, h, s, d, s], [[0, 1, 2, 4], [0, 1, 4, 3]], 4, mul, "+"),
         "O", ["S", "V"], flops, "flop"),
    ]


def c4_fused_nodes(b, h, s, d):
    """The same attention with the scale folded into the scores contraction (the constant
    multiplies the fp32 sums before the one rounding to fp16) and the softmax in the fused
    forms the reference's GPU manager special-cases (gpu_kernel_manager.cc:327-336, 377-405):
    row max, ab,a->a sum exp(x - m), ab,a,a->ab exp(x - m) / l.  Five nodes, 4 GiB of softmax
    traffic at the full size instead of 6 plus the 2 GiB of the scale node."""
    import einsummable_amd as ea

    E = ea.Einsummable
    full = c4_nodes(b, h, s, d)
    rows, flops = b * h * s, 2 * b * h * s * s * d
    mat = rows * s * 2
    return [
        ("scores, scale folded in", E([b, h, s, s, d], [[0, 1, 2, 4], [0, 1, 3, 4]], 4,
                                      "*[constant{f16|0.0883789},*[hole|f16@0,hole|f16@1]]", "+"),
         "S", ["Q", "K"], flops, "flop"),
        full[2],
        ("sum exp(x - m) ab,a->a", E([rows, s], [[0, 1], [0]], 1, EXP_SUB, "+"), "l", ["S", "m"],
         mat + 2 * rows * 2, "B"),
        ("exp(x - m) / l ab,a,a->ab",
         E([rows, s], [[0, 1], [0], [0]], 2,
           "*[exp[+[hole|f16@0,*[constant{f16|-1},hole|f16@1]]],power{-1}[hole|f16@2]]"),
         "S", ["S", "m", "l"], 2 * mat + 2 * rows * 2, "B"),
        full[6],
    ]


def run_c4(km, steps, warmup):
    """C4: b=4, h=32, s=2048, d=128, f16 with fp32 accumulation.  The elementwise nodes write
    over their first input (the engine donates it), so the 1 GiB score tensor exists once."""
    import torch

    b, h, s, d = 4, 32, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(4)
    mem = {k: torch.randn(b, h, s, d, device="cuda", dtype=torch.float16, generator=g)
           for k in ("Q", "K", "V")}
    mem["S"] = torch.empty(b, h, s, s, device="cuda", dtype=torch.float16)
    mem["O"] = torch.empty(b, h, s, d, device="cuda", dtype=torch.float16)
    mem["m"] = torch.empty(b * h * s, device="cuda", dtype=torch.float16)
    mem["l"] = torch.empty(b * h * s, device="cuda", dtype=torch.float16)
    nodes = c4_nodes(b, h, s, d)
    for _, e, *_r in nodes:
        assert km.build(e) == 0
    stream = torch.cuda.current_stream().cuda_stream
    calls = [lambda e=e, o=o, i=i: km(e, stream, mem[o].data_ptr(), [mem[x].data_ptr() for x in i])
             for _, e, o, i, _w, _u in nodes]
    timers = [Timed() for _ in calls]
    warm(lambda: [c() for c in calls], warmup)
    for _ in range(steps):
        for c, t in zip(calls, timers):
            t.record(c)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        for c in calls:
            c()
    torch.cuda.synchronize()
    chain_ms = (time.perf_counter() - t0) / steps * 1e3
    rows = []
    for (name, e, _o, _i, work, unit), t in zip(nodes, timers):
        ms = t.mean_ms()
        r = {"node": "c4 " + name, "kernel": km.describe(e), "ms": round(ms, 5)}
        if unit == "flop":
            # both attention products are bound by HBM (1 GiB of scores written / read for
            # 137 GFLOP): operand + result bytes over the time is the fraction that counts
            nbytes = sum(mem[x].numel() * 2 for x in _i) + mem[_o].numel() * 2
            r.update(flop=work, TFLOPs=round(work / ms / 1e9, 2),
                     mfma_frac=round(work / ms / 1e9 / PEAK_TFLOPS["f16"], 4), bytes=nbytes,
                     GBps=round(nbytes / ms / 1e6, 1),
                     hbm_frac=round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4))
        else:
            r.update(bytes=work, GBps=round(work / ms / 1e6, 1),
                     hbm_frac=round(work / ms / 1e6 / HBM_PEAK_GBPS, 4))
        rows.append(r)
    rows.append({"node": "c4 whole chain (7 nodes, no per-node events)", "ms": round(chain_ms, 4)})
    # The same chain with the scale folded into the scores contraction (one node fewer and
    # one pass over the 1 GiB score tensor less): the constant multiplies the fp32 sums
    # before the single rounding to fp16.
    import einsummable_amd as ea

    folded = ea.Einsummable([b, h, s, s, d], [[0, 1, 2, 4], [0, 1, 3, 4]], 4,
                            "*[constant{f16|0.0883789},*[hole|f16@0,hole|f16@1]]", "+")
    assert km.build(folded) == 0
    first = lambda: km(folded, stream, mem["S"].data_ptr(), [mem["Q"].data_ptr(), mem["K"].data_ptr()])
    calls6 = [first] + calls[2:]
    t_first = Timed()
    warm(lambda: [c() for c in calls6], warmup)
    for _ in range(steps):
        t_first.record(first)
        for c in calls6[1:]:
            c()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        for c in calls6:
            c()
    torch.cuda.synchronize()
    chain6_ms = (time.perf_counter() - t0) / steps * 1e3
    ms = t_first.mean_ms()
    flop = nodes[0][4]
    rows.append({"node": "c4 scores with the scale folded in", "kernel": km.describe(folded),
                 "ms": round(ms, 5), "flop": flop, "TFLOPs": round(flop / ms / 1e9, 2),
                 "mfma_frac": round(flop / ms / 1e9 / PEAK_TFLOPS["f16"], 4)})
    rows.append({"node": "c4 whole chain, scale folded into the scores contraction (6 nodes)",
                 "ms": round(chain6_ms, 4)})
    # And with the softmax in the fused forms as well: five nodes.
    fused = c4_fused_nodes(b, h, s, d)
    for _, e, *_r in fused:
        assert km.build(e) == 0
    calls5 = [lambda e=e, o=o, i=i: km(e, stream, mem[o].data_ptr(), [mem[x].data_ptr() for x in i])
              for _, e, o, i, _w, _u in fused]
    t5 = [Timed() for _ in calls5]
    warm(lambda: [c() for c in calls5], warmup)
    for _ in range(steps):
        for c, t in zip(calls5, t5):
            t.record(c)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        for c in calls5:
            c()
    torch.cuda.synchronize()
    chain5_ms = (time.perf_counter() - t0) / steps * 1e3
    for (name, e, _o, _i, nbytes, _u), t in list(zip(fused, t5))[2:4]:
        ms = t.mean_ms()
        rows.append({"node": "c4 " + name, "kernel": km.describe(e), "ms": round(ms, 5),
                     "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                     "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)})
    rows.append({"node": "c4 whole chain, scale folded and softmax in the fused forms (5 nodes)",
                 "ms": round(chain5_ms, 4)})
    # The same five nodes as an exec graph over one arena, the two row statistics deleted
    # after their last reader, through the graph's optimisation pass: the softmax becomes one
    # chain over rows (each row of the 1 GiB score tensor read once and written once).
    del calls, calls5, calls6
    sizes = {k: v.numel() * 2 for k, v in mem.items()}
    offs, at = {}, 0
    for k in ("Q", "K", "V", "S", "O", "m", "l"):
        offs[k] = at
        at += (sizes[k] + 255) // 256 * 256
    arena = torch.empty(at, dtype=torch.uint8, device="cuda")
    for k in ("Q", "K", "V"):
        arena[offs[k]:offs[k] + sizes[k]] = mem[k].view(torch.uint8).reshape(-1)
    mem.clear()
    graph = ea.ApplyGraph(km)
    ids = {}
    for name, e, o, i, _w, _u in fused:
        ids[name] = graph.add_einsummable(e, [(offs[o], sizes[o])] + [(offs[x], sizes[x]) for x in i])
    last = list(ids.values())
    graph.add_dummy((offs["m"], sizes["m"]), [last[2], last[3]])
    graph.add_dummy((offs["l"], sizes["l"]), [last[3]])
    graph.add_memory_dependencies()
    absorbed = graph.optimize()
    graph.finalize(1)
    run = lambda: graph.run(stream, arena.data_ptr())
    warm(run, warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    chain3_ms = (time.perf_counter() - t0) / steps * 1e3
    t_sm = Timed()
    softmax = [n for n in range(graph.num_nodes()) if graph.describe(n).startswith("chain ")]
    if softmax:
        one = lambda: graph.launch_node(softmax[0], stream, arena.data_ptr())
        warm(one, warmup)
        for _ in range(steps):
            t_sm.record(one)
        torch.cuda.synchronize()
        ms = t_sm.mean_ms()
        nbytes = 2 * sizes["S"]
        rows.append({"node": "c4 softmax as one chain over rows (max, sum exp(x - m), exp(x - m) / l)",
                     "kernel": "row_chain", "ms": round(ms, 5), "bytes": nbytes,
                     "GBps": round(nbytes / ms / 1e6, 1),
                     "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)})
    rows.append({"node": "c4 whole chain as an optimised exec graph (%d launches)" % graph.launches(),
                 "ms": round(chain3_ms, 4), "absorbed": absorbed})
    return rows


def run_llama_contractions(km, steps, warmup):
    """The contraction nodes of one LLaMA-7B decoder layer (dim 4096, 32 heads of 128,
    ffn 11008, batch 1, seq 2048), fp16 in / fp32 accumulate, in the merged forms the
    layer's graph produces (llama/modules.cc:282-356, 410-431)."""
    import einsummable_amd as ea

    mul = "*[hole|f16@0,hole|f16@1]"
    s, d, h, hd, f = 2048, 4096, 32, 128, 11008
    E = ea.Einsummable.from_str
    cases = [
        ("qkv/o proj ij,kj->ik 2048x4096x4096", E("ij,kj->ik", dict(i=s, j=d, k=d), mul, "+"),
         [(s, d), (d, d), (s, d)], 2 * s * d * d),
        ("w1/w3 ij,kj->ik 2048x4096x11008", E("ij,kj->ik", dict(i=s, j=d, k=f), mul, "+"),
         [(s, d), (f, d), (s, f)], 2 * s * d * f),
        ("w2 ij,kj->ik 2048x11008x4096", E("ij,kj->ik", dict(i=s, j=f, k=d), mul, "+"),
         [(s, f), (d, f), (s, d)], 2 * s * d * f),
        ("scores acbe,adbe->abcd", E("acbe,adbe->abcd", dict(a=1, b=h, c=s, d=s, e=hd), mul, "+"),
         [(1, s, h, hd), (1, s, h, hd), (1, h, s, s)], 2 * h * s * s * hd),
        ("values abce,aebd->abcd", E("abce,aebd->abcd", dict(a=1, b=h, c=s, e=s, d=hd), mul, "+"),
         [(1, h, s, s), (1, s, h, hd), (1, h, s, hd)], 2 * h * s * s * hd),
        ("out proj adbe,cde->abc", E("adbe,cde->abc", dict(a=1, d=h, b=s, e=hd, c=d), mul, "+"),
         [(1, h, s, hd), (d, h, hd), (1, s, d)], 2 * s * d * d),
    ]
    import torch

    nt = lambda a, b: torch.matmul(a, b.t())
    yard = [nt, nt, nt, None, None, None]
    rows = [run_contraction(km, name, e, shapes, "f16", flops, steps, warmup, y)
            for (name, e, shapes, flops), y in zip(cases, yard)]
    # the square products the tile rule and the roofline discussion refer to
    E2 = ea.Einsummable.from_str
    for n in (4096, 8192):
        rows.append(run_contraction(km, "ij,kj->ik %d^3" % n, E2("ij,kj->ik", dict(i=n, j=n, k=n), mul, "+"),
                                    [(n, n), (n, n), (n, n)], "f16", 2 * n ** 3, steps, warmup, nt))
    return rows


def run_c5(km, steps, warmup):
    """One LLaMA-7B decoder layer (dim 4096, 32 heads of 128, SwiGLU 11008, RMSNorm, rotary,
    batch 1, seq 2048, fp16, weights N(0, 0.02)) as its list of apply / touch / fill nodes,
    every node on the kernel manager, in order on one stream."""
    import numpy as np
    import torch

    from einsummable_amd.llama_layer import DeviceRunner, LayerGraph, freqs_cis_table

    g = LayerGraph()
    run = DeviceRunner(km, g)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for name, (dt, shape) in g.inputs.items():
        n = int(np.prod(shape))
        if name == "full_freqs_cis":
            run.set_input(name, freqs_cis_table(shape[0], shape[1]))
            continue
        sd = 1.0 if name == "x" else 0.02
        t = torch.randn(n, device="cuda", dtype=torch.float32, generator=gen) * sd
        if name.endswith("norm.weight"):
            t = t + 1.0
        run.mem[name].copy_(t.half().view(torch.uint8))
    warm(run.run, warmup)
    timers = [Timed() for _ in g.nodes]
    t0 = time.perf_counter()
    for _ in range(steps):
        run.run(timers=timers)
    torch.cuda.synchronize()
    timed_wall_ms = (time.perf_counter() - t0) / steps * 1e3
    # the layer without per-node events: launched node by node, and replayed as one HIP graph
    t0 = time.perf_counter()
    for _ in range(steps):
        run.run()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) / steps * 1e3
    graph = run.capture()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    graph_ms = (time.perf_counter() - t0) / steps * 1e3
    # the same layer through the exec-node layer: one arena, dependencies from the memory
    # ranges, nodes placed on 1 / 2 / 4 streams, one burst of launches per layer
    del graph
    exec_ms, opt_ms, opt_launches, per_launch = {}, {}, {}, []
    state = {name: run.mem[name].clone() for name in g.inputs}
    for ns, optimize in ((1, False), (2, False), (4, False), (1, True), (4, True)):
        del run
        torch.cuda.empty_cache()
        run = None
        from einsummable_amd.llama_layer import ArenaRunner
        par = ArenaRunner(km, g, ns, optimize=optimize)
        for name, t in state.items():
            par.view(name).copy_(t)
        # (building a runner leaves the device idle for a while: warm() runs until the clocks
        # have settled again, or a variant is charged for the one built before it)
        warm(par.run, max(warmup, 2))
        t0 = time.perf_counter()
        for _ in range(steps):
            par.run()
        torch.cuda.synchronize()
        (opt_ms if optimize else exec_ms)[str(ns)] = round(
            (time.perf_counter() - t0) / steps * 1e3, 4)
        opt_launches["optimized" if optimize else "as_listed"] = par.graph.launches()
        if optimize and ns == 1:
            per_launch = time_graph_nodes(par, max(steps // 2, 5))
        run = par
    del par, run, state
    rows = []
    for n, t in zip(g.nodes, timers):
        rows.append((n["label"], n["kind"], t.mean_ms(), n.get("flops", 0)))
    gemm_ms = sum(ms for _, _, ms, fl in rows if fl)
    top = sorted(rows, key=lambda r: -r[2])[:12]
    return {"node": "c5 LLaMA-7B decoder layer, b=1 s=2048 f16", "layer_ms": round(wall_ms, 4),
            "layer_hipgraph_ms": round(graph_ms, 4),
            "layer_exec_graph_ms_by_streams": exec_ms,
            # formation copies absorbed, single-reader elementwise nodes merged into their
            # readers; every range still written holds the same bytes
            "layer_exec_graph_optimized_ms_by_streams": opt_ms,
            "exec_graph_launches": opt_launches,
            # the optimised layer launch by launch (es_km_graph_launch_node with an event pair
            # around each): what it moves or multiplies and the fraction of the bound that
            # applies; the launches' sum against the burst above is the launch gaps
            "optimized_launches": per_launch,
            "optimized_launches_sum_ms": round(sum(r["ms"] for r in per_launch), 4),
            "layer_with_node_events_ms": round(timed_wall_ms, 4), "nodes": len(rows), "sum_node_ms": round(sum(r[2] for r in rows), 4),
            "contraction_ms": round(gemm_ms, 4),
            "contraction_TFLOPs": round(g.contraction_flops() / gemm_ms / 1e9, 1),
            "other_ms": round(sum(r[2] for r in rows) - gemm_ms, 4),
            "top_nodes": [{"label": l, "ms": round(ms, 4)} for l, _, ms, _ in top]}


def time_graph_nodes(runner, steps):
    """Every launching node of an ArenaRunner's graph, one at a time through
    es_km_graph_launch_node, timed with an event pair."""
    import torch

    g = runner.graph
    stream = torch.cuda.current_stream().cuda_stream
    ids = [i for i in range(g.num_nodes()) if g.node_mems(i)[0] != "dummy"]
    ws_bytes = max([g.node_workspace(i) for i in ids] + [1])
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    arena = runner.arena.data_ptr()
    timers = {i: Timed() for i in ids}

    def one_pass(timed):
        for i in ids:
            call = lambda i=i: g.launch_node(i, stream, arena, (ws.data_ptr(), ws_bytes))
            if timed:
                timers[i].record(call)
            else:
                call()

    for _ in range(3):
        one_pass(False)
    for _ in range(steps):
        one_pass(True)
    torch.cuda.synchronize()
    rows = []
    for i in ids:
        kind, mems = g.node_mems(i)
        text = g.describe(i)
        ms = timers[i].mean_ms()
        nbytes = sum(size for _, size in mems)
        row = {"node": text.split(" | ", 1)[1] if " | " in text else kind, "kind": kind,
               "ms": round(ms, 5), "bytes": nbytes}
        flop = 0
        if kind == "einsummable":
            key = text.split(" | ")[1]
            shape = [int(x) for x in key[key.index("[") + 1:key.index("]")].split(",")]
            join = text.split(" | ")[2]
            product = join.count("hole|") == 2 and join.startswith("*[") and "+[" not in join
            if key[key.index("]") + 1] == "+" and product:
                flop = 2
                for d in shape:
                    flop *= d
        intensity = flop / max(nbytes, 1)
        if flop and intensity >= 150:
            row.update(flop=flop, bound="mfma",
                       frac=round(flop / ms / 1e9 / PEAK_TFLOPS["f16"], 4))
        else:
            if flop:
                row["flop"] = flop
            row.update(bound="hbm", frac=round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4))
        rows.append(row)
    return rows


def run_c5opt(km, steps, warmup):
    """The optimised LLaMA-7B layer alone (for a kernel trace of exactly its launches)."""
    import numpy as np
    import torch

    from einsummable_amd.llama_layer import ArenaRunner, LayerGraph, freqs_cis_table

    g = LayerGraph()
    par = ArenaRunner(km, g, 1, optimize=True)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for name, (dt, shape) in g.inputs.items():
        n = int(np.prod(shape))
        if name == "full_freqs_cis":
            par.set_input(name, freqs_cis_table(shape[0], shape[1]))
            continue
        t = torch.randn(n, device="cuda", dtype=torch.float32, generator=gen) * (1.0 if name == "x" else 0.02)
        if name.endswith("norm.weight"):
            t = t + 1.0
        par.view(name).copy_(t.half().view(torch.uint8))
    warm(par.run, max(warmup, 2))
    t0 = time.perf_counter()
    for _ in range(steps):
        par.run()
    torch.cuda.synchronize()
    return {"node": "c5 optimised layer, one stream", "launches": par.graph.launches(),
            "layer_ms": round((time.perf_counter() - t0) / steps * 1e3, 4)}


def run_mfma_peak(km):
    """fp16 matrix-core throughput with operands in registers (no memory traffic at all): the
    ceiling a GEMM can approach on this device, for zero and for random operand bits."""
    import torch

    out = {}
    stream = torch.cuda.current_stream().cuda_stream
    blocks = 1024
    scratch = torch.empty(blocks * 256, device="cuda", dtype=torch.float32)
    for label, ops in (("zeros", torch.zeros(4096, device="cuda", dtype=torch.float16)),
                       ("random", torch.rand(4096, device="cuda", dtype=torch.float16) - 0.5)):
        best = 0.0
        for _ in range(3):
            best = max(best, km.probe_mfma_f16(ops.data_ptr(), scratch.data_ptr(), blocks, 20000,
                                               stream))
        out[label + "_TFLOPs"] = round(best, 1)
    out["published_peak_TFLOPs"] = PEAK_TFLOPS["f16"]
    return out


def run_read_ceiling(km, steps, warmup):
    """A kernel that only reads, on memory nobody has just written: the generated row max
    over 1 GiB of f16 next to the vendor library's reduction (torch.amax) over the same
    tensor.  Inside the attention chain the same kernel on the same shape is slower, because
    there its input has just been written by the preceding node."""
    import torch

    import einsummable_amd as ea

    rows, n = 262144, 2048
    x = torch.randn(rows, n, device="cuda", dtype=torch.float16)
    m = torch.empty(rows, device="cuda", dtype=torch.float16)
    e = ea.Einsummable([rows, n], [[0, 1]], 1, "hole|f16@0", "^")
    assert km.build(e) == 0
    stream = torch.cuda.current_stream().cuda_stream
    ours, lib = Timed(), Timed()
    call = lambda: km(e, stream, m.data_ptr(), [x.data_ptr()])
    warm(call, warmup)
    for _ in range(steps):
        ours.record(call)
    call = lambda: torch.amax(x, dim=1, out=m)
    warm(call, warmup)
    for _ in range(steps):
        lib.record(call)
    torch.cuda.synchronize()
    nbytes = rows * n * 2 + rows * 2
    return {"bytes": nbytes, "es_rowmax_GBps": round(nbytes / ours.mean_ms() / 1e6, 1),
            "torch_amax_GBps": round(nbytes / lib.mean_ms() / 1e6, 1)}


def run_col_reductions(km, steps, warmup):
    """Reductions whose aggregated mode is not the innermost one (column sums and the like):
    few outputs and a long aggregation run as two passes over a workspace."""
    import torch

    import einsummable_amd as ea

    E = ea.Einsummable
    cases = [
        ("ab->b 8192x8192 f16 add", E([8192, 8192], [[1, 0]], 1, "hole|f16@0", "+"),
         8192 * 8192, 8192, torch.float16),
        ("ab->b 65536x1024 f32 add", E([1024, 65536], [[1, 0]], 1, "hole|f32@0", "+"),
         65536 * 1024, 1024, torch.float32),
        ("abc->ac 64x2048x1024 f16 max", E([64, 1024, 2048], [[0, 2, 1]], 2, "hole|f16@0", "^"),
         64 * 2048 * 1024, 64 * 1024, torch.float16),
    ]
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for name, e, n_in, n_out, dt in cases:
        ws = km.build(e)
        w = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda")
        x = torch.randn(n_in, device="cuda", dtype=dt)
        y = torch.empty(n_out, device="cuda", dtype=dt)
        t = Timed()
        call = lambda: km(e, stream, y.data_ptr(), [x.data_ptr()],
                          (w.data_ptr(), ws) if ws else None)
        warm(call, warmup)
        for _ in range(steps):
            t.record(call)
        torch.cuda.synchronize()
        nbytes = (n_in + n_out) * x.element_size()
        rows.append(with_back_to_back(
            {"node": name, "kernel": km.describe(e), "workspace_bytes": ws,
             "bytes": nbytes, "ms": round(t.mean_ms(), 5),
             "GBps": round(nbytes / t.mean_ms() / 1e6, 1),
             "hbm_frac": round(nbytes / t.mean_ms() / 1e6 / HBM_PEAK_GBPS, 4)}, call, steps, nbytes))
    return rows


def run_copy(km, steps, warmup):
    """A plain copy of known size (1-D touch without castable, 512 MiB in, 512 MiB out): the
    yardstick the FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    import torch

    import einsummable_amd as ea

    n = 1 << 28
    x = torch.randn(n, device="cuda", dtype=torch.float16)
    y = torch.empty_like(x)
    t = ea.Touch([(n, n, 0, 0, n)], None, ea.F16)
    stream = torch.cuda.current_stream().cuda_stream
    call = lambda: km.touch(t, stream, y.data_ptr(), x.data_ptr())
    warm(call, warmup)
    tm = Timed()
    for _ in range(steps):
        tm.record(call)
    torch.cuda.synchronize()
    nbytes = 2 * n * 2
    ms = tm.mean_ms()
    return {"node": "copy 2^28 f16", "bytes": nbytes, "ms": round(ms, 5),
            "GBps": round(nbytes / ms / 1e6, 1),
            "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}


BUILD_PROBE = r"""
import json, sys, time
sys.path.insert(0, %r)
import torch
import einsummable_amd as ea
from einsummable_amd.llama_layer import ArenaRunner, LayerGraph
mode = %r
torch.cuda.init()
km = ea.KernelManager(0)
g = LayerGraph()
n = len([1 for node in g.nodes if node["kind"] == "einsummable"])
t0 = time.perf_counter()
if mode == "graph":
    # the exec graph builds its distinct einsummables together (es_km_graph_finalize)
    ArenaRunner(km, g, n_streams=1)
elif mode == "optimized":
    # the same through the optimisation pass: merged einsummables and chains over rows are
    # planned by the pass and compiled at finalize, as one program each
    ArenaRunner(km, g, n_streams=1, optimize=True)
else:
    for node in g.nodes:
        if node["kind"] == "einsummable":
            km.build(node["e"])
print(json.dumps({"ms": (time.perf_counter() - t0) * 1e3, "einsummables": n}))
"""


def run_build_latency():
    """Time to build the einsummables of the LLaMA-7B layer (runtime compilation of the
    generated kernels is most of it): through the exec graph, which builds a graph's
    distinct einsummables on several threads, in a fresh process with an empty code-object
    cache and again in a second process that finds the cache filled; and one build() call
    after the other (the reference's call pattern) in a third process with an empty cache."""
    import shutil
    import subprocess
    import tempfile

    root = os.path.dirname(os.path.abspath(__file__))
    out = {}
    runs = [("first_process_empty_cache", "graph", 0), ("second_process_cache_on_disk", "graph", 0),
            ("one_build_call_after_the_other_empty_cache", "serial", 1),
            ("optimized_graph_first_process_empty_cache", "optimized", 2)]
    caches = [tempfile.mkdtemp(prefix="es_km_cache_") for _ in range(3)]
    try:
        for label, mode, which in runs:
            env = dict(os.environ, ES_KM_CACHE_DIR=caches[which])
            p = subprocess.run([sys.executable, "-c", BUILD_PROBE % (root, mode)], env=env,
                               capture_output=True, text=True, timeout=600)
            if p.returncode != 0:
                out[label] = {"error": p.stderr[-300:]}
                continue
            r = json.loads(p.stdout.strip().splitlines()[-1])
            out[label] = {"build_ms": round(r["ms"], 1), "einsummables": r["einsummables"]}
        out["code_objects_cached"] = len([f for f in os.listdir(caches[0]) if f.endswith(".co")])
    finally:
        for c in caches:
            shutil.rmtree(c, ignore_errors=True)
    return out


def targets_block(others):
    """Every numeric target with the measurements that answer it, worst first, so that the
    line cannot be read as its headline alone."""
    mfma, hbm = [], []
    for r in others.get("llama7b_contractions", []):
        if "mfma_frac" not in r:
            continue
        # arithmetic intensity below 150 flop per byte (attention's scores and values): the
        # HBM bound applies (the planner's own rule for giving a product the small tile)
        nbytes = r["hbm_frac"] * HBM_PEAK_GBPS * 1e6 * r["ms"]
        if r["flop"] / max(nbytes, 1.0) < 150.0:
            hbm.append((r["hbm_frac"], r["node"]))
        else:
            mfma.append((r["mfma_frac"], r["node"], r.get("torch_matmul_TFLOPs")))
    for key in ("c2_nodes", "c3", "c4", "column_reductions"):
        for r in others.get(key, []):
            if isinstance(r, dict) and "hbm_frac" in r and "[not part" not in r["node"]:
                hbm.append((r["hbm_frac"], r["node"]))
    for r in others.get("c5", {}).get("optimized_launches", []):
        label = "c5 optimised layer: " + r["node"][:90]
        if r["bound"] == "mfma":
            mfma.append((r["frac"], label, None))
        elif r["bytes"] >= (8 << 20):
            # (a node that moves less than 8 MiB is bound by its launch, not by memory)
            hbm.append((r["frac"], label))
    mfma.sort()
    hbm.sort()
    out = {
        "fp16_contractions_mfma_frac_target_0.60": {
            "worst": mfma[0][0] if mfma else None, "best": mfma[-1][0] if mfma else None,
            "rows": [{"node": n, "mfma_frac": f,
                      "vendor_gemm_mfma_frac": round(t / PEAK_TFLOPS["f16"], 4) if t else None}
                     for f, n, t in mfma]},
        "memory_kernels_hbm_frac_target_0.70": {
            "worst": hbm[0][0] if hbm else None,
            "below_target": [{"node": n, "hbm_frac": f} for f, n in hbm if f < 0.70],
            "at_or_above_target": len([1 for f, _ in hbm if f >= 0.70])},
    }
    if "c5" in others:
        out["llama7b_layer_ms"] = others["c5"].get("layer_ms")
        opt = others["c5"].get("layer_exec_graph_optimized_ms_by_streams") or {}
        out["llama7b_layer_exec_graph_optimized_ms_target_2.0"] = min(opt.values()) if opt else None
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures the apply-node kernels of ONE GPU; --gpus %d is not supported "
              "(an apply node never spans devices)." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch

    import einsummable_amd as ea

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.init()
    km = ea.KernelManager(0)

    if args.workload == "mfma_peak":
        print(json.dumps(run_mfma_peak(km)))
        return
    if args.workload == "copy":
        print(json.dumps(run_copy(km, args.steps, args.warmup)))
        return
    if args.workload == "c5opt":
        # nothing but the optimised layer: a kernel trace of this run lists its launches only
        print(json.dumps(run_c5opt(km, args.steps, args.warmup)))
        return

    c2 = run_c2(km, args.steps, args.warmup)
    ms_per_step = c2["wall_s"] / args.steps * 1e3
    value = c2["bytes_per_step"] / (c2["wall_s"] / args.steps) / 1e9
    dom = max(c2["per_node"][:4], key=lambda p: p["bytes"])
    roofline = {"bound": "hbm", "kernel": dom["node"] + " [" + dom["kernel"] + "]",
                "achieved": dom["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
                "traffic": DOMINANT_KERNEL_TRAFFIC_BYTES}
    others = {"c2_nodes": c2["per_node"]}
    del c2
    torch.cuda.empty_cache()
    if args.workload in ("c1", "all"):
        others["c1"] = run_c1(km, args.steps, args.warmup)
    if args.workload in ("c1", "all"):
        # the same matmul in the other two dtypes the reference sends to its BLAS
        # (cublasDgemm / cublasCgemm, gpu_kernel_manager.cc:1543-1558); no configuration
        # uses them, they are here so that the paths have a number
        import einsummable_amd as ea
        n = 2048
        rows = []
        for dt, flop in (("f64", 2 * n ** 3), ("c64", 8 * n ** 3)):
            for spec, inns in (("ij,jk->ik", [[0, 2], [2, 1]]), ("ij,kj->ik", [[0, 2], [1, 2]])):
                e = ea.Einsummable([n, n, n], inns, 2, "*[hole|%s@0,hole|%s@1]" % (dt, dt), "+")
                yard = (lambda a, b: torch.matmul(a, b)) if spec == "ij,jk->ik" else \
                       (lambda a, b: torch.matmul(a, b.t()))
                rows.append(run_contraction(km, "%s %s 2048^3" % (spec, dt), e,
                                            [(n, n), (n, n), (n, n)], dt, flop,
                                            max(args.steps // 5, 3), max(args.warmup // 5, 1), yard))
        others["f64_c64_matmuls"] = rows
    if args.workload in ("c3", "all"):
        others["c3"] = run_c3(km, args.steps, args.warmup)
    if args.workload in ("c4", "all"):
        others["c4"] = run_c4(km, max(args.steps // 5, 3), max(args.warmup // 5, 1))
    if args.workload in ("c5", "all"):
        torch.cuda.empty_cache()
        others["c5"] = run_c5(km, max(args.steps // 5, 3), max(args.warmup // 5, 1))
        torch.cuda.empty_cache()
    if args.workload == "all":
        others["mfma_f16_register_ceiling"] = run_mfma_peak(km)
        others["read_only_1GiB"] = run_read_ceiling(km, args.steps, args.warmup)
    if args.workload in ("colred", "all"):
        others["column_reductions"] = run_col_reductions(km, args.steps, args.warmup)
    if args.workload == "all" and not args.no_cpu_baseline:
        others["cpu_baselines"] = cpu_baselines_other_configs()
    if args.workload in ("llama", "all"):
        others["llama7b_contractions"] = run_llama_contractions(km, max(args.steps // 5, 3),
                                                                max(args.warmup // 5, 1))
    if args.workload in ("build", "all"):
        others["build_latency_llama7b_layer"] = run_build_latency()
    others["targets"] = targets_block(others)

    line = {
        "metric": "elementwise/reduce GB/s (apply-node kernel path; contraction TFLOP/s and "
                  "touch/permute GB/s under 'others')",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "C2 fused elementwise + reduce, f16 8192x8192: max(x,0)*y; "
                               "row max; exp(x-rowmax); row sum"},
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline_c2(),
        "others": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
