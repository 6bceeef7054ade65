#!/usr/bin/env python3
"""Benchmark of the bitmap SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--n N] [--sparsity S]

A step is one SpMM call (main kernel + split-K reduction when the library's
automatic Split_K is > 1) over one resident compressed copy of the weight
matrix.  Calls rotate over enough copies of the weights that successive steps
cannot be served from the 256 MB last-level cache.  Prints one JSON line:
dense-equivalent TFLOP/s as `value`, plus `roofline` (HBM: algorithmic bytes
over the GPU time of one whole call, with the main kernel alone and this
machine's own read-stream ceiling beside it) and `cpu_baseline` (the CPU
checker timed on this machine's host cores over a bounded row slice).
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LLC_BYTES = 256 << 20


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=2000)
    p.add_argument("--warmup", type=int, default=100)
    p.add_argument("--prewarm-ms", type=float, default=120.0,
                   help="untimed calls before the warm-up steps: after idling, the first ~40 ms of calls run at ramping clocks")
    p.add_argument("--workload", default="opt30b_ffn1")
    p.add_argument("--n", type=int, default=None, help="override the workload's N")
    p.add_argument("--sparsity", type=float, default=None, help="override the workload's sparsity (0..1)")
    p.add_argument("--split-k", type=int, default=0, help="0 = the library's automatic choice")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-dense", action="store_true")
    p.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    p.add_argument("--no-qkv", action="store_true",
                   help="skip the short extra measurement of the OPT-13B fused-QKV shape (the 15360x5120 decode linear)")
    p.add_argument("--no-encoder", action="store_true", help="skip timing the device encoder on the workload's W")
    p.add_argument("--no-chain", action="store_true",
                   help="skip the OPT-13B decode-step chain (40 layers x 4 linears, sparse vs dense, same run)")
    p.add_argument("--chain-layers", type=int, default=40)
    p.add_argument("--no-stream-probe", action="store_true",
                   help="skip the read-stream probe (spmspm_amd/lib/stream_probe) behind roofline.stream_ceiling_gbs")
    p.add_argument("--no-sweep", action="store_true",
                   help="skip the sweep over the remaining benchmark cells (OPT-30B FFN1 at four sparsities x N = 8, "
                        "16, 32; OPT-66B FFN2 at N = 64, 128; the other three OPT-13B linears)")
    p.add_argument("--sweep-steps", type=int, default=200, help="timed calls per sweep cell")
    p.add_argument("--copy-probe", action="store_true",
                   help="also run three 256 MiB device-to-device copies (a known-size reference for HBM byte counters)")
    return p.parse_args()


class Hip:
    """The few HIP runtime calls the timing needs (events on the launch stream)."""

    def __init__(self):
        self.rt = ctypes.CDLL("libamdhip64.so")
        self.rt.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.rt.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.rt.hipEventSynchronize.argtypes = [ctypes.c_void_p]
        self.rt.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.rt.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def event(self):
        e = ctypes.c_void_p()
        assert self.rt.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        assert self.rt.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value


def cpu_baseline(comp, X, seconds):
    """Time the CPU checker (decode + fp32-accumulate product, OpenMP) on a bounded slice of 64-row blocks."""
    from oracle import oracle as O
    M, K = comp.M, comp.K
    N = X.shape[0]
    nkb = K // 64

    def run(row_blocks):
        g1 = row_blocks * nkb
        off = comp.offsets[:g1 + 1]
        t0 = time.perf_counter()
        O.spmm(comp.values[:int(off[-1])], comp.bitmaps[:g1 * 64], off, X, row_blocks * 64, N, K, 1, False)
        return time.perf_counter() - t0

    probe = min(M // 64, 16)
    run(min(probe, 2))  # warm the thread pool
    t_probe = run(probe)
    blocks = int(min(M // 64, max(probe, probe * seconds / max(t_probe, 1e-6))))
    t_once = run(blocks)
    reps = max(1, int(seconds / max(t_once, 1e-6)))  # whole passes over the slice until the time target is met
    t0 = time.perf_counter()
    for _ in range(reps):
        run(blocks)
    t = (time.perf_counter() - t0) / reps
    rows = blocks * 64
    flops = 2.0 * rows * N * K
    # the reference's own CPU path is its single-threaded encoder: time our restatement of it as well
    enc_rows = min(M, 4096)
    from spmspm_amd.synthetic import make_weight
    Wenc = make_weight(enc_rows, K, 0.7, seed=1)
    t0 = time.perf_counter()
    O.encode(Wenc, enc_rows, K)
    t_enc = time.perf_counter() - t0
    ref_rate = None
    if O.ref_lib() is not None:  # the reference's own encoder, compiled from its source where that tree was present
        t0 = time.perf_counter()
        O.ref_encode(Wenc, enc_rows, K)
        ref_rate = enc_rows * K / (time.perf_counter() - t0) / 1e6
    return {
        "value": flops / t / 1e12, "unit": "TFLOP/s", "cores": O.num_threads(), "kind": "port",
        "sample": f"rows 0..{rows} of {M} (K={K}, N={N}), {reps} passes of {t:.3f} s, host decode+GEMM, OpenMP",
        "seconds_per_pass": t, "passes": reps,
        "encoder_melems_per_s_1thread": enc_rows * K / t_enc / 1e6,
        "reference_encoder_melems_per_s_1thread": ref_rate,
    }


def ramp(torch, issue, ms=40.0):
    """Keeps the GPU busy for `ms` with `issue()` (a function that queues about a millisecond of work).  After any idle
    of a few milliseconds (a host phase, the first use of a new stream, a read-back) the shader clock needs about
    20 ms of load to come back, and calls in that window take 15-20 % longer (43 us falling to 36 us per call on the
    target shape): every timed region below starts from a ramped clock, so a short run measures the same machine state
    as a long one."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < ms * 1e-3:
        issue()
        torch.cuda.synchronize()


def bound_call(L, layer, x, out, stream_handle):
    """`SpMM_SplitK_API` on one resident weight copy with every argument converted beforehand: what a C caller's loop
    costs per step.  (The Python convenience wrapper `SparseLinear.__call__` checks and converts its arguments on
    every call, 20-40 us of host time per call on these boxes: more than the GPU needs for the smaller shapes, so a
    loop over it measures the host.)"""
    import ctypes as C
    N = x.shape[0]
    sk = layer._plan(N)[0]
    ws = layer.workspace(N)
    args = (C.c_void_p(stream_handle), C.c_void_p(layer.values.data_ptr()), C.c_void_p(layer.bitmaps.data_ptr()),
            C.c_void_p(layer.offsets.data_ptr()), C.c_void_p(x.data_ptr()), C.c_void_p(out.data_ptr()),
            C.c_int(layer.M), C.c_int(N), C.c_int(layer.K), C.c_void_p(ws.data_ptr() if ws is not None else None),
            C.c_int(sk))
    fn = L.SpMM_SplitK_API

    def call():
        if fn(*args):
            raise RuntimeError("SpMM_SplitK_API failed")
    return call


def quick_measure(torch, S, hip, dev, workload, steps, warmup, seed):
    """The timing of main(), in short, for one more named workload: whole-call TFLOP/s, main-kernel GB/s and
    roofline fraction, and the dense fp16 product of the same shape in the same run."""
    from spmspm_amd.synthetic import WORKLOADS, make_activations, make_weight
    w = WORKLOADS[workload]
    M, K, N = w["M"], w["K"], w["N"]
    W = make_weight(M, K, w["sparsity"], seed=seed, pruning=w["pruning"])
    X = make_activations(K, N, seed=seed)
    comp = S.InitSparseMatrixA_bitmap(W)
    algo = comp.algorithmic_bytes(N)
    copies = max(2, -(-3 * LLC_BYTES // algo))
    first = S.SparseLinear(comp, device=dev, split_k=0)
    layers = [first] + [first.clone() for _ in range(copies - 1)]
    x = torch.from_numpy(X.view(np.int16).copy()).to(dev).view(torch.float16)
    out = torch.empty((N, M), dtype=torch.float16, device=dev)
    stream = torch.cuda.current_stream()
    L = S.library()
    calls = [bound_call(L, l, x, out, stream.cuda_stream) for l in layers]
    ramp(torch, lambda: [calls[i % copies]() for i in range(40)])
    for i in range(warmup):
        calls[i % copies]()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        calls[i % copies]()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    events = [(hip.event(), hip.event()) for _ in range(steps)]
    for i in range(steps):
        L.SpMM_TimeNextCall(events[i][0], events[i][1])
        calls[i % copies]()
    torch.cuda.synchronize()
    kern = float(np.mean([hip.elapsed_ms(e0, e1) for e0, e1 in events])) / 1e3
    for e0, e1 in events:
        hip.rt.hipEventDestroy(e0), hip.rt.hipEventDestroy(e1)
    rows = np.random.default_rng(2).choice(M, 64, replace=False)
    got = out.cpu().numpy()[:, rows].astype(np.float64)
    ref = X.astype(np.float64) @ W[rows].astype(np.float64).T
    Wd = [torch.from_numpy(W.view(np.int16)).to(dev).view(torch.float16)]
    Wd += [Wd[0].clone() for _ in range(max(2, -(-3 * LLC_BYTES // (2 * M * K))) - 1)]
    ramp(torch, lambda: [torch.matmul(x, Wd[i % len(Wd)].t()) for i in range(30)])
    t0 = time.perf_counter()
    for i in range(steps):
        torch.matmul(x, Wd[i % len(Wd)].t())
    torch.cuda.synchronize()
    td = (time.perf_counter() - t0) / steps
    flops = 2.0 * M * N * K
    return {"workload": workload, "M": M, "K": K, "N": N, "sparsity": w["sparsity"], "pruning": w["pruning"],
            "split_k": S.SpMM_SplitK_Auto(M, N, K), "tflops": flops / wall / 1e12, "us_per_call": wall * 1e6,
            "kernel_avg_us": kern * 1e6, "gbs": algo / wall / 1e9, "roofline_frac": algo / wall / 1e9 / HBM_PEAK_GBS,
            "main_kernel_gbs": algo / kern / 1e9, "main_kernel_roofline_frac": algo / kern / 1e9 / HBM_PEAK_GBS,
            "algorithmic_bytes": int(algo), "dense_fp16_us": td * 1e6, "speedup_vs_dense": td / wall,
            "rel_l2": float(np.linalg.norm(got - ref) / np.linalg.norm(ref))}


def shader_clock_mhz(torch, L, side, burst):
    """Shader clock while `burst` (a function issuing SpMM calls on the current stream for a few milliseconds) runs:
    one idling wave on a second stream compares the shader-clock counter with the constant 100 MHz counter
    (SpMM_ShaderClockProbe) for 2 ms of that time."""
    ticks = torch.zeros(2, dtype=torch.int64, device="cuda:0")
    torch.cuda.synchronize()
    burst(20)  # the load is already running when the probe starts
    if L.SpMM_ShaderClockProbe(side.cuda_stream, ticks.data_ptr(), 2000) != 0:
        return None
    burst(120)
    torch.cuda.synchronize()
    c, r = (int(v) for v in ticks.cpu())
    return 100.0 * c / r if r > 0 else None


def device_weights(torch, M, K, sparsity, pruning, seed, dev):
    """Seeded synthetic weights made on the GPU (the host generator takes seconds per matrix of this size): fp16
    N(0, 0.02), pruned with a uniform random mask or by magnitude over the whole matrix."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W = torch.empty((M, K), dtype=torch.float16, device=dev)
    rows = max(1, (1 << 25) // K)
    for r0 in range(0, M, rows):
        r1 = min(M, r0 + rows)
        W[r0:r1] = (torch.randn((r1 - r0, K), generator=g, device=dev) * 0.02).to(torch.float16)
    if pruning == "random":
        for r0 in range(0, M, rows):
            r1 = min(M, r0 + rows)
            W[r0:r1][torch.rand((r1 - r0, K), generator=g, device=dev) < sparsity] = 0
    else:
        mag = W.abs().float().reshape(-1)
        kth = int(round(sparsity * mag.numel()))
        if kth > 0:
            thresh = torch.kthvalue(mag, kth).values
            W[W.abs().float() <= thresh] = 0
        del mag
    return W


class SweepMatrix:
    """One synthetic weight matrix of the sweep, generated and encoded on the device (the device encoder's arrays
    are the host encoder's, bit for bit: tests/test_encoder_gpu.py), with enough resident copies that successive
    calls cannot be served from the last-level cache."""

    def __init__(self, torch, S, dev, M, K, sparsity, pruning, seed):
        self.M, self.K, self.sparsity, self.pruning = M, K, sparsity, pruning
        self.W = device_weights(torch, M, K, sparsity, pruning, seed, dev)
        v, b, o = S.InitSparseMatrixA_bitmap_device(self.W)
        self.nnz = int(v.numel())
        self.fixed_bytes = 2 * self.nnz + 8 * b.numel() + 4 * o.numel()
        copies = max(2, -(-3 * LLC_BYTES // self.fixed_bytes))
        self.arrays = [(v, b, o)] + [(v.clone(), b.clone(), o.clone()) for _ in range(copies - 1)]


def sweep_cell(torch, S, hip, dev, mat, N, steps, seed, name):
    """One cell of the benchmark grid (the reference harness appends one CSV row per cell,
    kernel_benchmark/spmm_test_utils.h:249-290): whole-call and main-kernel time, roofline fractions, result check."""
    M, K = mat.M, mat.K
    L = S.library()
    g = torch.Generator(device=dev)
    g.manual_seed(seed + 77)
    x = (torch.rand((N, K), generator=g, device=dev) * 2 - 1).to(torch.float16)
    out = torch.empty((N, M), dtype=torch.float16, device=dev)
    sk = S.SpMM_SplitK_Auto(M, N, K)
    need = S.SpMM_WorkspaceBytes(M, N, K, sk)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream()
    copies = len(mat.arrays)

    def call(i):
        v, b, o = mat.arrays[i % copies]
        err = S.SpMM_SplitK_API(stream, v, b, o, x, out, M, N, K, ws, sk)
        if err != 0:
            raise RuntimeError(f"sweep cell {name}: hipError_t {err}")

    ramp(torch, lambda: [call(i) for i in range(30)])
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    g0.record(stream)
    for i in range(steps):
        call(i)
    g1.record(stream)
    torch.cuda.synchronize()
    call_s = g0.elapsed_time(g1) / 1e3 / steps
    events = [(hip.event(), hip.event()) for _ in range(steps)]
    for i in range(steps):
        L.SpMM_TimeNextCall(events[i][0], events[i][1])
        call(i)
    torch.cuda.synchronize()
    kern_s = float(np.mean([hip.elapsed_ms(e0, e1) for e0, e1 in events])) / 1e3
    for e0, e1 in events:
        hip.rt.hipEventDestroy(e0), hip.rt.hipEventDestroy(e1)
    # result check: 64 sampled rows against a float64 product of the dense weights on the device
    rows = torch.from_numpy(np.random.default_rng(3).choice(M, 64, replace=False)).to(dev)
    ref = x.double() @ mat.W[rows].double().t()
    got = out[:, rows].double()
    rel_l2 = float((got - ref).norm() / ref.norm())
    max_frac = float((got - ref).abs().max() / ref.abs().max())
    if not (rel_l2 <= 1e-3 and max_frac <= 1e-2):
        raise RuntimeError(f"sweep cell {name}: outside the tolerance (rel-L2 {rel_l2:.2e}, max {max_frac:.2e})")
    algo = mat.fixed_bytes + 2 * K * N + 2 * M * N
    flops = 2.0 * M * N * K
    return {"cell": name, "M": M, "K": K, "N": N, "sparsity": mat.sparsity, "pruning": mat.pruning, "split_k": sk,
            "kernel": L.SpMM_KernelName(M, N, K, sk).decode(), "us_per_call": call_s * 1e6,
            "main_kernel_us": kern_s * 1e6, "roofline_frac": algo / call_s / 1e9 / HBM_PEAK_GBS,
            "main_kernel_roofline_frac": algo / kern_s / 1e9 / HBM_PEAK_GBS, "tflops": flops / call_s / 1e12,
            "algorithmic_bytes": int(algo), "rel_l2": rel_l2}


def sweep(torch, S, hip, dev, steps, seed):
    """The benchmark grid beyond the headline cell, each cell timed like the headline (GPU time of whole calls
    back to back from stream events; the main kernel from events on its dispatches)."""
    cells = []
    grid = [("opt30b_ffn1", 28672, 7168, s, "random", (8, 16, 32)) for s in (0.4, 0.5, 0.6, 0.7)]
    grid += [("opt66b_ffn2", 9216, 36864, 0.4, "random", (64, 128))]
    grid += [("opt13b_out", 5120, 5120, 0.6, "magnitude", (16,)), ("opt13b_ffn1", 20480, 5120, 0.6, "magnitude", (16,)),
             ("opt13b_ffn2", 5120, 20480, 0.6, "magnitude", (16,))]
    for nm, M, K, sp, pruning, widths in grid:
        mat = SweepMatrix(torch, S, dev, M, K, sp, pruning, seed)
        for N in widths:
            cells.append(sweep_cell(torch, S, hip, dev, mat, N, steps, seed, f"{nm}_s{int(round(sp * 100))}_n{N}"))
        del mat
        torch.cuda.empty_cache()
    return {"steps_per_cell": steps, "cells": cells,
            "what": "weights generated and encoded on the GPU (seeded); us_per_call = GPU time of whole calls (main "
                    "kernel + split-K reduction) back to back; roofline_frac = algorithmic bytes / that time / 8 TB/s"}


def device_encoder(torch, S, dev, W, comp, host_encode_s):
    """Times the device encoder (both calls, incl. the read-back of the value count between them) on the
    workload's dense W resident in HBM and checks its arrays against the host encoder's."""
    Wd = torch.from_numpy(W.view(np.int16)).to(dev).view(torch.float16)
    vals, bm, off = S.InitSparseMatrixA_bitmap_device(Wd)
    torch.cuda.synchronize()
    same = (np.array_equal(off.cpu().numpy(), comp.offsets) and np.array_equal(bm.cpu().numpy().view(np.uint64), comp.bitmaps)
            and np.array_equal(vals.cpu().numpy().view(np.uint16), comp.values))
    reps = 5
    t0 = time.perf_counter()
    for _ in range(reps):
        S.InitSparseMatrixA_bitmap_device(Wd)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / reps
    algo = 2 * W.size + 2 * comp.values.size + 8 * comp.bitmaps.size + 4 * comp.offsets.size
    moved = algo + 2 * W.size  # W is read twice
    # the one-pass form (W read once; values into a buffer sized beforehand, here the worst case M*K)
    room = torch.empty(W.size, dtype=torch.int16, device=dev)
    v1, b1, o1 = S.InitSparseMatrixA_bitmap_device_onepass(Wd, values=room)
    torch.cuda.synchronize()
    same1 = (np.array_equal(o1.cpu().numpy(), comp.offsets) and np.array_equal(b1.cpu().numpy().view(np.uint64), comp.bitmaps)
             and np.array_equal(v1.cpu().numpy().view(np.uint16), comp.values))
    t0 = time.perf_counter()
    for _ in range(reps):
        S.InitSparseMatrixA_bitmap_device_onepass(Wd, values=room)
    torch.cuda.synchronize()
    t1 = (time.perf_counter() - t0) / reps
    # GPU time of the entry points alone, every buffer allocated beforehand: events on the stream around `reps` calls
    L, M, K = S.library(), W.shape[0], W.shape[1]
    scratch = torch.empty(L.SpMM_EncodeDevice_ScratchBytes(M, K) // 8 + 1, dtype=torch.int64, device=dev)
    ptr = lambda x: x.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream

    def gpu_us(call):
        ramp(torch, lambda: [call() for _ in range(5)])
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            call()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    def two_calls():
        assert L.SpMM_EncodeDevice_Bitmaps(stream, ptr(Wd), M, K, ptr(b1), ptr(o1)) == 0
        assert L.SpMM_EncodeDevice_Values(stream, ptr(Wd), M, K, ptr(o1), ptr(room)) == 0

    def one_call():
        assert L.SpMM_EncodeDevice_OnePass(stream, ptr(Wd), M, K, ptr(b1), ptr(o1), ptr(room), room.numel(), ptr(scratch)) == 0

    us2, us1 = gpu_us(two_calls), gpu_us(one_call)
    del room, scratch
    return {"ms": t * 1e3, "gpu_us": us2, "identical_to_host_encoder": bool(same), "algorithmic_bytes": int(algo),
            "one_pass": {"ms": t1 * 1e3, "gpu_us": us1, "identical_to_host_encoder": bool(same1),
                         "gbs_algorithmic": algo / us1 / 1e3, "frac_of_hbm_peak": algo / us1 / 1e3 / HBM_PEAK_GBS,
                         "what": "SpMM_EncodeDevice_OnePass: W read once, offsets by look-back between workgroups; ms = "
                                 "wall time of the Python call incl. its allocations, scratch clear and the read-back of "
                                 "the count; gpu_us = GPU time of the entry point alone (stream events), which the rates "
                                 "are taken from"},
            "gbs_algorithmic": algo / us2 / 1e3, "gbs_moved": moved / us2 / 1e3, "frac_of_hbm_peak": algo / us2 / 1e3 / HBM_PEAK_GBS,
            "host_encoder_ms": host_encode_s * 1e3, "host_threads": os.cpu_count(),
            "what": "dense fp16 W in HBM -> bitmaps, offsets, values in HBM; W read once = algorithmic, read twice = moved; "
                    "ms = wall time of the Python call (two entry points, two allocations, the read-back of the count "
                    "between them); gpu_us = GPU time of the two entry points back to back, which the rates are taken from"}


def decode_chain(torch, S, dev, layers, seed):
    """OPT-13B decode step, linears only: `layers` x {QKV, out, FFN1, FFN2} at N=16, every layer with weight
    copies of its own, chained on one stream (FFN2's output feeds the next layer's QKV; the attention between QKV
    and the output projection is not run, its result is a fixed buffer).  Timed eagerly and as a replayed HIP
    graph, for the compressed weights and for dense fp16 weights (torch.matmul) in the same run."""
    from spmspm_amd.synthetic import WORKLOADS, make_weight
    N = 16
    names = ["opt13b_qkv", "opt13b_out", "opt13b_ffn1", "opt13b_ffn2"]
    first, dense0, info = [], [], []
    for i, nm in enumerate(names):
        w = WORKLOADS[nm]
        W = make_weight(w["M"], w["K"], w["sparsity"], seed=seed + 11 * i, pruning=w["pruning"])
        comp = S.InitSparseMatrixA_bitmap(W)
        first.append(S.SparseLinear(comp, device=dev, split_k=0))
        dense0.append(torch.from_numpy(W.view(np.int16)).to(dev).view(torch.float16))
        info.append({"name": nm, "M": w["M"], "K": w["K"], "sparsity": w["sparsity"],
                     "split_k": S.SpMM_SplitK_Auto(w["M"], N, w["K"]), "bytes": comp.algorithmic_bytes(N)})
        del W, comp
    sparse = [[l if j == 0 else l.clone() for l in first] for j in range(layers)]
    dense = [[d if j == 0 else d.clone() for d in dense0] for j in range(layers)]
    for row in sparse:
        for l in row:
            l.workspace(N)
    h = (torch.rand((N, 5120), device=dev) * 2 - 1).to(torch.float16)
    attn = (torch.rand((N, 5120), device=dev) * 2 - 1).to(torch.float16)
    qkv = torch.empty((N, 15360), dtype=torch.float16, device=dev)
    o = torch.empty((N, 5120), dtype=torch.float16, device=dev)
    f = torch.empty((N, 20480), dtype=torch.float16, device=dev)
    hs = [torch.empty((N, 5120), dtype=torch.float16, device=dev) for _ in range(2)]

    def run_sparse(stream):
        x = h
        for j, (lq, lo, l1, l2) in enumerate(sparse):
            lq(x, out=qkv, stream=stream)
            lo(attn, out=o, stream=stream)
            l1(o, out=f, stream=stream)
            x = l2(f, out=hs[j & 1], stream=stream)

    def run_dense(stream):
        x = h
        for j, (wq, wo, w1, w2) in enumerate(dense):
            torch.matmul(x, wq.t(), out=qkv)
            torch.matmul(attn, wo.t(), out=o)
            torch.matmul(o, w1.t(), out=f)
            x = torch.matmul(f, w2.t(), out=hs[j & 1])

    def timed(fn, reps):
        ramp(torch, fn)
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    out = {"layers": layers, "N": N, "linears": info, "calls_per_step": 4 * layers,
           "what": "ms per decode step over the linears of all layers; weights of every layer resident separately"}
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        # Before anything is timed: one pass of the chain, then every linear of the last layer recomputed in fp32
        # from the dense weights on the very inputs the chain gave it (the buffers still hold that layer's values).
        run_sparse(side)
        side.synchronize()
        j = layers - 1
        x_in = hs[(j - 1) & 1] if j > 0 else h
        worst = {"max_abs_frac": 0.0, "rel_l2": 0.0}
        for nm, w, x, y in zip(names, dense[j], (x_in, attn, o, f), (qkv, o, f, hs[j & 1])):
            ref = torch.matmul(x.float(), w.float().t())
            d = (y.float() - ref)
            worst["max_abs_frac"] = max(worst["max_abs_frac"], float(d.abs().max() / ref.abs().max()))
            worst["rel_l2"] = max(worst["rel_l2"], float(d.norm() / ref.norm()))
        out["check"] = dict(worst, what="last layer of the chain, every linear vs an fp32 product of the dense "
                                        "weights with the chain's own inputs")
        if not (worst["max_abs_frac"] <= 1e-2 and worst["rel_l2"] <= 1e-3):
            raise RuntimeError(f"decode chain: outputs outside the tolerance: {worst}")
        out["sparse_eager_ms"] = timed(lambda: run_sparse(side), 5)
        out["dense_eager_ms"] = timed(lambda: run_dense(side), 5)
        for name, fn in (("sparse", run_sparse), ("dense", run_dense)):
            try:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    fn(side)
                out[name + "_graph_ms"] = timed(g.replay, 10)
            except Exception as e:  # capture is an extra; the eager figures stand on their own
                out[name + "_graph_ms"] = None
                out[name + "_graph_error"] = str(e)[:200]
    torch.cuda.synchronize()
    sp = out.get("sparse_graph_ms") or out["sparse_eager_ms"]
    de = out.get("dense_graph_ms") or out["dense_eager_ms"]
    out["speedup_vs_dense"] = de / sp
    out["weight_bytes_sparse"] = int(sum(i["bytes"] for i in info)) * layers
    out["weight_bytes_dense"] = int(sum(2 * i["M"] * i["K"] for i in info)) * layers
    return out


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build drives one GPU; run with --gpus 1 (row blocks are independent, so the path "
              "would shard by rows without any exchange, but no multi-GPU launch is part of this build)", file=sys.stderr)
        sys.exit(2)
    import torch

    import spmspm_amd as S
    from spmspm_amd.synthetic import WORKLOADS, make_activations, make_weight

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    w = dict(WORKLOADS[a.workload])
    if a.n is not None:
        w["N"] = a.n
    if a.sparsity is not None:
        w["sparsity"] = a.sparsity
    M, K, N = w["M"], w["K"], w["N"]
    dev = torch.device("cuda:0")

    t0 = time.perf_counter()
    W = make_weight(M, K, w["sparsity"], seed=a.seed, pruning=w["pruning"])
    X = make_activations(K, N, seed=a.seed)
    t_gen = time.perf_counter() - t0
    t0 = time.perf_counter()
    comp = S.InitSparseMatrixA_bitmap(W)
    t_enc = time.perf_counter() - t0

    algo_bytes = comp.algorithmic_bytes(N)
    copies = max(2, -(-3 * LLC_BYTES // algo_bytes))
    layers = [S.SparseLinear(comp, device=dev, split_k=a.split_k) for _ in range(copies)]
    xs = [torch.from_numpy(X.view(np.int16).copy()).to(dev).view(torch.float16) for _ in range(copies)]
    outs = [torch.empty((N, M), dtype=torch.float16, device=dev) for _ in range(copies)]
    split_k = a.split_k if a.split_k > 0 else S.SpMM_SplitK_Auto(M, N, K)
    ws_bytes = S.SpMM_WorkspaceBytes(M, N, K, a.split_k)
    for l in layers:
        l.workspace(N)

    hip = Hip()
    L = S.library()
    stream = torch.cuda.current_stream()
    shandle = stream.cuda_stream

    calls = [bound_call(L, layers[j], xs[j], outs[j], shandle) for j in range(copies)]

    def step(i, ev=None):
        if ev is not None:
            L.SpMM_TimeNextCall(ev[0], ev[1])
        calls[i % copies]()

    # Calls after the GPU has been idle run 15-20 % slower for about 20 ms (ramp()); keep it busy before the W warm-up
    # steps.  The shader clock read below (1.9-2.3 GHz under this load) says which state the timed region saw.
    def burst(n):
        for i in range(n):
            step(i)

    # The first use of a second stream idles the GPU for some milliseconds (its queue is set up): do it now, with a
    # throw-away probe, so that the probe before the timed region reads a ramped clock and leaves no gap behind it.
    side = torch.cuda.Stream()
    shader_clock_mhz(torch, L, side, burst)
    ramp(torch, lambda: burst(50), a.prewarm_ms)
    clock_before = shader_clock_mhz(torch, L, side, burst)
    ramp(torch, lambda: burst(50), 20.0 if a.prewarm_ms > 0 else 0.0)
    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()

    # timed region 1: K steps, wall clock between synchronisations -> value; the same steps on the GPU's clock
    # (events recorded on the launch stream before the first and after the last call) -> roofline
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    g0.record(stream)
    for i in range(a.steps):
        step(i)
    g1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    call_gpu_s = g0.elapsed_time(g1) / 1e3 / a.steps

    # timed region 2: the same K steps with a HIP event pair attached to every main-kernel dispatch -> roofline
    events = [(hip.event(), hip.event()) for _ in range(a.steps)]
    for i in range(a.steps):
        step(i, events[i])
    torch.cuda.synchronize()
    kern_ms = np.array([hip.elapsed_ms(e0, e1) for e0, e1 in events])
    for e0, e1 in events:
        hip.rt.hipEventDestroy(e0), hip.rt.hipEventDestroy(e1)

    clock_after = shader_clock_mhz(torch, L, side, burst)

    if a.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    ms_per_step = wall / a.steps * 1e3
    flops = 2.0 * M * N * K
    value = flops / (wall / a.steps) / 1e12
    kern_avg_s = float(kern_ms.mean()) / 1e3
    achieved = algo_bytes / call_gpu_s / 1e9          # whole call: main kernel + split-K reduction + the gap between
    achieved_main = algo_bytes / kern_avg_s / 1e9     # main kernel alone

    # correctness of what was timed: a row sample against float64
    rows = np.random.default_rng(1).choice(M, 128, replace=False)
    got = outs[0].cpu().numpy()[:, rows].astype(np.float64)
    ref = X.astype(np.float64) @ W[rows].astype(np.float64).T
    max_abs_frac = float(np.abs(got - ref).max() / np.abs(ref).max())
    rel_l2 = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))

    dense = None
    if not a.no_dense:
        Wd = [torch.from_numpy(W.view(np.int16)).to(dev).view(torch.float16) for _ in range(max(2, -(-3 * LLC_BYTES // (2 * M * K))))]
        ramp(torch, lambda: [torch.matmul(xs[0], Wd[i % len(Wd)].t()) for i in range(20)])
        t0 = time.perf_counter()
        reps = max(20, a.steps // 4)
        for i in range(reps):
            torch.matmul(xs[0], Wd[i % len(Wd)].t())
        torch.cuda.synchronize()
        td = (time.perf_counter() - t0) / reps
        dense = {"ms": td * 1e3, "tflops": flops / td / 1e12, "gbs": (2.0 * M * K + 2 * K * N + 2 * M * N) / td / 1e9,
                 "what": "torch.matmul fp16 (hipBLASLt), same run, rotating weight copies"}
        del Wd

    # HBM bytes per launch of the main kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE.  The record
    # is only quoted when it was taken for exactly what ran here: same workload, width, sparsity, Split_K, kernel.
    kernel_name = L.SpMM_KernelName(M, N, K, split_k).decode()
    traffic, traffic_note = None, "no record for this configuration in profiles/traffic.json"
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        rec = json.load(open(tpath)).get(f"{a.workload}_n{N}_s{int(round(w['sparsity'] * 100))}")
        if rec and rec.get("split_k") == split_k and rec.get("kernel") == kernel_name:
            traffic, traffic_note = rec["bytes_per_launch"], rec["source"]
        elif rec:
            traffic_note = (f"record is for {rec.get('kernel')} at Split_K={rec.get('split_k')}, this run used "
                            f"{kernel_name} at Split_K={split_k}: not quoted")

    stream_ceiling = None
    probe = os.path.join(os.path.dirname(S.library_path()), "stream_probe")
    if not a.no_stream_probe and os.path.exists(probe):
        import subprocess
        pr = subprocess.run([probe], capture_output=True, text=True, timeout=120)
        for line in pr.stdout.splitlines():
            if line.startswith("{"):
                stream_ceiling = json.loads(line)

    out = {
        "metric": "SpMM dense-equiv TFLOP/s", "value": value, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"{a.workload}: W {M}x{K} fp16 N(0,0.02) {w['pruning']}-pruned to "
                               f"{w['sparsity'] * 100:.0f}% sparsity, X {K}x{N} U(-1,1), seed {a.seed}",
                   "M": M, "K": K, "N": N, "sparsity": w["sparsity"], "split_k": split_k,
                   "weight_copies_rotated": copies, "nnz_padded": int(comp.offsets[-1]),
                   "workspace_bytes": ws_bytes},
        "gbs_whole_call": algo_bytes / (wall / a.steps) / 1e9,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_note,
                     "algorithmic_bytes_per_launch": algo_bytes,
                     "what": "algorithmic bytes / GPU time of one call (main kernel + split-K reduction and the gap "
                             "between them), from events recorded on the launch stream around the K timed steps",
                     "call_us": call_gpu_s * 1e6,
                     "main_kernel": {"name": kernel_name, "avg_us": kern_avg_s * 1e6,
                                     "min_us": float(kern_ms.min()) * 1e3, "achieved": achieved_main,
                                     "frac": achieved_main / HBM_PEAK_GBS,
                                     "timing": "HIP events attached to each main-kernel dispatch (kernel begin/end "
                                               "timestamps), the same K steps repeated after the first region"},
                     "shader_clock_mhz": {"before": clock_before, "after": clock_after,
                                          "what": "shader-clock counter against the 100 MHz counter over 2 ms of "
                                                  "the same calls, one idling wave on a second stream "
                                                  "(SpMM_ShaderClockProbe), before and after the timed regions"},
                     "main_kernel_cycles_per_group_tile_and_cu":
                         None if not clock_after else kern_avg_s * clock_after * 1e6 / ((M // 64) * (K // 64) / 256.0),
                     "stream_ceiling_gbs": None if stream_ceiling is None else stream_ceiling["stream_ceiling_gbs"],
                     "frac_of_stream_ceiling": None if stream_ceiling is None
                     else achieved / stream_ceiling["stream_ceiling_gbs"],
                     "stream_ceiling_what": None if stream_ceiling is None
                     else "best plain read stream of this GPU in this run (spmspm_amd/lib/stream_probe): "
                          + stream_ceiling["best"]},
        "check": {"max_abs_over_max_ref": max_abs_frac, "rel_l2": rel_l2, "rows_sampled": 128},
        "dense_fp16": dense,
        "host": {"generate_s": t_gen, "encode_s": t_enc, "encode_threads": os.cpu_count()},
    }
    if not a.no_qkv and a.workload != "opt13b_qkv":
        out["opt13b_qkv"] = quick_measure(torch, S, hip, dev, "opt13b_qkv", max(20, a.steps // 2), a.warmup, a.seed)
    if not a.no_encoder:
        out["device_encoder"] = device_encoder(torch, S, dev, W, comp, t_enc)
    if not a.no_sweep:
        del layers, xs, outs
        layers = xs = outs = None
        torch.cuda.empty_cache()
        out["sweep"] = sweep(torch, S, hip, dev, a.sweep_steps, a.seed)
    if not a.no_chain:
        layers = xs = outs = None
        torch.cuda.empty_cache()
        out["decode_chain_opt13b"] = decode_chain(torch, S, dev, a.chain_layers, a.seed)
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(comp, X, a.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
