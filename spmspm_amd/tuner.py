"""Measures the best Split_K per shape on the GPU and keeps the result in the library's table.

The reference keeps these choices by hand: SplitKDict in
end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:23 (keyed by M) and the SPLIT_K array of
kernel_benchmark/run_all_main.sh:5.  Here they are measured: every candidate split runs the whole call
(main kernel + reduction) back to back on one stream, rotating among several resident copies of the
weights so that the 256 MB last-level cache does not serve them, and the fastest wins.

    python -m spmspm_amd.tuner --preset opt13b --n 16 --out splitk.txt
    SPMM_SPLITK_TABLE=splitk.txt python your_program.py      # or spmspm_amd.SpMM_SplitK_TableLoad("splitk.txt")
"""
import argparse
import json
import sys

import numpy as np

from . import api as A
from .synthetic import make_activations, make_weight

# (M, K) of the decode-step linears of the benchmark configurations
PRESETS = {
    "opt13b": [(15360, 5120), (5120, 5120), (20480, 5120), (5120, 20480)],
    "opt30b": [(21504, 7168), (7168, 7168), (28672, 7168), (7168, 28672)],
    "opt66b": [(27648, 9216), (9216, 9216), (36864, 9216), (9216, 36864)],
}


def candidate_splits(K, limit=12, M=None, N=None):
    """1..limit, never more batches than a quarter of the group-tile columns (one tile per wave and batch).  With M
    and N given and the shape dispatched to the wide kernel (four row blocks per workgroup, so its good splits are
    larger): 1..32, never more than half of the group-tile columns."""
    nkb = K // 64
    if M is not None and N is not None and b"wide" in (A.library().SpMM_KernelName(M, N, K, 1) or b""):
        return [s for s in range(1, 33) if s <= max(1, nkb // 2)]
    return [s for s in range(1, limit + 1) if s <= max(1, nkb // 4)]


def time_split_k(layers, x, split_k, iters=300, warmup=20):
    """Average time in microseconds of one call at this Split_K, rotating among `layers` (resident copies)."""
    import torch
    for L in layers:
        L.split_k = split_k
    outs = [torch.empty((x.shape[0], layers[0].M), dtype=torch.float16, device=x.device) for _ in layers]
    for i in range(warmup):
        layers[i % len(layers)](x, out=outs[i % len(layers)])
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        layers[i % len(layers)](x, out=outs[i % len(layers)])
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def tune_shape(M, N, K, sparsity=0.6, candidates=None, device="cuda:0", iters=300, copies_bytes=768 << 20, seed=0):
    """Times every candidate Split_K for one shape; returns (best_split, {split: microseconds}).

    The matrix is synthetic (Bernoulli mask at `sparsity`): the choice depends on the shape and on the bytes
    per tile, not on the values."""
    import torch
    W = make_weight(M, K, sparsity, seed=seed)
    comp = A.InitSparseMatrixA_bitmap(W)
    first = A.SparseLinear(comp, device=device)
    per_copy = 2 * first.nnz_padded + 8 * first.bitmaps.numel()
    n_copies = int(min(8, max(2, copies_bytes // max(per_copy, 1) + 1)))
    layers = [first] + [first.clone() for _ in range(n_copies - 1)]
    x = torch.from_numpy(make_activations(K, N, seed=seed).view(np.int16).copy()).to(device).view(torch.float16)
    times = {}
    cands = list(candidates or candidate_splits(K, M=M, N=N))
    time_split_k(layers, x, cands[0], iters=max(iters, 300))  # not kept: the first calls after idle run at ramping clocks
    for sk in cands:
        times[sk] = time_split_k(layers, x, sk, iters=iters)
    best = min(times, key=times.get)
    return best, times


def _cost_model_choice(M, N, K):
    """What the built-in cost model picks for a shape (the table is not consulted)."""
    return A.SpMM_SplitK_CostModel(M, N, K)


def tune(shapes, N, sparsity=0.6, record=True, log=None, **kw):
    """tune_shape over (M, K) pairs; with `record`, each winner goes into the library's table.
    Returns {(M, N, K): (best, times)}."""
    out = {}
    for M, K in shapes:
        best, times = tune_shape(M, N, K, sparsity=sparsity, **kw)
        out[(M, N, K)] = (best, times)
        if record:
            A.SpMM_SplitK_TableSet(M, N, K, best)
        if log:
            model = _cost_model_choice(M, N, K) if record else None
            log(f"M={M} N={N} K={K}: best Split_K {best} ({times[best]:.1f} us)"
                + (f", cost model {model} ({times.get(model, float('nan')):.1f} us)" if model else "")
                + "  " + " ".join(f"{s}:{t:.1f}" for s, t in sorted(times.items())))
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--preset", choices=sorted(PRESETS), help="decode-step linears of a model")
    ap.add_argument("--shape", action="append", default=[], metavar="MxK", help="extra shape, e.g. 28672x7168")
    ap.add_argument("--n", type=int, action="append", help="batch columns (repeatable; default 16)")
    ap.add_argument("--sparsity", type=float, default=0.6)
    ap.add_argument("--iters", type=int, default=300)
    ap.add_argument("--out", help="write the table here (text, one 'M N K Split_K' per line)")
    ap.add_argument("--json", help="also write every measured time here")
    a = ap.parse_args(argv)
    shapes = list(PRESETS.get(a.preset, []))
    for s in a.shape:
        m, k = s.lower().split("x")
        shapes.append((int(m), int(k)))
    if not shapes:
        ap.error("no shapes: give --preset or --shape")
    report = {}
    for N in (a.n or [16]):
        res = tune(shapes, N, sparsity=a.sparsity, iters=a.iters, log=lambda m: print(m, file=sys.stderr, flush=True))
        for (M, n, K), (best, times) in res.items():
            report[f"{M} {n} {K}"] = {"best": best, "us": {str(s): round(t, 2) for s, t in times.items()}}
    if a.out:
        print(f"{A.SpMM_SplitK_TableSave(a.out)} entries -> {a.out}", file=sys.stderr)
    if a.json:
        with open(a.json, "w") as f:
            json.dump(report, f, indent=1)
    print(json.dumps({k: v["best"] for k, v in report.items()}))


if __name__ == "__main__":
    main()
