"""Seeded synthetic inputs of the shapes the benchmark configurations name.

W ~ N(0, 0.02) in fp32, cast to fp16, then pruned either with a uniform
random mask ("random") or by zeroing the smallest magnitudes of the whole
matrix ("magnitude"); X ~ U(-1, 1) fp16 laid out [N][K].  numpy
`default_rng(seed)` is the generator throughout.
"""
import numpy as np


def make_weight(M, K, sparsity, seed=0, pruning="random"):
    """Dense row-major fp16 [M][K] with about `sparsity` (0..1) of its entries zero."""
    rng = np.random.default_rng(seed)
    W = np.empty((M, K), np.float16)
    rows = max(1, (1 << 22) // max(K, 1))
    for r0 in range(0, M, rows):  # chunked so the fp32 temporaries stay small
        r1 = min(M, r0 + rows)
        W[r0:r1] = (rng.standard_normal((r1 - r0, K), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    if sparsity <= 0:
        return W
    if pruning == "random":
        for r0 in range(0, M, rows):
            r1 = min(M, r0 + rows)
            W[r0:r1][rng.random((r1 - r0, K), dtype=np.float32) < sparsity] = 0
    elif pruning == "magnitude":
        mag = np.abs(W.view(np.uint16) & np.uint16(0x7fff))  # fp16 magnitudes order like their bit patterns
        kth = int(round(sparsity * mag.size))
        if kth > 0:
            thresh = np.partition(mag.reshape(-1), kth - 1)[kth - 1]
            W[mag <= thresh] = 0
    else:
        raise ValueError("pruning must be 'random' or 'magnitude'")
    return W


def make_activations(K, N, seed=0):
    """X as [N][K] fp16, U(-1, 1)."""
    rng = np.random.default_rng(seed + 0x9E3779B1)
    return rng.uniform(-1.0, 1.0, size=(N, K)).astype(np.float32).astype(np.float16)


# Shapes named by the benchmark configurations.
WORKLOADS = {
    "cpu_plumbing_4096": dict(M=4096, K=4096, sparsity=0.5, pruning="random", N=16),
    "opt13b_qkv": dict(M=15360, K=5120, sparsity=0.6, pruning="magnitude", N=16),
    "opt30b_ffn1": dict(M=28672, K=7168, sparsity=0.7, pruning="random", N=16),
    "opt66b_ffn2": dict(M=9216, K=36864, sparsity=0.4, pruning="random", N=64),
    "opt13b_out": dict(M=5120, K=5120, sparsity=0.6, pruning="magnitude", N=16),
    "opt13b_ffn1": dict(M=20480, K=5120, sparsity=0.6, pruning="magnitude", N=16),
    "opt13b_ffn2": dict(M=5120, K=20480, sparsity=0.6, pruning="magnitude", N=16),
}
