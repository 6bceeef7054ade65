"""Writes tests/golden/encoder_fixtures.npz: inputs and the outputs of the REFERENCE encoder.

Run in the build container only (needs the reference tree to have been
compiled into oracle/_ref/libref_encoder.so by oracle/Makefile):

    python tests/golden/make_encoder_fixtures.py

Each case stores the dense fp16 input as uint16 bit patterns plus everything
InitSparseMatrixA_bitmap (csrc/SpMM_API.cuh:112-241) returned for it.  The
fixture is data only; nothing of the reference's text is stored.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402


def gaussian(rng, M, K, sparsity):
    W = (rng.standard_normal((M, K)) * 0.02).astype(np.float16)
    W[rng.random((M, K)) < sparsity] = 0
    return W.view(np.uint16)


def special(rng, M, K):
    W = gaussian(rng, M, K, 0.5).copy()
    flat = W.reshape(-1)
    idx = rng.permutation(flat.size)
    pats = [0x8000,  # -0.0 : dropped by the encoder
            0x0001, 0x8001, 0x03ff,  # subnormals : kept
            0x7e00, 0xfe00, 0x7c01,  # NaNs : kept
            0x7c00, 0xfc00,  # infinities : kept
            0x0400, 0x7bff]  # smallest normal, largest finite
    for i, p in enumerate(pats * 40):
        flat[idx[i]] = p
    return W


def cases():
    rng = np.random.default_rng(20250101)
    yield "g64x64_s50", gaussian(rng, 64, 64, 0.5)
    yield "g128x192_s70", gaussian(rng, 128, 192, 0.7)
    yield "g64x128_dense", gaussian(rng, 64, 128, 0.0)
    yield "z128x64_allzero", np.zeros((128, 64), np.uint16)
    yield "special64x128", special(rng, 64, 128)
    yield "g128x128_s90", gaussian(rng, 128, 128, 0.9)
    yield "g128x64_s99", gaussian(rng, 128, 64, 0.99)
    yield "ragged100x150_s50", gaussian(rng, 100, 150, 0.5)
    W, _ = O.init_host_matrices(192, 128, 8, 50, reseed=True)  # the reference harness generator
    yield "rand192x128_p50", W.view(np.uint16)


def main():
    if O.ref_lib() is None:
        raise SystemExit("build oracle/_ref first: make -C oracle")
    out = {}
    names = []
    for name, W in cases():
        M, K = W.shape
        r = O.ref_encode(W, M, K)
        G = r["num_gtiles"]
        names.append(name)
        out[name + "/W"] = W
        out[name + "/values"] = r["values"]
        out[name + "/offsets"] = r["global"]
        out[name + "/median"] = r["median"]
        # tiles beyond the last whole group tile are left uninitialised by the reference: keep 64*G
        out[name + "/bitmaps"] = r["bitmap"][:64 * G]
        out[name + "/tile_counts"] = r["tile_cnt"][:64 * G]
        out[name + "/scalars"] = np.array([G, r["max_nnz"]], np.int64)
    out["names"] = np.array(names)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "encoder_fixtures.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(names), "cases")


if __name__ == "__main__":
    main()
