"""Device encoder (SpMM_EncodeDevice_*) against the CPU oracle (the restatement of csrc/SpMM_API.cuh:112-241), the
committed golden encodings and the host encoder, bit for bit, and its output fed to the SpMM."""
import numpy as np
import pytest

import spmspm_amd as S
from spmspm_amd.synthetic import make_activations, make_weight

from conftest import assert_spmm_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available()
    return torch


def _special_matrix(M, K, seed):
    """Random sparse matrix sprinkled with -0.0, NaN, +-inf and subnormals, plus empty and full group tiles."""
    rng = np.random.default_rng(seed)
    W = make_weight(M, K, 0.6, seed=seed)
    u = W.view(np.uint16)
    for pat in (0x8000, 0x7e00, 0xfe01, 0x7c00, 0xfc00, 0x0001, 0x83ff):
        idx = rng.integers(0, M * K, 50)
        u.reshape(-1)[idx] = pat
    W[:64, :64] = 0                                      # an empty group tile
    W[64:128, 64:128] = np.float16(1.5)                  # a completely full one
    u[128:192, :64] = 0x8000                             # all -0.0: encodes as empty
    return W


@pytest.mark.parametrize("M,K,sparsity", [(64, 64, 0.5), (128, 192, 0.7), (512, 1024, 0.9), (1024, 256, 0.0),
                                          (256, 256, 1.0), (2048, 4096, 0.6), (65536, 64, 0.5)])
def test_device_encoder_is_bit_identical_to_the_oracle_and_the_host_encoder(torch, oracle, M, K, sparsity):
    W = _special_matrix(M, K, seed=M + K) if (M >= 192 and K >= 128) else make_weight(M, K, sparsity, seed=M + K)
    if sparsity == 1.0:
        W[:] = 0
    want = oracle.encode(W, M, K)
    comp = S.InitSparseMatrixA_bitmap(W)
    Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    print(f"case M={M} K={K} s={sparsity}", flush=True)
    values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device(Wd)
    torch.cuda.synchronize()
    got_o, got_b, got_v = offsets.cpu().numpy(), bitmaps.cpu().numpy().view(np.uint64), values.cpu().numpy().view(np.uint16)
    assert np.array_equal(got_o, want["global"])
    assert np.array_equal(got_b, want["bitmap"])
    assert np.array_equal(got_v, want["values"])
    assert np.array_equal(got_o, comp.offsets) and np.array_equal(got_b, comp.bitmaps) and np.array_equal(got_v, comp.values)


def test_device_encoder_reproduces_the_golden_encodings(torch, golden):
    """Every committed golden input whose shape the device encoder takes (multiples of 64): W -> device -> arrays must
    be the arrays the reference's own encoder wrote into the fixture."""
    ran = 0
    for name, case in golden.items():
        W = case["W"]
        M, K = W.shape
        if M % 64 or K % 64:
            continue
        print(f"golden {name} {M}x{K}", flush=True)
        Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
        values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device(Wd)
        torch.cuda.synchronize()
        assert np.array_equal(offsets.cpu().numpy(), case["offsets"]), name
        assert np.array_equal(bitmaps.cpu().numpy().view(np.uint64), case["bitmaps"]), name
        assert np.array_equal(values.cpu().numpy().view(np.uint16), case["values"]), name
        ran += 1
    assert ran >= 7


@pytest.mark.parametrize("M,K,sparsity", [(64, 64, 0.5), (128, 192, 0.7), (512, 1024, 0.9), (1024, 256, 0.0),
                                          (256, 256, 1.0), (2048, 4096, 0.6), (65536, 64, 0.5), (64 * 37, 64 * 61, 0.8),
                                          (8192, 64 * 129, 0.7), (64, 64 * 40, 0.3)])
def test_one_pass_device_encoder_is_bit_identical_to_the_oracle(torch, oracle, M, K, sparsity):
    """SpMM_EncodeDevice_OnePass (W read once, offsets by look-back between workgroups) against the oracle.  A
    workgroup takes a chunk of 16 group tiles and the look-back works on blocks of 64 chunks: 2257 group tiles are
    142 chunks (the last one of a single tile) in 3 blocks (the last one partial), 16512 group tiles are 1032 chunks
    in 17 blocks.  Group tiles more than half full (sparsity 0.0 and 0.3) are compacted in two halves."""
    W = _special_matrix(M, K, seed=M + K) if (M >= 192 and K >= 128) else make_weight(M, K, sparsity, seed=M + K)
    if sparsity == 1.0:
        W[:] = 0
    want = oracle.encode(W, M, K)
    Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    print(f"one-pass case M={M} K={K} s={sparsity}", flush=True)
    for rep in range(2):  # the second run finds the scratch and output buffers of the first in the allocator
        values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device_onepass(Wd)
        torch.cuda.synchronize()
        assert np.array_equal(offsets.cpu().numpy(), want["global"])
        assert np.array_equal(bitmaps.cpu().numpy().view(np.uint64), want["bitmap"])
        assert np.array_equal(values.cpu().numpy().view(np.uint16), want["values"])


def test_one_pass_device_encoder_looks_back_over_more_than_one_trip(torch, oracle):
    """65792 group tiles = 4112 chunks in 65 blocks: the chunks of the last block look back over 64 blocks, find no
    block that shows a prefix only if the others lag, and otherwise stop early; either way the sum must come out."""
    M, K = 16384, 64 * 257
    W = np.tile(make_weight(2048, K, 0.7, seed=99), (8, 1))
    want = oracle.encode(W, M, K)
    Wd = torch.from_numpy(W.view(np.int16)).to("cuda:0").view(torch.float16)
    print(f"one-pass case M={M} K={K}", flush=True)
    values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device_onepass(Wd)
    torch.cuda.synchronize()
    assert np.array_equal(offsets.cpu().numpy(), want["global"])
    assert np.array_equal(bitmaps.cpu().numpy().view(np.uint64), want["bitmap"])
    assert np.array_equal(values.cpu().numpy().view(np.uint16), want["values"])


def test_one_pass_device_encoder_golden_and_capacity(torch, golden):
    ran = 0
    for name, case in golden.items():
        W = case["W"]
        M, K = W.shape
        if M % 64 or K % 64:
            continue
        Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
        values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device_onepass(Wd)
        torch.cuda.synchronize()
        assert np.array_equal(offsets.cpu().numpy(), case["offsets"]), name
        assert np.array_equal(bitmaps.cpu().numpy().view(np.uint64), case["bitmaps"]), name
        assert np.array_equal(values.cpu().numpy().view(np.uint16), case["values"]), name
        ran += 1
    assert ran >= 7
    # a values buffer that is too small: reported, nothing written past its end, bitmaps and offsets still complete
    W = make_weight(256, 256, 0.5, seed=5)
    comp = S.InitSparseMatrixA_bitmap(W)
    Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    need = int(comp.offsets[-1])
    buf = torch.full((need + 64,), 0x5a5a, dtype=torch.int16, device="cuda:0")
    with pytest.raises(ValueError, match="the matrix needs %d" % need):
        S.InitSparseMatrixA_bitmap_device_onepass(Wd, values=buf[:need - 8])
    assert (buf[need - 8:] == 0x5a5a).all()
    v, b, o = S.InitSparseMatrixA_bitmap_device_onepass(Wd, values=buf[:need])  # exactly enough
    assert np.array_equal(v.cpu().numpy().view(np.uint16), comp.values) and (buf[need:] == 0x5a5a).all()
    L = S.library()
    assert L.SpMM_EncodeDevice_OnePass(None, Wd.data_ptr(), 256, 256, b.data_ptr(), o.data_ptr(), buf.data_ptr(), need, None) == 1
    # 16 group tiles = one chunk in one block; 2257 group tiles = 142 chunks in 3 blocks
    assert L.SpMM_EncodeDevice_ScratchBytes(256, 256) == 16 + 8 * (1 + 1) and L.SpMM_EncodeDevice_ScratchBytes(100, 64) == 0
    assert L.SpMM_EncodeDevice_ScratchBytes(64 * 37, 64 * 61) == 16 + 8 * (142 + 3)


def test_device_encoded_weights_multiply_correctly(torch, oracle):
    M, K, N = 1024, 2048, 16
    W = make_weight(M, K, 0.7, seed=77)
    X = make_activations(K, N, seed=77)
    Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device(Wd)
    x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
    out = torch.empty((N, M), dtype=torch.int16, device="cuda:0")
    ws = torch.empty(S.SpMM_WorkspaceBytes(M, N, K, 0) + 16, dtype=torch.uint8, device="cuda:0")
    assert S.SpMM_SplitK_API(None, values, bitmaps, offsets, x, out, M, N, K, ws, 0) == 0
    torch.cuda.synchronize()
    ref = X.astype(np.float64) @ W.astype(np.float64).T
    assert_spmm_close(out.cpu().numpy().view(np.float16), ref, "device-encoded weights")


def test_device_encoder_rejects_ragged_shapes(torch, capfd):
    t = torch.zeros(64, dtype=torch.int16, device="cuda:0")
    L = S.library()
    assert L.SpMM_EncodeDevice_Bitmaps(None, t.data_ptr(), 100, 64, t.data_ptr(), t.data_ptr()) == S.api.HIP_ERROR_INVALID_VALUE
    assert "multiples of 64" in capfd.readouterr().out
    assert L.SpMM_EncodeDevice_Values(None, t.data_ptr(), 64, 70, t.data_ptr(), t.data_ptr()) == S.api.HIP_ERROR_INVALID_VALUE


def test_device_encoder_offsets_scan_across_many_blocks(torch, oracle):
    """More than 1024 group tiles, not a multiple of 1024: the in-place running sum crosses block boundaries."""
    M, K = 64 * 37, 64 * 61  # 2257 group tiles
    W = make_weight(M, K, 0.8, seed=9)
    comp = S.InitSparseMatrixA_bitmap(W)
    want = oracle.encode(W, M, K)
    assert np.array_equal(comp.offsets, want["global"]) and np.array_equal(comp.values, want["values"])
    Wd = torch.from_numpy(W.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    values, bitmaps, offsets = S.InitSparseMatrixA_bitmap_device(Wd)
    torch.cuda.synchronize()
    assert np.array_equal(offsets.cpu().numpy(), comp.offsets)
    assert np.array_equal(values.cpu().numpy().view(np.uint16), comp.values)


def test_weight_files_load_into_device_arrays_and_multiply(torch, oracle, tmp_path):
    """SpMM_LoadWeightFiles: the six files Our_GenSparseMatrixBinFile writes -> device arrays equal to the oracle's
    encoding, usable by the SpMM as they are; a damaged file leaves nothing behind."""
    import ctypes as C
    M, K, N = 256, 512, 16
    W = make_weight(M, K, 0.6, seed=31)
    X = make_activations(K, N, seed=31)
    dense = tmp_path / "w.bin"
    W.tofile(dense)
    names = [str(tmp_path / n).encode() for n in ("v", "g", "m", "b", "x", "s")]
    S.Our_GenSparseMatrixBinFile(str(dense), M, K, *[n.decode() for n in names])
    L = S.library()
    ptrs = [C.c_void_p() for _ in range(5)]
    count = C.c_int(-1)
    G = L.SpMM_LoadWeightFiles(*names, M, K, *[C.byref(p) for p in ptrs], C.byref(count))
    want = oracle.encode(W, M, K)
    assert G == (M // 64) * (K // 64) and count.value == int(want["global"][-1])
    values_d, offsets_d, median_d, bitmaps_d, max_nnz_d = [p.value for p in ptrs]
    assert all(p for p in (values_d, offsets_d, median_d, bitmaps_d, max_nnz_d))

    def fetch(ptr, dtype, n):  # device -> host through a torch tensor of the same size
        t = torch.empty(n, dtype=dtype, device="cuda:0")
        hip = C.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        assert hip.hipMemcpy(t.data_ptr(), ptr, t.numel() * t.element_size(), 3) == 0  # device to device
        return t.cpu().numpy()

    assert np.array_equal(fetch(values_d, torch.int16, count.value).view(np.uint16), want["values"])
    assert np.array_equal(fetch(offsets_d, torch.int32, G + 1), want["global"])
    assert np.array_equal(fetch(bitmaps_d, torch.int64, 64 * G).view(np.uint64), want["bitmap"])
    assert np.array_equal(fetch(median_d, torch.int32, 4 * G), want["median"])
    x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
    out = torch.empty((N, M), dtype=torch.int16, device="cuda:0")
    ws = torch.empty(S.SpMM_WorkspaceBytes(M, N, K, 0) + 16, dtype=torch.uint8, device="cuda:0")
    assert S.SpMM_SplitK_API(None, values_d, bitmaps_d, offsets_d, x, out, M, N, K, ws, 0) == 0
    torch.cuda.synchronize()
    assert_spmm_close(out.cpu().numpy().view(np.float16), X.astype(np.float64) @ W.astype(np.float64).T, "loaded weights")
    L.SpMM_FreeWeights(*ptrs)
    # a values file cut short: refused, the out-pointers stay as they were
    with open(names[0].decode(), "r+b") as f:
        f.truncate(10)
    ptrs = [C.c_void_p() for _ in range(5)]
    assert L.SpMM_LoadWeightFiles(*names, M, K, *[C.byref(p) for p in ptrs], None) == -1
    assert all(p.value is None for p in ptrs)
