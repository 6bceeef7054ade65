"""Host encoder of libSpMM_API.so: bit-exact against the golden vectors and the oracle."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

import spmspm_amd as S

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _same(c, e, G):
    return (c.num_gtiles == G and np.array_equal(c.values, e["values"]) and np.array_equal(c.offsets, e["global"])
            and np.array_equal(c.median, e["median"]) and np.array_equal(c.bitmaps[:64 * G], e["bitmap"][:64 * G])
            and np.array_equal(c.tile_counts[:64 * G], e["tile_cnt"][:64 * G]) and c.max_nnz == e["max_nnz"])


def test_encoder_matches_golden(golden):
    for name, g in golden.items():
        c = S.InitSparseMatrixA_bitmap(g["W"])
        G = int(g["scalars"][0])
        assert c.num_gtiles == G and c.max_nnz == int(g["scalars"][1]), name
        assert np.array_equal(c.values, g["values"]), name
        assert np.array_equal(c.offsets, g["offsets"]), name
        assert np.array_equal(c.median, g["median"]), name
        assert np.array_equal(c.bitmaps[:64 * G], g["bitmaps"]), name
        assert np.array_equal(c.tile_counts[:64 * G], g["tile_counts"]), name


@pytest.mark.parametrize("M,K,s", [(64, 64, 0.5), (320, 200, 0.5), (1024, 512, 0.7), (512, 2048, 0.4),
                                   (128, 128, 0.0), (128, 128, 1.0), (63, 200, 0.5), (4096, 4096, 0.5)])
def test_encoder_matches_oracle(oracle, M, K, s):
    rng = np.random.default_rng(M * 31 + K)
    W = (rng.standard_normal((M, K)) * 0.02).astype(np.float16)
    W[rng.random((M, K)) < s] = 0
    e = oracle.encode(W, M, K)
    assert _same(S.InitSparseMatrixA_bitmap(W), e, e["num_gtiles"])


def test_encoder_thread_count_does_not_change_output(oracle, monkeypatch):
    from spmspm_amd.synthetic import make_weight
    W = make_weight(512, 768, 0.6, seed=3)
    e = oracle.encode(W, 512, 768)
    for n in ("1", "3", "16"):
        monkeypatch.setenv("SPMM_ENCODER_THREADS", n)
        assert _same(S.InitSparseMatrixA_bitmap(W), e, e["num_gtiles"])


def test_known_answers_through_product_encoder(oracle):
    for M, G, nnz, mx in [(256, 16, 32816, 2112), (1024, 256, 525360, 2176), (4096, 4096, 8405952, 2240)]:
        W, _ = oracle.init_host_matrices(M, M, 1, 50, reseed=True)
        c = S.InitSparseMatrixA_bitmap(W)
        assert (c.num_gtiles, int(c.offsets[-1]), c.max_nnz_rounded) == (G, nnz, mx)


def test_rejects_other_tilings():
    W = np.zeros((64, 64), np.float16)
    with pytest.raises(ValueError):
        S.InitSparseMatrixA_bitmap(W, tile_M=16)


def test_cpp_overload_with_reference_mangled_name():
    """Callers compiled against the reference link to this exact symbol (build/libSpMM_API.so exports it)."""
    L = S.library()
    fn = getattr(L, "_Z24InitSparseMatrixA_bitmapP6__halfiiiiiiiiPS0_PPiS3_S3_PPmRi")
    fn.restype = C.c_int
    W = (np.arange(64 * 64).reshape(64, 64) % 3).astype(np.float16)
    vals, cnt, med, glo, bmp = (C.c_void_p() for _ in range(5))
    mx = C.c_int(0)
    G = fn(C.c_void_p(W.ctypes.data), 64, 64, 8, 16, 64, 8, 64, 64, C.byref(vals), C.byref(cnt), C.byref(med),
           C.byref(glo), C.byref(bmp), C.byref(mx))
    assert G == 1
    want = S.InitSparseMatrixA_bitmap(W)
    assert mx.value == want.max_nnz
    got = np.ctypeslib.as_array(C.cast(glo, C.POINTER(C.c_int)), shape=(2,))
    assert list(got) == list(want.offsets)
    libc = C.CDLL(None)
    libc.free.argtypes = [C.c_void_p]
    for p in (vals, cnt, med, glo, bmp):
        libc.free(p)


def test_weight_files_byte_layout(tmp_path, oracle):
    """Six files with the reference's contents (csrc/SpMM_API.cuh:292-319)."""
    from spmspm_amd.synthetic import make_weight
    M, K = 128, 192
    W = make_weight(M, K, 0.6, seed=9)
    dense = tmp_path / "w.bin"
    W.tofile(dense)
    names = [str(tmp_path / f"w.{s}.bin") for s in ("NZWeights", "gtile", "mtile", "ltile", "intile", "OutputSizes")]
    S.Our_GenSparseMatrixBinFile(str(dense), M, K, *names)
    e = oracle.encode(W, M, K)
    G = e["num_gtiles"]
    assert np.array_equal(np.fromfile(names[0], np.uint16), e["values"])
    assert np.array_equal(np.fromfile(names[1], np.int32), e["global"])
    assert np.array_equal(np.fromfile(names[2], np.int32), e["median"])
    assert np.array_equal(np.fromfile(names[3], np.uint64), e["bitmap"][:64 * G])
    assert list(np.fromfile(names[4], np.int32)) == [oracle.round_max_nnz(e["max_nnz"])]
    assert list(np.fromfile(names[5], np.int32)) == [int(e["global"][-1]), G + 1, 4 * G, 64 * G]
    back = S.load_weight_files(*names, M, K)
    assert np.array_equal(back.values, e["values"]) and np.array_equal(back.bitmaps, e["bitmap"][:64 * G])
    assert np.array_equal(back.tile_counts, e["tile_cnt"][:64 * G])
    # the library's own reader (C ABI) returns the same arrays
    read = S.SpMM_ReadWeightFiles(*names, M, K)
    assert read.num_gtiles == G and read.max_nnz == oracle.round_max_nnz(e["max_nnz"])
    assert np.array_equal(read.values, e["values"]) and np.array_equal(read.bitmaps, e["bitmap"][:64 * G])
    assert np.array_equal(read.offsets, e["global"]) and np.array_equal(read.median, e["median"])
    assert np.array_equal(read.tile_counts, e["tile_cnt"][:64 * G])


def test_weight_file_reader_reports_what_is_wrong(tmp_path, oracle):
    """SpMM_ReadWeightFiles never ends the process: a missing or truncated file is -1 (OSError here), files that do
    not match M and K or each other are -2 (ValueError)."""
    from spmspm_amd.synthetic import make_weight
    M, K = 128, 192
    W = make_weight(M, K, 0.5, seed=3)
    dense = tmp_path / "w.bin"
    W.tofile(dense)
    names = [str(tmp_path / f"w.{s}.bin") for s in ("NZWeights", "gtile", "mtile", "ltile", "intile", "OutputSizes")]
    S.Our_GenSparseMatrixBinFile(str(dense), M, K, *names)
    assert S.SpMM_ReadWeightFiles(*names, M, K).num_gtiles == 6
    with pytest.raises(ValueError):
        S.SpMM_ReadWeightFiles(*names, M, K + 64)          # sizes file written for another shape
    with pytest.raises(ValueError):
        S.SpMM_ReadWeightFiles(*names, M + 1, K)           # not a multiple of 64
    vals = np.fromfile(names[0], np.uint16)
    vals[:-8].tofile(names[0])                             # values file eight halves short
    with pytest.raises(OSError):
        S.SpMM_ReadWeightFiles(*names, M, K)
    vals.tofile(names[0])
    off = np.fromfile(names[1], np.int32)
    bad = off.copy()
    bad[2] += 4                                            # a run that is no multiple of eight
    bad.tofile(names[1])
    with pytest.raises(ValueError):
        S.SpMM_ReadWeightFiles(*names, M, K)
    off.tofile(names[1])
    os.unlink(names[3])
    with pytest.raises(OSError):
        S.SpMM_ReadWeightFiles(*names, M, K)
    # an all-zero matrix: an empty values file is a valid one
    np.zeros((64, 64), np.float16).tofile(dense)
    S.Our_GenSparseMatrixBinFile(str(dense), 64, 64, *names)
    z = S.SpMM_ReadWeightFiles(*names, 64, 64)
    assert z.values.size == 0 and list(z.offsets) == [0, 0]


def test_weight_file_missing_input_exits_like_reference(tmp_path):
    code = ("import spmspm_amd as S; S.Our_GenSparseMatrixBinFile(%r, 64, 64, *[%r + str(i) for i in range(6)])"
            % (str(tmp_path / "missing.bin"), str(tmp_path / "o")))
    p = subprocess.run(["python", "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert p.returncode == 255  # exit(-1)
    assert "cannot be opened" in p.stdout


def test_cpu_reference_plumbing_config(oracle):
    """The CPU-only configuration: W 4096x4096 N(0, 0.02) at 50 % sparsity, X 4096x16 U(-1, 1), seed 0 -- product
    encoder == oracle encoder bit for bit, decode(encode(W)) == W, and the host SpMM on the encoded arrays agrees
    with a float64 product on a sample of rows (the full oracle product is the GPU tests' reference)."""
    from spmspm_amd.synthetic import WORKLOADS, make_activations, make_weight
    w = WORKLOADS["cpu_plumbing_4096"]
    M, K, N = w["M"], w["K"], w["N"]
    W = make_weight(M, K, w["sparsity"], seed=0, pruning=w["pruning"])
    X = make_activations(K, N, seed=0)
    comp = S.InitSparseMatrixA_bitmap(W)
    e = oracle.encode(W, M, K)
    assert np.array_equal(comp.values, e["values"]) and np.array_equal(comp.bitmaps, e["bitmap"])
    assert np.array_equal(comp.offsets, e["global"]) and np.array_equal(comp.median, e["median"])
    assert 0.49 < 1.0 - np.count_nonzero(W) / W.size < 0.51
    back = oracle.decode(comp.values, comp.bitmaps, comp.offsets, M, K)
    Wpos = W.copy()
    Wpos[Wpos == 0] = 0  # -0.0 is not stored and comes back as +0.0
    assert np.array_equal(back.view(np.uint16), Wpos.view(np.uint16))
    # host SpMM on the first four row blocks only (keeps the CPU suite short)
    rows = 256
    g1 = (rows // 64) * (K // 64)
    off = comp.offsets[:g1 + 1]
    C = oracle.spmm(comp.values[:int(off[-1])], comp.bitmaps[:g1 * 64], off, X, rows, N, K, 1, False).astype(np.float64)
    ref = X.astype(np.float64) @ W[:rows].astype(np.float64).T
    assert np.abs(C - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.linalg.norm(C - ref) <= 1e-3 * np.linalg.norm(ref)
