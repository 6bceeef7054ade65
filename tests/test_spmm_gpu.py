"""Parity of the HIP SpMM (through the C ABI) with the CPU oracle, the golden vectors and float64 mathematics."""
import os

import numpy as np
import pytest

import spmspm_amd as S
from conftest import assert_spmm_close
from spmspm_amd.synthetic import make_activations, make_weight

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch():
    import torch
    assert torch.cuda.is_available()
    return torch


class Device:
    """Uploads one compressed matrix the way the reference's harness does (kernel_benchmark/spmm_test.cu:334-372)."""

    def __init__(self, torch, comp):
        self.torch = torch
        self.c = comp
        dev = "cuda:0"
        vals = comp.values if comp.values.size else np.zeros(8, np.uint16)
        self.values = torch.from_numpy(vals.view(np.int16).copy()).to(dev)
        self.bitmaps = torch.from_numpy(comp.bitmaps.view(np.int64).copy()).to(dev)
        self.offsets = torch.from_numpy(comp.offsets.copy()).to(dev)
        self.median = torch.from_numpy(comp.median.copy() if comp.median.size else np.zeros(4, np.int32)).to(dev)
        self.max_nnz = torch.tensor([comp.max_nnz_rounded], dtype=torch.int32, device=dev)

    def spmm(self, X, split_k, entry="api", lib=None):
        """`lib`: a ctypes handle of another build of the library (the variants build) to call instead."""
        torch = self.torch
        N, K = X.shape
        M = self.c.M
        x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
        out = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")  # NaN-filled: C must be overwritten
        if lib is not None:
            stream = torch.cuda.current_stream().cuda_stream
            sk = split_k if split_k > 0 else S.SpMM_SplitK_Auto(M, N, K)
            if entry == "api":
                ws = torch.empty(max(4 * M * N * sk, 16), dtype=torch.uint8, device="cuda:0")
                err = lib.SpMM_SplitK_API(stream, self.values.data_ptr(), self.bitmaps.data_ptr(),
                                          self.offsets.data_ptr(), x.data_ptr(), out.data_ptr(), M, N, K,
                                          ws.data_ptr(), sk)
            else:
                ws = torch.empty(max(2 * M * N * sk, 16), dtype=torch.uint8, device="cuda:0")
                err = lib.SpMM_SplitK_API_bitmap_v3(stream, None, self.values.data_ptr(), self.offsets.data_ptr(),
                                                    self.median.data_ptr(), self.bitmaps.data_ptr(),
                                                    self.max_nnz.data_ptr(), x.data_ptr(), out.data_ptr(), M, N, K,
                                                    ws.data_ptr(), sk)
        elif entry == "api":
            nbytes = S.SpMM_WorkspaceBytes(M, N, K, split_k)
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda:0") if nbytes else None
            err = S.SpMM_SplitK_API(None, self.values, self.bitmaps, self.offsets, x, out, M, N, K, ws, split_k)
        else:
            ws = torch.empty(max(2 * M * N * max(split_k, 1), 16), dtype=torch.uint8, device="cuda:0")
            err = S.SpMM_SplitK_API_bitmap_v3(None, None, self.values, self.offsets, self.median, self.bitmaps,
                                              self.max_nnz, x, out, M, N, K, ws, split_k)
        assert err == 0, f"hipError_t {err}"
        torch.cuda.synchronize()
        return out.cpu().numpy().view(np.float16)


@pytest.fixture(scope="module")
def variants_lib():
    """The test build of the library (libSpMM_API_variants.so): the same entry points plus SpMM_Debug_SetKernelVariant."""
    import ctypes as C
    path = os.path.join(os.path.dirname(S.library_path()), "libSpMM_API_variants.so")
    assert os.path.exists(path), "build it with __graft_entry__.build()"
    L = C.CDLL(path)
    L.SpMM_SplitK_API.restype = C.c_int
    L.SpMM_SplitK_API.argtypes = [C.c_void_p] * 6 + [C.c_int] * 3 + [C.c_void_p, C.c_int]
    L.SpMM_SplitK_API_bitmap_v3.restype = C.c_int
    L.SpMM_SplitK_API_bitmap_v3.argtypes = [C.c_void_p] * 9 + [C.c_int] * 3 + [C.c_void_p, C.c_int]
    L.SpMM_Debug_SetKernelVariant.argtypes = [C.c_int]
    yield L
    L.SpMM_Debug_SetKernelVariant(2)


def _oracle_C(oracle, comp, X, split_k=1, partial_fp16=False):
    N, K = X.shape
    return oracle.spmm(comp.values, comp.bitmaps, comp.offsets, X, comp.M, N, K, split_k, partial_fp16)


SHAPES = [
    # M, K, N, sparsity, split_k
    (64, 64, 16, 0.5, 1),
    (64, 64, 8, 0.5, 1),
    (128, 192, 16, 0.7, 1),
    (256, 256, 32, 0.5, 1),
    (256, 512, 64, 0.6, 1),
    (128, 256, 128, 0.4, 1),
    (64, 128, 256, 0.5, 1),
    (256, 1024, 16, 0.7, 3),
    (256, 1024, 16, 0.7, 4),
    (192, 576, 8, 0.6, 2),
    (128, 640, 32, 0.5, 5),
    (128, 512, 64, 0.5, 7),
    (64, 320, 128, 0.5, 5),
    (512, 2048, 16, 0.9, 8),
    (1024, 1024, 16, 0.0, 2),
    (256, 256, 16, 1.0, 2),
]


@pytest.mark.parametrize("M,K,N,s,sk", SHAPES)
def test_matches_oracle(torch, oracle, M, K, N, s, sk):
    W = make_weight(M, K, s, seed=M + K + N)
    X = make_activations(K, N, seed=N)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    print(f"case M={M} K={K} N={N} s={s} sk={sk}", flush=True)
    C = dev.spmm(X, sk, "api")
    ref64 = X.astype(np.float64) @ W.astype(np.float64).T
    assert_spmm_close(C, _oracle_C(oracle, comp, X, sk, False), "api vs oracle")
    assert_spmm_close(C, ref64, "api vs float64")
    Cv3 = dev.spmm(X, sk, "v3")
    assert_spmm_close(Cv3, _oracle_C(oracle, comp, X, sk, True), "v3 vs oracle (fp16 partials)")
    assert_spmm_close(Cv3, ref64, "v3 vs float64")


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4], ids=["baseline", "stream", "shipped", "rows-everywhere", "wide-everywhere"])
def test_other_kernel_variants_match_oracle(torch, oracle, variant):
    """The comparison kernels (simple staging kernel, lane-per-bit decode through a dense LDS tile) stay correct, and
    so do the row-per-lane kernel at N >= 128 and the wide kernel at N = 64 and on fewer than 256 rows, which the
    shipped dispatch does not use there.
    They live in the test build of the library only (libSpMM_API_variants.so, -DSPMM_KEEP_VARIANTS), which also has
    the switch that selects them; the shipped library has neither."""
    import ctypes as C
    path = os.path.join(os.path.dirname(S.library_path()), "libSpMM_API_variants.so")
    assert os.path.exists(path), "build it with __graft_entry__.build()"
    assert not hasattr(S.library(), "SpMM_Debug_SetKernelVariant")
    L = C.CDLL(path)
    L.SpMM_SplitK_API.restype = C.c_int
    L.SpMM_SplitK_API.argtypes = [C.c_void_p] * 6 + [C.c_int] * 3 + [C.c_void_p, C.c_int]
    L.SpMM_Debug_SetKernelVariant.argtypes = [C.c_int]
    L.SpMM_Debug_SetKernelVariant(variant)
    try:
        for M, K, N, s, sk in [(128, 192, 16, 0.7, 1), (256, 1024, 8, 0.6, 3), (128, 512, 64, 0.5, 2),
                               (256, 256, 32, 0.0, 1), (320, 704, 64, 0.5, 3), (128, 512, 128, 0.6, 2),
                               (576, 384, 256, 0.3, 1)]:
            W = make_weight(M, K, s, seed=M + K + N)
            X = make_activations(K, N, seed=N)
            comp = S.InitSparseMatrixA_bitmap(W)
            dev = Device(torch, comp)
            print(f"case variant {variant} M={M} K={K} N={N} sk={sk}", flush=True)
            x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
            out = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")
            ws = torch.empty(max(4 * M * N * sk, 16), dtype=torch.uint8, device="cuda:0")
            err = L.SpMM_SplitK_API(torch.cuda.current_stream().cuda_stream, dev.values.data_ptr(),
                                    dev.bitmaps.data_ptr(), dev.offsets.data_ptr(), x.data_ptr(), out.data_ptr(),
                                    M, N, K, ws.data_ptr(), sk)
            assert err == 0
            torch.cuda.synchronize()
            C_out = out.cpu().numpy().view(np.float16)
            assert_spmm_close(C_out, _oracle_C(oracle, comp, X, sk, False), f"variant {variant} {M}x{K}x{N}")
    finally:
        L.SpMM_Debug_SetKernelVariant(2)


def _small_integer_problem(rng, M, K, N, density):
    """Inputs whose products and partial sums are small integers: fp32 accumulation is exact in any order, so the
    fp16 output is fixed bit for bit."""
    W = rng.choice(np.array([-3, -2, -1, 1, 2, 3], np.float16), (M, K))
    W[rng.random((M, K)) >= density] = 0
    X = rng.integers(-2, 3, (N, K)).astype(np.float16)
    return W, X


def test_exact_on_small_integers(torch, oracle):
    """Where fp32 accumulation is exact the result must be bit-identical to the oracle, any Split_K."""
    rng = np.random.default_rng(5)
    M, K, N = 256, 512, 16
    W, X = _small_integer_problem(rng, M, K, N, 0.4)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    want = _oracle_C(oracle, comp, X).view(np.uint16)
    for sk in (1, 2, 4, 8):
        for entry in ("api", "v3"):
            got = dev.spmm(X, sk, entry).view(np.uint16)
            assert np.array_equal(got, want), (sk, entry)


@pytest.mark.parametrize("N", [8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("density", [0.3, 0.85, 1.0])
def test_exact_on_small_integers_every_width_and_dense_tiles(torch, oracle, N, density):
    """Bit-identical results for every column-block width (N = 8 is the masked-column case of the 16-wide
    kernel), for group tiles above 3072 values (density 0.85 and 1.0: their last value chunks are fetched when the
    tile is staged), for the library's own Split_K and for explicit ones, through both entry points."""
    rng = np.random.default_rng(100 + N)
    M, K = 192, 640
    W, X = _small_integer_problem(rng, M, K, N, density)
    comp = S.InitSparseMatrixA_bitmap(W)
    if density >= 0.85:
        assert comp.max_nnz > 3072
    dev = Device(torch, comp)
    want = _oracle_C(oracle, comp, X).view(np.uint16)
    print(f"case N={N} density={density}", flush=True)
    for sk in (0, 1, 3, 10):
        assert np.array_equal(dev.spmm(X, sk, "api").view(np.uint16), want), ("api", sk)
    for sk in (1, 5):
        assert np.array_equal(dev.spmm(X, sk, "v3").view(np.uint16), want), ("v3", sk)


WIDE_CASES = [
    # M, K, N, density, explicit splits
    (256, 512, 128, 0.5, (1, 2, 8)),      # one workgroup per batch; Split_K = 8 leaves one k block per batch
    (320, 576, 128, 0.6, (1, 4)),         # five row blocks: the second workgroup has one wave with a row block;
                                          # nine k blocks in four batches: the last batch is empty
    (832, 1536, 256, 0.9, (1, 2, 5)),     # two column groups of 128; tiles above 3072 values
    (512, 1024, 128, 1.0, (1, 3)),        # every tile full: the last value chunks are fetched when the tile is staged
    (1024, 4096, 128, 0.05, (1, 2, 7)),   # nearly empty tiles, fewer value chunks than registers for them
    (256, 128, 384, 0.4, (1, 2)),         # two k blocks, three column groups
]


@pytest.mark.parametrize("M,K,N,density,splits", WIDE_CASES)
def test_wide_kernel_exact_on_small_integers(torch, oracle, variants_lib, M, K, N, density, splits):
    """The wide kernel (a group tile decoded once per 128 columns, X staged in LDS per workgroup) on shapes that
    exercise its corners.  The shipped dispatch sends only large matrices to it, so these small ones are run through
    the test build with the wide kernel forced, and once more through the shipped library (whatever kernel it picks).
    Bit-identical to the oracle where fp32 accumulation is exact: the library's own Split_K and explicit ones, fp32
    partial slabs ("api") and fp16 ones ("v3")."""
    rng = np.random.default_rng(M + K + N)
    W, X = _small_integer_problem(rng, M, K, N, density)
    W[64:128, :] = 0                      # an all-zero row block
    W[:, 64:128] = 0                      # and an all-zero column of group tiles
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    want = _oracle_C(oracle, comp, X).view(np.uint16)
    variants_lib.SpMM_Debug_SetKernelVariant(4)
    try:
        for sk in (0,) + tuple(splits):
            print(f"case wide M={M} K={K} N={N} density={density} sk={sk}", flush=True)
            assert np.array_equal(dev.spmm(X, sk, "api", lib=variants_lib).view(np.uint16), want), ("api", sk)
        for sk in splits[:2]:
            assert np.array_equal(dev.spmm(X, sk, "v3", lib=variants_lib).view(np.uint16), want), ("v3", sk)
    finally:
        variants_lib.SpMM_Debug_SetKernelVariant(2)
    for sk in (0, splits[-1]):
        assert np.array_equal(dev.spmm(X, sk, "api").view(np.uint16), want), ("shipped dispatch", sk)


def test_golden_fixtures_decode_on_device(torch, golden):
    """Every committed golden encoding multiplies to the same product as its dense input."""
    for name, g in golden.items():
        M, K = g["W"].shape
        Mt, Kt = M // 64 * 64, K // 64 * 64
        if Mt == 0 or Kt == 0:
            continue
        comp = S.CompressedMatrix(M=Mt, K=Kt, num_gtiles=int(g["scalars"][0]), values=g["values"],
                                  tile_counts=g["tile_counts"], median=g["median"], offsets=g["offsets"],
                                  bitmaps=g["bitmaps"], max_nnz=int(g["scalars"][1]))
        W = g["W"].view(np.float16)[:Mt, :Kt].astype(np.float64)
        if not np.isfinite(W).all():
            continue  # the special-values case is covered by test_special_values_propagate
        X = make_activations(Kt, 16, seed=1)
        C = Device(torch, comp).spmm(X, 1)
        assert_spmm_close(C, X.astype(np.float64) @ W.T, name)


def test_special_values_propagate(torch):
    """-0.0 is dropped by the encoder, NaN/inf/subnormal weights are kept and reach the right outputs."""
    M, K, N = 64, 128, 16
    W = np.zeros((M, K), np.float16)
    W[3, 5] = np.float16(np.nan)
    W[10, 70] = np.float16(np.inf)
    W[20, 9] = np.float16(6e-8)  # subnormal
    W[21, 9] = np.float16(-0.0)
    W[40, 127] = np.float16(2.0)
    X = np.ones((N, K), np.float16)
    comp = S.InitSparseMatrixA_bitmap(W)
    C = Device(torch, comp).spmm(X, 1)
    assert np.isnan(C[:, 3]).all() and np.isposinf(C[:, 10]).all()
    assert (C[:, 20] == np.float16(6e-8)).all() and (C[:, 40] == 2).all()
    rest = np.delete(C, [3, 10, 20, 40], axis=1)
    assert not rest.any()


def test_ragged_row_populations(torch, oracle):
    """Group tiles from empty to completely full inside one matrix, every strip offset exercised."""
    rng = np.random.default_rng(23)
    M, K, N = 256, 1024, 16
    W = (rng.standard_normal((M, K)) * 0.02).astype(np.float16)
    dens = rng.random((M // 64, K // 64))
    dens[0, 0], dens[1, 3], dens[2, 5] = 0.0, 1.0, 1.0
    for gm in range(M // 64):
        for gk in range(K // 64):
            blk = W[gm * 64:(gm + 1) * 64, gk * 64:(gk + 1) * 64]
            blk[rng.random((64, 64)) >= dens[gm, gk]] = 0
    W[64:128, 192:256] = np.where(W[64:128, 192:256] == 0, np.float16(0.01), W[64:128, 192:256])  # truly dense
    X = make_activations(K, N, seed=2)
    comp = S.InitSparseMatrixA_bitmap(W)
    assert comp.max_nnz == 4096
    dev = Device(torch, comp)
    for sk in (1, 3):
        assert_spmm_close(dev.spmm(X, sk), _oracle_C(oracle, comp, X, sk), f"ragged sk={sk}")


def test_reference_harness_inputs_and_error_metric(torch, oracle):
    """The reference's own generator and its sum-of-abs-diff check (kernel_benchmark/spmm_test_utils.h:88-110)."""
    M = K = 512
    N = 16
    W, X = oracle.init_host_matrices(M, K, N, 50, reseed=True)
    comp = S.InitSparseMatrixA_bitmap(W)
    C = Device(torch, comp).spmm(X, 1, "v3")
    ref = (X.astype(np.float64) @ W.astype(np.float64).T)
    ref16 = ref.astype(np.float16)
    assert_spmm_close(C, ref, "harness inputs")
    # values are multiples of 0.1-ish fp16 numbers: total error stays tiny relative to sum|C|
    assert oracle.total_error(ref16, C) <= 1e-3 * np.abs(ref).sum()


def test_auto_split_k_and_invariance(torch, oracle):
    M, K, N = 512, 4096, 16
    W = make_weight(M, K, 0.6, seed=4, pruning="magnitude")
    X = make_activations(K, N, seed=4)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    ref = X.astype(np.float64) @ W.astype(np.float64).T
    auto = S.SpMM_SplitK_Auto(M, N, K)
    assert auto > 1
    for sk in (0, 1, 2, 64, 1000):  # 0 = automatic; 1000 is clamped to K/64
        assert_spmm_close(dev.spmm(X, sk), ref, f"sk={sk}")


@pytest.mark.parametrize("M,K,N,s", [
    (256, 512, 16, 0.6),
    (65536, 192, 16, 0.7),    # three group tiles per row block
    (8192, 128, 32, 0.5),     # two group tiles per row block
    (1024, 4096, 8, 0.7),
    (4096, 1024, 64, 0.5),
    (2048, 2048, 128, 0.6),   # two column blocks
])
def test_library_split_repeated_calls_reuse_workspace(torch, oracle, M, K, N, s):
    """Split_K <= 0: the workspace's previous contents (garbage, or an earlier call's partial sums) must not
    matter."""
    W = make_weight(M, K, s, seed=M + K)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    nbytes = S.SpMM_WorkspaceBytes(M, N, K, 0)
    ws = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda:0")  # garbage on purpose
    for rep in range(3):
        X = make_activations(K, N, seed=rep)
        x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
        out = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")
        print(f"case M={M} K={K} N={N} rep={rep}", flush=True)
        err = S.SpMM_SplitK_API(None, dev.values, dev.bitmaps, dev.offsets, x, out, M, N, K, ws, 0)
        assert err == 0
        torch.cuda.synchronize()
        C = out.cpu().numpy().view(np.float16)
        assert_spmm_close(C, _oracle_C(oracle, comp, X), f"rep {rep}")


def test_library_split_needs_workspace(torch, capfd):
    """A missing workspace is reported before anything is launched."""
    t = torch.zeros(64, dtype=torch.int16, device="cuda:0")
    assert S.SpMM_WorkspaceBytes(512, 16, 4096, 0) > 0
    assert S.SpMM_SplitK_API(None, t, t, t, t, t, 512, 16, 4096, None, 0) == S.api.HIP_ERROR_INVALID_VALUE
    assert "workspace" in capfd.readouterr().out


def test_sized_entry_point_matches_and_refuses(torch, oracle, capfd):
    """SpMM_SplitK_API_Sized: the same result as SpMM_SplitK_API bit for bit with a workspace that is large enough,
    C untouched and hipErrorInvalidValue with one that is a byte short (explicit and automatic split)."""
    M, K, N = 512, 2048, 16
    W = make_weight(M, K, 0.6, seed=11)
    X = make_activations(K, N, seed=12)
    comp = S.InitSparseMatrixA_bitmap(W)
    d = Device(torch, comp)
    x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
    for sk in (0, 3):
        need = S.SpMM_WorkspaceBytes(M, N, K, sk)
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device="cuda:0")
        out = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")
        assert S.SpMM_SplitK_API_Sized(None, d.values, d.bitmaps, d.offsets, x, out, M, N, K, ws, need, sk) == 0
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint16), d.spmm(X, sk).view(np.uint16))
        out.fill_(0x7e00)
        assert S.SpMM_SplitK_API_Sized(None, d.values, d.bitmaps, d.offsets, x, out, M, N, K, ws, need - 1,
                                       sk) == S.api.HIP_ERROR_INVALID_VALUE
        torch.cuda.synchronize()
        assert (out == 0x7e00).all()
    assert "workspace" in capfd.readouterr().out


def test_linearity_at_full_size(torch):
    """OPT-13B QKV shape: C(X1 + X2) == C(X1) + C(X2) within the contract, and C(0) == 0."""
    M, K, N = 15360, 5120, 16
    W = make_weight(M, K, 0.6, seed=0, pruning="magnitude")
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    rng = np.random.default_rng(1)
    X1 = (rng.integers(-4, 5, (N, K)) / 8).astype(np.float16)
    X2 = (rng.integers(-4, 5, (N, K)) / 8).astype(np.float16)
    C1, C2, C12 = dev.spmm(X1, 0), dev.spmm(X2, 0), dev.spmm(X1 + X2, 0)
    assert_spmm_close(C12, C1.astype(np.float64) + C2.astype(np.float64), "linearity")
    assert not dev.spmm(np.zeros((N, K), np.float16), 0).any()
    # a sampled set of rows against float64
    rows = rng.choice(M, 64, replace=False)
    ref = X1.astype(np.float64) @ W[rows].astype(np.float64).T
    assert_spmm_close(C1[:, rows], ref, "sampled rows")


def test_target_shape_against_oracle(torch, oracle):
    """OPT-30B FFN1 28672x7168, 70 % sparse, N=16: whole output against the oracle."""
    M, K, N = 28672, 7168, 16
    W = make_weight(M, K, 0.7, seed=0)
    X = make_activations(K, N, seed=0)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    want = _oracle_C(oracle, comp, X)
    for sk in (0, 1):
        assert_spmm_close(dev.spmm(X, sk), want, f"target sk={sk}")
    assert_spmm_close(dev.spmm(X, 4, "v3"), want, "target v3 sk=4")


def test_cpu_reference_configuration_on_the_device(torch, oracle):
    """The configuration the reference runs on a CPU alone (4096x4096, 50 % random unstructured, N = 16, seed 0):
    the whole output against the oracle, with the library's split, unsplit, and through the 14-argument entry."""
    from spmspm_amd.synthetic import WORKLOADS
    w = WORKLOADS["cpu_plumbing_4096"]
    M, K, N = w["M"], w["K"], w["N"]
    W = make_weight(M, K, w["sparsity"], seed=0, pruning=w["pruning"])
    X = make_activations(K, N, seed=0)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    want = _oracle_C(oracle, comp, X)
    for sk in (0, 1):
        assert_spmm_close(dev.spmm(X, sk), want, f"4096x4096 sk={sk}")
    assert_spmm_close(dev.spmm(X, 3, "v3"), _oracle_C(oracle, comp, X, 3, True), "4096x4096 v3 sk=3")


@pytest.mark.parametrize("sparsity", [0.4, 0.5])
def test_opt30b_ffn1_full_size_other_batches_and_sparsities(torch, sparsity):
    """OPT-30B FFN1 28672x7168 at the denser settings of the benchmark set, N = 8 and 32, magnitude pruning:
    sampled rows against float64 through both entry points."""
    M, K = 28672, 7168
    W = make_weight(M, K, sparsity, seed=7, pruning="magnitude")
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    rng = np.random.default_rng(9)
    rows = rng.choice(M, 96, replace=False)
    Wrows = W[rows].astype(np.float64)
    del W
    for N in (8, 32):
        X = make_activations(K, N, seed=N)
        ref = X.astype(np.float64) @ Wrows.T
        assert_spmm_close(dev.spmm(X, 0)[:, rows], ref, f"s={sparsity} N={N} auto")
        assert_spmm_close(dev.spmm(X, 2, "v3")[:, rows], ref, f"s={sparsity} N={N} v3 sk=2")


@pytest.mark.parametrize("sparsity", [0.4, 0.5, 0.6, 0.7])
def test_opt30b_ffn1_sweep_random_unstructured(torch, oracle, sparsity):
    """The whole OPT-30B FFN1 sweep of the benchmark set: 28672x7168 with a uniform random mask at 40, 50, 60 and
    70 % sparsity, N = 8, 16 and 32.  N = 16: the full output against the oracle; N = 8 and 32: sampled rows
    against float64, automatic Split_K and an explicit one through the 14-argument entry point."""
    M, K = 28672, 7168
    W = make_weight(M, K, sparsity, seed=30 + int(sparsity * 10), pruning="random")
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    rng = np.random.default_rng(17)
    rows = rng.choice(M, 96, replace=False)
    Wrows = W[rows].astype(np.float64)
    del W
    X = make_activations(K, 16, seed=16)
    print(f"case s={sparsity} N=16 full output", flush=True)
    want = _oracle_C(oracle, comp, X)
    assert_spmm_close(dev.spmm(X, 0), want, f"s={sparsity} N=16 auto")
    assert_spmm_close(want[:, rows], X.astype(np.float64) @ Wrows.T, "oracle vs float64")
    for N in (8, 32):
        X = make_activations(K, N, seed=N)
        ref = X.astype(np.float64) @ Wrows.T
        print(f"case s={sparsity} N={N}", flush=True)
        assert_spmm_close(dev.spmm(X, 0)[:, rows], ref, f"s={sparsity} N={N} auto")
        assert_spmm_close(dev.spmm(X, 3, "v3")[:, rows], ref, f"s={sparsity} N={N} v3 sk=3")


OPT13B_LINEARS = [("opt13b_qkv", 15360, 5120), ("opt13b_out", 5120, 5120), ("opt13b_ffn1", 20480, 5120),
                  ("opt13b_ffn2", 5120, 20480)]


def _tuned_split(M, N, K):
    """Split_K of the shipped measured table (spmspm_amd/tuned/), or None if the shape is not listed."""
    path = os.path.join(os.path.dirname(S.__file__), "tuned", "splitk_mi355x.txt")
    for line in open(path):
        f = line.split()
        if len(f) == 4 and not line.startswith("#") and (int(f[0]), int(f[1]), int(f[2])) == (M, N, K):
            return int(f[3])
    return None


@pytest.mark.parametrize("name,M,K", OPT13B_LINEARS)
def test_opt13b_decode_linears_full_size(torch, oracle, name, M, K):
    """The four linears of an OPT-13B decode step at full size (60 % magnitude pruning, N = 16): the whole output
    against the oracle with the library's own Split_K and with the shipped table's measured one."""
    N = 16
    W = make_weight(M, K, 0.6, seed=M // 64 + K // 64, pruning="magnitude")
    X = make_activations(K, N, seed=5)
    comp = S.InitSparseMatrixA_bitmap(W)
    del W
    dev = Device(torch, comp)
    want = _oracle_C(oracle, comp, X)
    tuned = _tuned_split(M, N, K)
    assert tuned is not None, "the shipped table lists every OPT-13B linear"
    for sk in (0, tuned):
        print(f"case {name} sk={sk}", flush=True)
        assert_spmm_close(dev.spmm(X, sk), want, f"{name} sk={sk}")


def test_opt13b_two_layer_chain_against_oracle(torch, oracle):
    """Two OPT-13B-shaped layers chained on one stream the way the benchmark chains them (QKV, output projection on
    a fixed attention result, FFN1, FFN2 feeding the next layer's QKV): every buffer of the chain against the
    oracle run on the same inputs layer by layer."""
    N = 16
    rng = np.random.default_rng(77)
    comps, lins = [], []
    for layer in range(2):
        row = []
        for i, (name, M, K) in enumerate(OPT13B_LINEARS):
            W = make_weight(M, K, 0.6, seed=500 + 10 * layer + i, pruning="magnitude")
            # keep activations of order one down the chain: N(0, 0.02) weights shrink them by ~sqrt(0.4 K) * 0.02
            W = (W.astype(np.float32) * np.float32(1.0 / (0.02 * np.sqrt(0.4 * K)))).astype(np.float16)
            row.append(S.InitSparseMatrixA_bitmap(W))
            del W
        comps.append(row)
        lins.append([S.SparseLinear(c, split_k=0) for c in row])
    H = rng.uniform(-1, 1, (N, 5120)).astype(np.float16)
    A = rng.uniform(-1, 1, (N, 5120)).astype(np.float16)
    up = lambda a: torch.from_numpy(a.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    h, attn = up(H), up(A)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    got = []
    with torch.cuda.stream(side):
        x = h
        for lq, lo, l1, l2 in lins:
            q = lq(x, stream=side)
            o = lo(attn, stream=side)
            f = l1(o, stream=side)
            x = l2(f, stream=side)
            got.append((q, o, f, x))
    side.synchronize()

    def ref(c, Xh):
        Nn, Kk = Xh.shape
        return oracle.spmm(c.values, c.bitmaps, c.offsets, Xh, c.M, Nn, Kk, S.SpMM_SplitK_Auto(c.M, Nn, Kk), False)

    x_ref = H
    for layer, ((cq, co, c1, c2), (q, o, f, x)) in enumerate(zip(comps, got)):
        print(f"chain layer {layer}", flush=True)
        # every linear is checked on the input the device actually gave it, so one rounding difference upstream
        # does not decide the comparisons downstream; the chained buffers are compared as well
        x_in = H if layer == 0 else got[layer - 1][3].cpu().numpy()
        assert_spmm_close(q.cpu().numpy(), ref(cq, x_in), f"layer {layer} qkv")
        assert_spmm_close(o.cpu().numpy(), ref(co, A), f"layer {layer} out-proj")
        assert_spmm_close(f.cpu().numpy(), ref(c1, o.cpu().numpy()), f"layer {layer} ffn1")
        assert_spmm_close(x.cpu().numpy(), ref(c2, f.cpu().numpy()), f"layer {layer} ffn2")
        o_ref = ref(co, A)
        x_ref = ref(c2, ref(c1, o_ref))
        assert_spmm_close(x.cpu().numpy(), x_ref, f"layer {layer} chained output")


def test_opt13b_decode_chain_at_full_depth(torch):
    """The OPT-13B decode-step configuration at its stated depth: 40 layers x {QKV, out-proj, FFN1, FFN2} at N = 16,
    60 % magnitude pruning, built the way the benchmark builds it (four encoded matrices, a resident copy of each per
    layer: 11.8 GB of compressed weights), chained on one stream.  Every one of the 160 linears is checked on 64
    sampled rows against a float64 product of the dense weights with the input that linear was actually given; the
    attention result fed to the output projection differs from layer to layer, so no two layers compute the same."""
    N, layers = 16, 40
    dev = "cuda:0"
    first, dense = [], []
    for i, (name, M, K) in enumerate(OPT13B_LINEARS):
        W = make_weight(M, K, 0.6, seed=900 + i, pruning="magnitude")
        # keep activations of order one down the chain (see the two-layer test)
        W = (W.astype(np.float32) * np.float32(1.0 / (0.02 * np.sqrt(0.4 * K)))).astype(np.float16)
        first.append(S.SparseLinear(S.InitSparseMatrixA_bitmap(W), device=dev, split_k=0))
        dense.append(torch.from_numpy(W.view(np.int16)).to(dev).view(torch.float16))
        del W
    chain = [[l if j == 0 else l.clone() for l in first] for j in range(layers)]
    g = torch.Generator(device=dev)
    g.manual_seed(4)
    h = (torch.rand((N, 5120), generator=g, device=dev) * 2 - 1).half()
    attn = [(torch.rand((N, 5120), generator=g, device=dev) * 2 - 1).half() for _ in range(layers)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    got = []
    with torch.cuda.stream(side):
        x = h
        for j, (lq, lo, l1, l2) in enumerate(chain):
            q = lq(x, stream=side)
            o = lo(attn[j], stream=side)
            f = l1(o, stream=side)
            x2 = l2(f, stream=side)
            got.append(((x, q), (attn[j], o), (o, f), (f, x2)))
            x = x2
    side.synchronize()
    rng = np.random.default_rng(8)
    worst = 0.0
    for j, pairs in enumerate(got):
        for (name, M, K), Wd, (xin, y) in zip(OPT13B_LINEARS, dense, pairs):
            rows = torch.from_numpy(rng.choice(M, 64, replace=False)).to(dev)
            ref = xin.double() @ Wd[rows].double().t()
            d = y[:, rows].double() - ref
            assert torch.isfinite(y).all(), f"layer {j} {name}: non-finite output"
            rel = float(d.norm() / ref.norm())
            frac = float(d.abs().max() / ref.abs().max())
            assert rel <= 1e-3 and frac <= 1e-2, f"layer {j} {name}: rel-L2 {rel:.2e}, max {frac:.2e}"
            worst = max(worst, rel)
    print(f"40-layer chain: worst rel-L2 over 160 linears {worst:.2e}", flush=True)


def test_opt66b_ffn2_full_size_wide_batches(torch):
    """OPT-66B FFN2 9216x36864 at 40 % sparsity, N = 64 and 128 (the widest configuration of the benchmark set):
    sampled rows against float64, and the sum over all rows of every output column against the same sum taken
    on the weights first (sum_m C[n][m] = sum_k X[n][k] * sum_m W[m][k])."""
    M, K = 9216, 36864
    W = make_weight(M, K, 0.4, seed=3)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    rng = np.random.default_rng(5)
    rows = rng.choice(M, 48, replace=False)
    Wrows = W[rows].astype(np.float64)
    colsum = np.zeros(K, np.float64)
    for r0 in range(0, M, 1024):  # in slices: a float64 copy of W would be 2.7 GB
        colsum += W[r0:r0 + 1024].astype(np.float32).sum(axis=0, dtype=np.float64)
    del W
    for N in (64, 128):
        X = (rng.integers(-8, 9, (N, K)) / 16).astype(np.float16)
        for sk in (0, 3):
            C = dev.spmm(X, sk)
            assert_spmm_close(C[:, rows], X.astype(np.float64) @ Wrows.T, f"N={N} sk={sk} sampled rows")
            got, want = C.astype(np.float64).sum(axis=1), X.astype(np.float64) @ colsum
            # every output carries its own fp16 rounding (2^-11 relative); M of them add up in quadrature
            tol = 4.0 * 2.0 ** -11 * np.sqrt((C.astype(np.float64) ** 2).sum(axis=1)) + 1e-6
            assert (np.abs(got - want) <= tol).all(), f"N={N} sk={sk}: column sums off by {np.abs(got - want).max():.3e}"


def test_error_returns_on_device(torch, capfd):
    t = torch.zeros(16, dtype=torch.int16, device="cuda:0")
    assert S.SpMM_SplitK_API(None, t, t, t, t, t, 64, 48, 64, None, 1) == S.api.HIP_ERROR_UNKNOWN
    assert "Unsupported N dimension 48" in capfd.readouterr().out
    assert S.SpMM_SplitK_API_bitmap_v3(None, None, t, t, t, t, t, t, t, 64, 16, 96, t, 1) == S.api.HIP_ERROR_INVALID_VALUE
    torch.cuda.synchronize()


def test_stream_argument_is_honoured(torch, oracle):
    M, K, N = 256, 512, 16
    W = make_weight(M, K, 0.5, seed=8)
    X = make_activations(K, N, seed=8)
    comp = S.InitSparseMatrixA_bitmap(W)
    lin = S.SparseLinear(comp, split_k=2)
    x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0").view(torch.float16)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        y = lin(x, stream=side)
    side.synchronize()
    assert_spmm_close(y.cpu().numpy(), _oracle_C(oracle, comp, X, 2), "side stream")


def test_calls_recorded_in_a_hip_graph_replay_correctly(torch, oracle):
    """Three chained SpMM calls (split and unsplit) captured from a stream and replayed: every replay, with eager
    work and synchronisations of the program's own in between, must give what the eager chain gives."""
    M, K, N = 512, 512, 16
    comps = [S.InitSparseMatrixA_bitmap(make_weight(M, K, 0.6, seed=40 + i)) for i in range(3)]
    lins = [S.SparseLinear(c, split_k=sk) for c, sk in zip(comps, (1, 4, 0))]
    for l in lins:
        l.workspace(N)
    x0 = torch.zeros((N, K), dtype=torch.float16, device="cuda:0")
    bufs = [torch.empty((N, M), dtype=torch.float16, device="cuda:0") for _ in range(3)]

    def chain(stream):
        x = x0
        for l, b in zip(lins, bufs):
            x = l(x, out=b, stream=stream)

    def expected(X):
        x = X
        for c, sk in zip(comps, (1, 4, S.SpMM_SplitK_Auto(M, N, K))):
            x = oracle.spmm(c.values, c.bitmaps, c.offsets, x, M, N, K, sk, False)
        return x

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain(side)  # warm-up outside the capture
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            chain(side)
        for rep in range(4):
            X = (make_activations(K, N, seed=100 + rep).astype(np.float32) * 8).astype(np.float16)
            x0.copy_(torch.from_numpy(X.view(np.int16).copy()).to("cuda:0").view(torch.float16))
            for b in bufs:
                b.fill_(float("nan"))
            print(f"graph replay {rep}", flush=True)
            g.replay()
            side.synchronize()
            got = bufs[2].cpu().numpy()
            assert_spmm_close(got, expected(X), f"replay {rep}")
            chain(side)  # eager work between replays
            side.synchronize()
            assert np.array_equal(got.view(np.uint16), bufs[2].cpu().numpy().view(np.uint16)), "eager != replay"


@pytest.mark.parametrize("M,K,N,s,sk", [(256, 512, 16, 0.6, 1), (512, 1024, 8, 0.7, 4), (1024, 256, 32, 0.5, 0),
                                        (320, 4096, 64, 0.6, 0), (128, 128, 128, 0.3, 2), (512, 768, 128, 0.6, 1),
                                        (320, 1024, 256, 0.5, 3)])
@pytest.mark.parametrize("act", [0, 1, 2])
@pytest.mark.parametrize("with_bias", [False, True])
def test_bias_activation_entry_point(torch, oracle, M, K, N, s, sk, act, with_bias):
    """SpMM_SplitK_API_BiasAct against the oracle's fp32 tail and against float64; a garbage workspace on entry."""
    W = make_weight(M, K, s, seed=M + N + act)
    X = make_activations(K, N, seed=K + act)
    comp = S.InitSparseMatrixA_bitmap(W)
    dev = Device(torch, comp)
    bias = (np.random.default_rng(M).uniform(-2, 2, M)).astype(np.float16) if with_bias else None
    b = None if bias is None else torch.from_numpy(bias.view(np.int16).copy()).to("cuda:0")
    x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
    out = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")
    nbytes = S.SpMM_WorkspaceBytesBiasAct(M, N, K, sk)
    assert nbytes >= 4 * M * N
    ws = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda:0")
    print(f"case M={M} K={K} N={N} sk={sk} act={act} bias={with_bias}", flush=True)
    err = S.SpMM_SplitK_API_BiasAct(None, dev.values, dev.bitmaps, dev.offsets, x, out, M, N, K, ws, sk, b, act)
    assert err == 0
    torch.cuda.synchronize()
    C = out.cpu().numpy().view(np.float16)
    sk_eff = sk if sk > 0 else S.SpMM_SplitK_Auto(M, N, K)
    ref = oracle.spmm_bias_act(comp.values, comp.bitmaps, comp.offsets, X, M, N, K, sk_eff, bias, act)
    assert_spmm_close(C, ref, "vs oracle")
    pre = X.astype(np.float64) @ W.astype(np.float64).T + (0 if bias is None else bias.astype(np.float64)[None, :])
    ref64 = pre if act == 0 else (np.maximum(pre, 0) if act == 1
                                  else 0.5 * pre * (1 + np.tanh(0.7978845608028654 * (pre + 0.044715 * pre ** 3))))
    assert_spmm_close(C, ref64, "vs float64")
    if act == 0 and not with_bias:  # the tail switched off is the plain entry point, bit for bit
        assert np.array_equal(C.view(np.uint16), dev.spmm(X, sk).view(np.uint16))


def test_bias_activation_errors_and_layer(torch, oracle, capfd):
    t = torch.zeros(64, dtype=torch.int16, device="cuda:0")
    assert S.SpMM_SplitK_API_BiasAct(None, t, t, t, t, t, 64, 16, 64, t, 1, None, 7) == S.api.HIP_ERROR_INVALID_VALUE
    assert "activation" in capfd.readouterr().out
    assert S.SpMM_SplitK_API_BiasAct(None, t, t, t, t, t, 64, 16, 64, None, 1, None, 1) == S.api.HIP_ERROR_INVALID_VALUE
    assert "workspace" in capfd.readouterr().out
    M, K, N = 256, 256, 16
    W = make_weight(M, K, 0.5, seed=3)
    X = make_activations(K, N, seed=3)
    comp = S.InitSparseMatrixA_bitmap(W)
    bias = np.linspace(-1, 1, M).astype(np.float16)
    lin = S.SparseLinear(comp, bias=bias, activation=S.ACT_RELU)
    y = lin(torch.from_numpy(X.view(np.int16).copy()).to("cuda:0").view(torch.float16))
    torch.cuda.synchronize()
    ref = oracle.spmm_bias_act(comp.values, comp.bitmaps, comp.offsets, X, M, N, K, S.SpMM_SplitK_Auto(M, N, K), bias, 1)
    assert_spmm_close(y.cpu().numpy(), ref, "layer")


def test_seeded_random_shapes(torch, oracle):
    """Forty seeded random cases (shape, columns, density incl. nearly empty and nearly full, split) through both
    entry points against the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        M = 64 * int(rng.integers(1, 9))
        K = 64 * int(rng.integers(1, 25))
        N = int(rng.choice([8, 16, 32, 64, 128]))
        s = float(rng.choice([0.0, 0.05, 0.3, 0.5, 0.7, 0.9, 0.99]))
        sk = int(rng.integers(0, min(8, K // 64) + 1))
        W = make_weight(M, K, s, seed=1000 + case)
        X = make_activations(K, N, seed=2000 + case)
        comp = S.InitSparseMatrixA_bitmap(W)
        dev = Device(torch, comp)
        print(f"case {case}: M={M} K={K} N={N} s={s} sk={sk}", flush=True)
        sk_eff = sk if sk > 0 else S.SpMM_SplitK_Auto(M, N, K)
        sk_eff = min(sk_eff, K // 64)
        assert_spmm_close(dev.spmm(X, sk), _oracle_C(oracle, comp, X, sk_eff), f"case {case} api")
        if sk > 0:
            assert_spmm_close(dev.spmm(X, sk, "v3"), _oracle_C(oracle, comp, X, sk_eff, True), f"case {case} v3")


def test_randomized_exact_on_every_dispatch(torch, variants_lib):
    """Eighty seeded random problems in small integers (exact in fp32, so the product is known bit for bit from a
    float64 product) through the shipped dispatch, the row-per-lane kernel everywhere and the wide kernel everywhere:
    up to 2048 rows and 4096 columns, every supported width up to 384 columns, a different density for every group
    tile of a matrix (empty, nearly empty, ..., full side by side), the library's own split, no split, and two
    random ones of which one may exceed the number of k blocks (the library then uses one batch per k block)."""
    rng = np.random.default_rng(31)
    stream = torch.cuda.current_stream().cuda_stream
    try:
        for case in range(80):
            M = 64 * int(rng.integers(1, 33))
            K = 64 * int(rng.integers(1, 65))
            N = int(rng.choice([8, 16, 32, 64, 128, 256, 384]))
            dens = rng.choice([0.0, 0.02, 0.3, 0.5, 0.8, 1.0], size=(M // 64, K // 64), p=[0.1, 0.1, 0.4, 0.2, 0.1, 0.1])
            W = rng.integers(-2, 3, (M, K)).astype(np.float16)
            W[rng.random((M, K)) >= np.kron(dens, np.ones((64, 64)))] = 0
            X = rng.integers(-2, 3, (N, K)).astype(np.float16)
            want = (X.astype(np.float64) @ W.astype(np.float64).T).astype(np.float16).view(np.uint16)
            dev = Device(torch, S.InitSparseMatrixA_bitmap(W))
            nkb = K // 64
            splits = sorted({0, 1, int(rng.integers(1, nkb + 1)), int(rng.integers(1, nkb + 4))})
            print(f"case {case}: M={M} K={K} N={N} splits={splits}", flush=True)
            for variant in (2, 3, 4):
                if variant == 4 and (N % 64 != 0 or M < 256):
                    continue
                variants_lib.SpMM_Debug_SetKernelVariant(variant)
                for sk in splits:
                    got = dev.spmm(X, sk, "api", lib=variants_lib).view(np.uint16)
                    assert np.array_equal(got, want), (case, M, K, N, variant, sk)
    finally:
        variants_lib.SpMM_Debug_SetKernelVariant(2)


@pytest.mark.parametrize("args", [(1024, 1024, 16, 70, 2), (2048, 512, 8, 50, 1), (512, 4096, 32, 60, 4),
                                  (1024, 2048, 64, 40, 3), (256, 1024, 128, 90, 2)])
def test_cpp_caller_of_the_library(args):
    """tests/cpp/harness.cpp, built against libSpMM_API.so by build(): the reference harness's call sequence from
    C++ (encoder overload with the reference's signature, 14-argument SpMM on the null stream, then the shorter
    entry point), checked inside the program against a float64 product of sampled rows."""
    import subprocess
    exe = os.path.join(os.path.dirname(S.library_path()), "spmm_harness")
    assert os.path.exists(exe), "build it with __graft_entry__.build()"
    print("harness", args, flush=True)
    p = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "PASS" in p.stdout and "spmm-gfx950" in p.stdout


def test_tuner_records_a_measured_split_that_the_library_then_uses(torch, oracle, tmp_path):
    from spmspm_amd import tuner
    M, K, N, s = 2048, 4096, 16, 0.6
    S.SpMM_SplitK_TableClear()
    try:
        res = tuner.tune([(M, K)], N, sparsity=s, iters=10, candidates=[1, 2, 4, 8])
        best, times = res[(M, N, K)]
        assert best in (1, 2, 4, 8) and set(times) == {1, 2, 4, 8} and all(t > 0 for t in times.values())
        assert S.SpMM_SplitK_Auto(M, N, K) == best
        path = tmp_path / "splitk.txt"
        assert S.SpMM_SplitK_TableSave(path) == 1
        # a split that only the table can have chosen, and results that do not depend on it
        S.SpMM_SplitK_TableSet(M, N, K, 7)
        W, X = make_weight(M, K, s, seed=21), make_activations(K, N, seed=21)
        comp = S.InitSparseMatrixA_bitmap(W)
        x = torch.from_numpy(X.view(np.int16).copy()).cuda().view(torch.float16)
        layer = S.SparseLinear(comp)  # split_k=0: the library's choice, i.e. the table's
        assert layer.workspace(N).numel() == 4 * M * N * 7
        got = layer(x)
        torch.cuda.synchronize()
        want = oracle.spmm(comp.values, comp.bitmaps, comp.offsets, X, M, N, K, 7, False)
        assert_spmm_close(got.cpu().numpy(), want)
        S.SpMM_SplitK_TableClear()
        assert S.SpMM_SplitK_TableLoad(path) == 1 and S.SpMM_SplitK_Auto(M, N, K) == best
    finally:
        S.SpMM_SplitK_TableClear()
