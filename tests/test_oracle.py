"""Pins the CPU oracle: reference-held known answers, golden vectors written by the
reference's own encoder, closed forms, inverses and float64 mathematics."""
import numpy as np
import pytest

# (M=K, group tiles, padded NNZ, max_nnz rounded to x64) printed by the reference's harness for
# S=50 with its un-seeded glibc rand() generator (csrc/out:4,16,28,40,52,64,76).
RECORDED = [
    (256, 16, 32816, 2112),
    (512, 64, 131168, 2176),
    (1024, 256, 525360, 2176),
    (2048, 1024, 2100296, 2176),
    (4096, 4096, 8405952, 2240),
    (8192, 16384, 33613608, 2240),
]
RECORDED_LARGE = [(16384, 65536, 134455104, 2240)]


@pytest.mark.parametrize("M,G,nnz,max_nnz", RECORDED)
def test_reference_recorded_known_answers(oracle, M, G, nnz, max_nnz):
    W, _ = oracle.init_host_matrices(M, M, M, 50, reseed=True)
    e = oracle.encode(W, M, M)
    assert e["num_gtiles"] == G
    assert int(e["global"][-1]) == nnz
    assert oracle.round_max_nnz(e["max_nnz"]) == max_nnz


@pytest.mark.parametrize("M,G,nnz,max_nnz", RECORDED_LARGE)
def test_reference_recorded_known_answer_16384(oracle, M, G, nnz, max_nnz):
    # N only affects draws made after W, so a narrow X keeps this case cheap.
    W, _ = oracle.init_host_matrices(M, M, 1, 50, reseed=True)
    e = oracle.encode(W, M, M)
    assert (e["num_gtiles"], int(e["global"][-1]), oracle.round_max_nnz(e["max_nnz"])) == (G, nnz, max_nnz)


def test_golden_vectors(oracle, golden):
    for name, c in golden.items():
        M, K = c["W"].shape
        e = oracle.encode(c["W"], M, K)
        G = int(c["scalars"][0])
        assert e["num_gtiles"] == G, name
        assert e["max_nnz"] == int(c["scalars"][1]), name
        assert np.array_equal(e["values"], c["values"]), name
        assert np.array_equal(e["global"], c["offsets"]), name
        assert np.array_equal(e["median"], c["median"]), name
        assert np.array_equal(e["bitmap"][:64 * G], c["bitmaps"]), name
        assert np.array_equal(e["tile_cnt"][:64 * G], c["tile_counts"]), name


def test_against_reference_build_when_present(oracle):
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(7)
    for M, K, s in [(64, 64, 0.3), (192, 320, 0.6), (512, 256, 0.8), (128, 1024, 0.95)]:
        W = (rng.standard_normal((M, K)) * 0.02).astype(np.float16)
        W[rng.random((M, K)) < s] = 0
        a, b = oracle.encode(W, M, K), oracle.ref_encode(W, M, K)
        for k in ("values", "tile_cnt", "median", "global", "bitmap"):
            assert np.array_equal(a[k], b[k]), (M, K, s, k)
        assert a["max_nnz"] == b["max_nnz"]


def test_all_dense_closed_form(oracle):
    M, K = 128, 192
    W = np.arange(1, M * K + 1, dtype=np.float32).reshape(M, K)
    W = (W % 2047 + 1).astype(np.float16)
    e = oracle.encode(W, M, K)
    G = 2 * 3
    assert e["num_gtiles"] == G and e["max_nnz"] == 4096
    assert np.all(e["bitmap"] == np.uint64(0xFFFFFFFFFFFFFFFF))
    assert np.array_equal(e["global"], 4096 * np.arange(G + 1))
    assert np.array_equal(e["median"], np.tile([0, 1024, 2048, 3072], G))
    assert np.all(e["tile_cnt"] == 64)


def test_all_zero_closed_form(oracle):
    e = oracle.encode(np.zeros((128, 64), np.float16), 128, 64)
    assert e["num_gtiles"] == 2 and e["max_nnz"] == 0 and e["values"].size == 0
    assert not e["bitmap"].any() and not e["global"].any() and not e["median"].any()


def test_tile_index_and_bit_closed_form(oracle):
    """A single non-zero at (row, col) must land in tile t = ((gm*(K/64)+gk)*4+strip)*16 + q*4 + j*2 + i, bit r*8+c."""
    M, K = 128, 192
    rng = np.random.default_rng(3)
    for _ in range(200):
        row, col = int(rng.integers(M)), int(rng.integers(K))
        W = np.zeros((M, K), np.float16)
        W[row, col] = 1.5
        e = oracle.encode(W, M, K)
        gm, gk = row // 64, col // 64
        strip, i, r = (row % 64) // 16, (row % 16) // 8, row % 8
        q, j, c = (col % 64) // 16, (col % 16) // 8, col % 8
        t = ((gm * (K // 64) + gk) * 4 + strip) * 16 + q * 4 + j * 2 + i
        nz = np.flatnonzero(e["bitmap"])
        assert list(nz) == [t]
        assert int(e["bitmap"][t]) == 1 << (r * 8 + c)
        g = gm * (K // 64) + gk
        assert np.array_equal(np.diff(e["global"]), 8 * (np.arange(e["num_gtiles"]) == g))
        assert e["values"][e["global"][g]] == np.float16(1.5).view(np.uint16)
        assert not e["values"][e["global"][g] + 1:e["global"][g] + 8].any()  # padding is +0.0
        assert list(e["median"][4 * g:4 * g + 4]) == [0] + [int(strip < s) for s in (1, 2, 3)]


def test_value_order_inside_group_tile(oracle):
    """Values follow storage-tile order and, inside a tile, ascending bit order."""
    M = K = 64
    W = (np.arange(M * K, dtype=np.float32).reshape(M, K) % 1000 + 1).astype(np.float16)
    e = oracle.encode(W, M, K)
    expect = []
    for strip in range(4):
        for q in range(4):
            for j in range(2):
                for i in range(2):
                    blk = W[strip * 16 + i * 8:strip * 16 + i * 8 + 8, q * 16 + j * 8:q * 16 + j * 8 + 8]
                    expect.append(blk.reshape(-1))
    assert np.array_equal(e["values"], np.concatenate(expect).view(np.uint16))


def test_special_values(oracle):
    W = np.zeros((64, 64), np.uint16)
    W[0, 0] = 0x8000  # -0.0 dropped
    W[0, 1] = 0x0001  # smallest subnormal kept
    W[0, 2] = 0x7e00  # NaN kept
    W[0, 3] = 0xfc00  # -inf kept
    e = oracle.encode(W, 64, 64)
    assert int(e["bitmap"][0]) == 0b1110
    assert list(e["values"][:3]) == [0x0001, 0x7e00, 0xfc00]
    assert int(e["global"][1]) == 8


def test_invariants_and_roundtrip(oracle):
    rng = np.random.default_rng(11)
    for M, K, s in [(64, 64, 0.5), (256, 128, 0.7), (192, 448, 0.4)]:
        W = (rng.standard_normal((M, K)) * 0.02).astype(np.float16)
        W[rng.random((M, K)) < s] = 0
        e = oracle.encode(W, M, K)
        G = e["num_gtiles"]
        pc = np.array([bin(int(b)).count("1") for b in e["bitmap"]])
        assert np.array_equal(pc, e["tile_cnt"])
        per_group = pc.reshape(G, 64).sum(1)
        assert np.array_equal(np.diff(e["global"]), (per_group + 7) // 8 * 8)
        strips = pc.reshape(G, 4, 16).sum(2)
        assert np.array_equal(e["median"].reshape(G, 4)[:, 1:], np.cumsum(strips, 1)[:, :3])
        assert not e["median"].reshape(G, 4)[:, 0].any()
        assert e["max_nnz"] == int(np.diff(e["global"]).max())
        back = oracle.decode(e["values"], e["bitmap"], e["global"], M, K)
        assert np.array_equal(back.view(np.uint16), W.view(np.uint16) * (W != 0))  # -0.0 -> +0.0


def test_half_conversions_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint16)
    ours = np.array([oracle.half_to_float(int(x)) for x in h[::7]], np.float32)
    ref = h[::7].view(np.float16).astype(np.float32)
    assert np.array_equal(ours.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    rng = np.random.default_rng(5)
    f = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-2, 1, 300, 7e4)])
    f = np.concatenate([f, np.array([0.0, -0.0, 65504, 65519.99, 65520, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), 1),
                                     2.0 ** -24, 6.1e-5, np.inf, -np.inf], np.float32)])
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([oracle.float_to_half(float(x)) for x in f], np.uint16)
    assert np.array_equal(got, want)


def test_splitk_partition_closed_form(oracle):
    for nkb in (1, 5, 9, 10, 80, 112, 576):
        for sk in (1, 2, 3, 4, 7, 8, 13):
            avg = -(-nkb // sk)
            covered = []
            for b in range(sk):
                first, cnt = oracle.splitk_range(nkb * 64, sk, b)
                assert first == b * avg
                assert cnt == max(0, min(avg, nkb - first))
                covered += list(range(first, first + cnt))
            assert covered == list(range(nkb))
            # where the reference's remainder formula is in bounds it is the same partition
            pad = avg * sk - nkb
            if (sk - 1) * avg <= nkb:
                assert oracle.splitk_range(nkb * 64, sk, sk - 1)[1] == avg - pad


def _dense_case(rng, M, K, N, s):
    W = (rng.standard_normal((M, K)) * 0.02).astype(np.float16)
    W[rng.random((M, K)) < s] = 0
    X = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    return W, X


def test_spmm_matches_float64_gemm(oracle):
    from conftest import assert_spmm_close
    rng = np.random.default_rng(13)
    for M, K, N, s in [(64, 64, 8, 0.5), (128, 320, 16, 0.7), (256, 192, 32, 0.4), (64, 1024, 64, 0.6)]:
        W, X = _dense_case(rng, M, K, N, s)
        e = oracle.encode(W, M, K)
        ref = X.astype(np.float64) @ W.astype(np.float64).T
        assert np.allclose(oracle.gemm_f64(W, X, M, N, K), ref, rtol=0, atol=1e-12)
        for sk, pf in [(1, False), (2, False), (3, True), (5, True)]:
            C = oracle.spmm(e["values"], e["bitmap"], e["global"], X, M, N, K, sk, pf)
            assert_spmm_close(C, ref, f"{M}x{K}x{N} sk={sk}")
        # exactness where fp32 accumulation is exact: small integers
        Wi = rng.integers(-3, 4, (M, K)).astype(np.float16)
        Xi = rng.integers(-2, 3, (N, K)).astype(np.float16)
        ei = oracle.encode(Wi, M, K)
        Ci = oracle.spmm(ei["values"], ei["bitmap"], ei["global"], Xi, M, N, K, 1, False)
        assert np.array_equal(Ci.astype(np.float64), Xi.astype(np.float64) @ Wi.astype(np.float64).T)


def test_spmm_brute_force_tiny(oracle):
    rng = np.random.default_rng(17)
    M = K = 64
    N = 8
    W, X = _dense_case(rng, M, K, N, 0.8)
    e = oracle.encode(W, M, K)
    C = oracle.spmm(e["values"], e["bitmap"], e["global"], X, M, N, K, 1, False)
    for m in range(0, M, 5):
        for n in range(N):
            s = np.float32(0)
            for k in range(K):
                s = np.float32(s + np.float32(W[m, k]) * np.float32(X[n, k]))
            assert C[n, m] == np.float16(s)


def test_splitk_reduce_and_error_metric(oracle):
    rng = np.random.default_rng(19)
    M, N, sk = 64, 8, 3
    ws = rng.standard_normal((sk, N, M)).astype(np.float16)
    want = ws.astype(np.float32).sum(0).astype(np.float16)
    assert np.array_equal(oracle.splitk_reduce_fp16(ws, M, N, sk), want)
    a, b = ws[0], ws[1]
    assert np.isclose(oracle.total_error(a, b), np.abs(a.astype(np.float64) - b.astype(np.float64)).sum())


# ---------------------------------------------------------------- bias + activation tail

def _gelu64(x):
    return 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))


@pytest.mark.parametrize("act", [0, 1, 2])
@pytest.mark.parametrize("with_bias", [False, True])
def test_spmm_bias_act_against_float64(oracle, act, with_bias):
    """C = fp16(act(W X + bias)) against numpy float64: a wrong sign, a bias added after the activation or along
    the wrong axis, or ReLU/GELU swapped all fail this."""
    from spmspm_amd.synthetic import make_activations, make_weight
    M, K, N = 192, 256, 16
    W = make_weight(M, K, 0.6, seed=5)
    X = make_activations(K, N, seed=5)
    e = oracle.encode(W, M, K)
    vals, glo, bmp = e["values"], e["global"], e["bitmap"]
    bias = (np.linspace(-1.5, 1.5, M)).astype(np.float16) if with_bias else None
    got = oracle.spmm_bias_act(vals, bmp, glo, X, M, N, K, 2, bias, act).astype(np.float64)
    pre = X.astype(np.float64) @ W.astype(np.float64).T
    if with_bias:
        pre = pre + bias.astype(np.float64)[None, :]
    ref = pre if act == 0 else (np.maximum(pre, 0.0) if act == 1 else _gelu64(pre))
    assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.linalg.norm(got - ref) <= 2e-3 * np.linalg.norm(ref)
    if act == 1:
        assert (got >= 0).all() and (got[pre < -1e-2] == 0).all()


def test_spmm_bias_act_reduces_to_plain_spmm(oracle):
    from spmspm_amd.synthetic import make_activations, make_weight
    M, K, N = 128, 128, 8
    W = make_weight(M, K, 0.5, seed=6)
    X = make_activations(K, N, seed=6)
    e = oracle.encode(W, M, K)
    vals, glo, bmp = e["values"], e["global"], e["bitmap"]
    a = oracle.spmm(vals, bmp, glo, X, M, N, K, 1, False)
    b = oracle.spmm_bias_act(vals, bmp, glo, X, M, N, K, 1, None, 0)
    c = oracle.spmm_bias_act(vals, bmp, glo, X, M, N, K, 1, np.zeros(M, np.float16), 0)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    assert np.array_equal(a.view(np.uint16), c.view(np.uint16))
