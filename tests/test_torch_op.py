"""`torch.ops.spmspm_amd.sparse_linear`: registration and fake implementation (CPU), results against the oracle, graph
capture and torch.compile (GPU)."""
import numpy as np
import pytest

import spmspm_amd as S
from conftest import assert_spmm_close
from spmspm_amd.synthetic import make_activations, make_weight


@pytest.fixture(scope="module")
def ops():
    import torch
    import spmspm_amd.torch_ops as T
    return torch, T


def test_operator_is_registered_with_a_schema_and_a_fake_implementation(ops):
    torch, T = ops
    op = torch.ops.spmspm_amd.sparse_linear
    schema = str(op.default._schema)
    assert "Tensor x" in schema and "Tensor? bias" in schema and "split_k" in schema and "-> Tensor" in schema
    # on meta tensors only the fake implementation can run: shapes and dtype without any device work
    M, K, N = 256, 512, 16
    G = (M // 64) * (K // 64)
    x = torch.empty((N, K), dtype=torch.float16, device="meta")
    y = op(x, torch.empty(100, dtype=torch.int16, device="meta"), torch.empty(64 * G, dtype=torch.int64, device="meta"),
           torch.empty(G + 1, dtype=torch.int32, device="meta"), None, M, 0, 0)
    assert y.shape == (N, M) and y.dtype == torch.float16 and y.device.type == "meta"


def _problem(M, K, N, s, seed):
    W = make_weight(M, K, s, seed=seed)
    X = make_activations(K, N, seed=seed)
    return W, X, S.InitSparseMatrixA_bitmap(W)


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N,s,sk", [(256, 512, 16, 0.6, 0), (512, 2048, 8, 0.7, 4), (128, 256, 64, 0.5, 1),
                                        (256, 1024, 128, 0.5, 3)])
def test_operator_matches_the_oracle(ops, oracle, M, K, N, s, sk):
    torch, T = ops
    W, X, comp = _problem(M, K, N, s, seed=M + N)
    layer = T.SparseLinearModule.from_compressed(comp, split_k=sk)
    x = torch.from_numpy(X.view(np.int16).copy()).cuda().view(torch.float16)
    y = layer(x)
    y2 = torch.ops.spmspm_amd.sparse_linear(x, layer.values, layer.bitmaps, layer.offsets, None, M, sk, 0)
    torch.cuda.synchronize()
    sk_eff = sk if sk > 0 else S.SpMM_SplitK_Auto(M, N, K)
    want = oracle.spmm(comp.values, comp.bitmaps, comp.offsets, X, M, N, K, sk_eff, False)
    assert_spmm_close(y.cpu().numpy(), want, "module")
    assert torch.equal(y, y2)
    # bias and activation go through the fused entry point
    bias = np.linspace(-1, 1, M).astype(np.float16)
    fused = T.SparseLinearModule.from_compressed(comp, bias=bias, activation=S.ACT_GELU, split_k=sk)
    yf = fused(x)
    torch.cuda.synchronize()
    want_f = oracle.spmm_bias_act(comp.values, comp.bitmaps, comp.offsets, X, M, N, K, sk_eff, bias, S.ACT_GELU)
    assert_spmm_close(yf.cpu().numpy(), want_f, "fused module")
    # the resident layer of the ctypes front end gives the very same operator
    res = S.SparseLinear(comp, split_k=sk)
    assert torch.equal(res.module()(x), res(x))


@pytest.mark.gpu
def test_operator_passes_opcheck(ops):
    torch, T = ops
    W, X, comp = _problem(128, 256, 16, 0.5, seed=1)
    layer = T.SparseLinearModule.from_compressed(comp)
    x = torch.from_numpy(X.view(np.int16).copy()).cuda().view(torch.float16)
    torch.library.opcheck(torch.ops.spmspm_amd.sparse_linear,
                          (x, layer.values, layer.bitmaps, layer.offsets, None, 128, 0, 0),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.gpu
def test_bad_arguments_raise(ops):
    torch, T = ops
    W, X, comp = _problem(128, 256, 16, 0.5, seed=2)
    layer = T.SparseLinearModule.from_compressed(comp)
    x = torch.from_numpy(X.view(np.int16).copy()).cuda().view(torch.float16)
    with pytest.raises(ValueError):
        layer(x.float())
    with pytest.raises(ValueError):
        torch.ops.spmspm_amd.sparse_linear(x, layer.values, layer.bitmaps, layer.offsets, None, 192, 0, 0)
    with pytest.raises(RuntimeError):  # 24 columns: the library's unsupported-N error comes back as an exception
        layer(torch.zeros((24, 256), dtype=torch.float16, device="cuda"))
    # operand types, devices and sizes are refused on the host, before any launch
    op = torch.ops.spmspm_amd.sparse_linear
    v, b, o = layer.values, layer.bitmaps, layer.offsets
    with pytest.raises(ValueError, match="int32"):
        op(x, v, b, o.long(), None, 128, 0, 0)
    with pytest.raises(ValueError, match="int64"):
        op(x, v, b.int(), o, None, 128, 0, 0)
    with pytest.raises(ValueError, match="int16 or fp16"):
        op(x, v.float(), b, o, None, 128, 0, 0)
    with pytest.raises(ValueError, match="share x's device"):
        op(x, v.cpu(), b, o, None, 128, 0, 0)
    with pytest.raises(ValueError, match="share x's device"):
        op(x, v, b.cpu(), o, None, 128, 0, 0)
    with pytest.raises(ValueError, match="share x's device"):
        op(x, v, b, o, torch.zeros(128, dtype=torch.float16), 128, 0, 0)
    with pytest.raises(ValueError, match="contiguous"):
        op(x, torch.stack([v, v], 1)[:, 0], b, o, None, 128, 0, 0)
    with pytest.raises(ValueError, match="offsets end at"):
        op(x, v[:-8], b, o, None, 128, 0, 0, layer.nnz)
    with pytest.raises(ValueError, match="offsets end at"):
        T.SparseLinearModule(128, 256, v[:-8], b, o)
    y = op(x, v.view(torch.float16), b, o, None, 128, 0, 0, layer.nnz)  # fp16-typed values are the same bytes
    assert torch.equal(y, layer(x))


def _chain(T, comps, biases):
    import torch
    return torch.nn.Sequential(*[T.SparseLinearModule.from_compressed(c, bias=b, activation=S.ACT_RELU if b is not None
                                                                      else S.ACT_NONE)
                                 for c, b in zip(comps, biases)])


@pytest.mark.gpu
def test_two_layer_chain_under_torch_compile_and_in_a_graph(ops, oracle):
    """A two-layer chain (512 -> 1024 with bias + ReLU -> 256) through torch.compile(fullgraph=True) — the operator
    must trace without a graph break — and captured in a HIP graph that is replayed with eager work in between;
    every result against the oracle's chain."""
    torch, T = ops
    N = 16
    W1 = make_weight(1024, 512, 0.6, seed=61)
    W2 = make_weight(256, 1024, 0.6, seed=62)
    c1, c2 = S.InitSparseMatrixA_bitmap(W1), S.InitSparseMatrixA_bitmap(W2)
    b1 = np.linspace(-0.5, 0.5, 1024).astype(np.float16)
    net = _chain(T, [c1, c2], [b1, None])

    def expected(X):
        h = oracle.spmm_bias_act(c1.values, c1.bitmaps, c1.offsets, X, 1024, N, 512, S.SpMM_SplitK_Auto(1024, N, 512),
                                 b1, S.ACT_RELU)
        return oracle.spmm(c2.values, c2.bitmaps, c2.offsets, h, 256, N, 1024, S.SpMM_SplitK_Auto(256, N, 1024), False)

    X = (make_activations(512, N, seed=7).astype(np.float32) * 4).astype(np.float16)
    x = torch.from_numpy(X.view(np.int16).copy()).cuda().view(torch.float16)
    eager = net(x)
    torch.cuda.synchronize()
    assert_spmm_close(eager.cpu().numpy(), expected(X), "eager chain")

    try:
        compiled = torch.compile(net, fullgraph=True)
        got = compiled(x)
    except Exception as e:  # no code generator for the glue in this image: the tracing half still has to hold
        if "triton" not in str(e).lower() and "inductor" not in str(e).lower():
            raise
        compiled = torch.compile(net, fullgraph=True, backend="aot_eager")
        got = compiled(x)
    torch.cuda.synchronize()
    assert torch.equal(got, eager), "compiled chain differs from the eager chain"

    # graph capture: static input buffer, replays with eager work and synchronisations in between
    xs = x.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        net(xs)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            ys = net(xs)
        for rep in range(3):
            Xr = (make_activations(512, N, seed=70 + rep).astype(np.float32) * 4).astype(np.float16)
            xs.copy_(torch.from_numpy(Xr.view(np.int16).copy()).cuda().view(torch.float16))
            g.replay()
            side.synchronize()
            assert_spmm_close(ys.cpu().numpy(), expected(Xr), f"graph replay {rep}")
            again = net(xs)
            side.synchronize()
            assert torch.equal(again, ys), "eager != replay"
