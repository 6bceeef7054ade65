"""SpMM_SplitK_API_NoAlloc (partial sums in the library's own device array) against SpMM_SplitK_API, bit for bit."""
import numpy as np
import pytest

import spmspm_amd as S
from spmspm_amd.synthetic import make_activations, make_weight

pytestmark = pytest.mark.gpu


def _upload(torch, comp):
    dev = "cuda:0"
    vals = comp.values if comp.values.size else np.zeros(8, np.uint16)
    return (torch.from_numpy(vals.view(np.int16).copy()).to(dev),
            torch.from_numpy(comp.bitmaps.view(np.int64).copy()).to(dev),
            torch.from_numpy(comp.offsets.copy()).to(dev))


def _both(torch, M, K, N, sparsity, split_k, seed):
    """(output of the workspace entry point, output of the no-allocation one) for one seeded problem."""
    W = make_weight(M, K, sparsity, seed=seed)
    X = make_activations(K, N, seed=seed)
    comp = S.InitSparseMatrixA_bitmap(W)
    values, bitmaps, offsets = _upload(torch, comp)
    x = torch.from_numpy(X.view(np.int16).copy()).to("cuda:0")
    nbytes = S.SpMM_WorkspaceBytes(M, N, K, split_k)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda:0")
    ref = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")
    out = torch.full((N, M), 0x7e00, dtype=torch.int16, device="cuda:0")
    assert S.SpMM_SplitK_API(None, values, bitmaps, offsets, x, ref, M, N, K, ws, split_k) == 0
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    assert S.SpMM_SplitK_API_NoAlloc(None, values, bitmaps, offsets, x, out, M, N, K, split_k) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    # torch's counter only sees torch's own allocator; the device's free memory (hipMemGetInfo) sees a hipMalloc
    # made by anyone.  Measured around a second call: by then the kernels are loaded and the array's address is
    # cached, so a call that allocates nothing leaves the figure as it was.
    free_before = torch.cuda.mem_get_info()[0]
    assert S.SpMM_SplitK_API_NoAlloc(None, values, bitmaps, offsets, x, out, M, N, K, split_k) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    return ref.cpu().numpy(), out.cpu().numpy()


def test_no_alloc_entry_matches_the_workspace_entry_on_two_calls_in_a_row(capfd):
    import torch
    assert torch.cuda.is_available()
    # first call: split K over 5 batches; second call: a smaller problem, which leaves most of the first call's
    # partial sums in the shared array
    ref, out = _both(torch, 1024, 2048, 32, 0.6, 5, seed=11)
    assert np.array_equal(ref, out)
    ref, out = _both(torch, 256, 512, 16, 0.7, 3, seed=12)
    assert np.array_equal(ref, out)
    # the library's own choice of Split_K, and an unsplit K (no partial sums at all)
    ref, out = _both(torch, 2048, 2048, 16, 0.5, 0, seed=13)
    assert np.array_equal(ref, out)
    ref, out = _both(torch, 128, 256, 64, 0.5, 1, seed=14)
    assert np.array_equal(ref, out)
    capfd.readouterr()
    # partial sums beyond the array: refused before anything is launched
    M, N, K, sk = 16384, 128, 4096, 8
    assert 4 * M * N * sk > S.NOALLOC_SCRATCH_BYTES
    assert S.SpMM_SplitK_API_NoAlloc(None, 0, 0, 0, 0, 0, M, N, K, sk) == 1
    assert "holds at most" in capfd.readouterr().out


def test_no_alloc_entry_records_into_a_graph_after_a_warm_up_call():
    """The stated use: a call under HIP graph capture (which forbids allocation).  A warm-up call outside the
    capture looks up the array's address; the captured call with a split K is replayed three times with eager work
    in between and every replay must give the workspace entry point's bits."""
    import torch
    M, K, N, sk = 1024, 2048, 16, 4
    W = make_weight(M, K, 0.6, seed=21)
    comp = S.InitSparseMatrixA_bitmap(W)
    values, bitmaps, offsets = _upload(torch, comp)
    xs = [torch.from_numpy(make_activations(K, N, seed=30 + i).view(np.int16).copy()).to("cuda:0") for i in range(3)]
    ws = torch.empty(S.SpMM_WorkspaceBytes(M, N, K, sk), dtype=torch.uint8, device="cuda:0")
    x = xs[0].clone()
    out = torch.zeros((N, M), dtype=torch.int16, device="cuda:0")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert S.SpMM_SplitK_API_NoAlloc(side, values, bitmaps, offsets, x, out, M, N, K, sk) == 0  # warm-up
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        assert S.SpMM_SplitK_API_NoAlloc(None, values, bitmaps, offsets, x, out, M, N, K, sk) == 0
    for i in range(3):
        x.copy_(xs[i])
        ref = torch.zeros((N, M), dtype=torch.int16, device="cuda:0")
        assert S.SpMM_SplitK_API(None, values, bitmaps, offsets, xs[i], ref, M, N, K, ws, sk) == 0  # eager work
        torch.cuda.synchronize()
        out.fill_(0x7e00)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref), f"replay {i}"
