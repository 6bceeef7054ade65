"""`torch.ops.spmspm_amd.sparse_linear`: the compressed linear layer as a registered PyTorch operator.

Takes the place of the reference's per-layer weight record and its wrapper call
(third_party/ft_spinfer.patch:599-610 the record, :3722-3753 `cublasMMWrapper::SpMM`; the per-matrix Split_K
the converter stores next to the weights, end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:23,360).
The operator is a thin shell around the C ABI (`SpMM_SplitK_API` / `SpMM_SplitK_API_BiasAct` of
include/spmm_api.h): torch supplies device memory and the current stream, nothing else.  It has a fake (meta)
implementation, so `torch.compile(fullgraph=True)` traces through it, and it records into HIP graphs like any
other kernel launch.

    import spmspm_amd.torch_ops                      # registers the operator
    layer = spmspm_amd.torch_ops.SparseLinearModule.from_compressed(comp, bias=b, activation=spmspm_amd.ACT_RELU)
    y = layer(x)                                     # x: [N][K] fp16 on the GPU  ->  [N][M] fp16
    y = torch.ops.spmspm_amd.sparse_linear(x, layer.values, layer.bitmaps, layer.offsets, None, M, 0, 0)
"""
from typing import Optional

import numpy as np
import torch

from . import api as A

__all__ = ["sparse_linear", "SparseLinearModule"]


@torch.library.custom_op("spmspm_amd::sparse_linear", mutates_args=(), device_types="cuda")
def sparse_linear(x: torch.Tensor, values: torch.Tensor, bitmaps: torch.Tensor, offsets: torch.Tensor,
                  bias: Optional[torch.Tensor], M: int, split_k: int, activation: int,
                  nnz: int = -1) -> torch.Tensor:
    """y[N][M] = act(W x + bias) for the compressed W given by (values, bitmaps, offsets).

    x [N][K] fp16 contiguous; values int16/fp16 (compact non-zeros), bitmaps int64 (64 per group tile), offsets
    int32 (G+1); bias fp16 [M] or None; split_k <= 0 lets the library choose; activation 0 none, 1 ReLU, 2 GELU;
    nnz, when not negative, is offsets[G] as the caller knows it (the number of halves `values` must hold), checked
    here without reading device memory.  Every check happens on the host before anything is launched: the kernels
    trust their pointers."""
    if x.dim() != 2 or x.dtype != torch.float16 or not x.is_contiguous() or not x.is_cuda:
        raise ValueError("x must be a contiguous [N][K] fp16 tensor on the GPU")
    N, K = x.shape
    G = offsets.numel() - 1
    if M <= 0 or M % 64 or K % 64 or G != (M // 64) * (K // 64) or bitmaps.numel() != 64 * G:
        raise ValueError(f"compressed arrays do not describe a {M}x{K} matrix")
    if offsets.dtype != torch.int32 or bitmaps.dtype != torch.int64 or values.dtype not in (torch.int16, torch.float16):
        raise ValueError("offsets must be int32, bitmaps int64 and values int16 or fp16 "
                         f"(got {offsets.dtype}, {bitmaps.dtype}, {values.dtype})")
    for name, t in (("values", values), ("bitmaps", bitmaps), ("offsets", offsets), ("bias", bias)):
        if t is None:
            continue
        if t.device != x.device:
            raise ValueError(f"{name} is on {t.device}, x on {x.device}: all operands must share x's device")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    if nnz >= 0 and values.numel() < nnz:
        raise ValueError(f"values holds {values.numel()} halves, the offsets end at {nnz}")
    fused = bias is not None or activation != A.ACT_NONE
    if bias is not None and (bias.numel() != M or bias.dtype != torch.float16):
        raise ValueError("bias must be M contiguous fp16 values")
    sk = split_k if split_k > 0 else A.SpMM_SplitK_Auto(M, N, K)  # resolved once: the workspace matches the call
    need = (A.SpMM_WorkspaceBytesBiasAct if fused else A.SpMM_WorkspaceBytes)(M, N, K, sk)
    ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
    out = torch.empty((N, M), dtype=torch.float16, device=x.device)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device)
        if fused:
            err = A.SpMM_SplitK_API_BiasAct(stream, values, bitmaps, offsets, x, out, M, N, K, ws, sk, bias,
                                            int(activation))
        else:
            err = A.SpMM_SplitK_API(stream, values, bitmaps, offsets, x, out, M, N, K, ws, sk)
    if err != A.HIP_SUCCESS:
        raise RuntimeError(f"spmspm_amd::sparse_linear: the library returned hipError_t {err} "
                           f"(M={M}, N={N}, K={K}, Split_K={sk})")
    return out


@sparse_linear.register_fake
def _(x, values, bitmaps, offsets, bias, M, split_k, activation, nnz=-1):
    return x.new_empty((x.shape[0], M))


class SparseLinearModule(torch.nn.Module):
    """`nn.Module` front end of the operator: the compressed arrays are buffers (they move with `.to()`, are saved
    with `state_dict()`), `forward` is one operator call."""

    def __init__(self, M, K, values, bitmaps, offsets, bias=None, activation=A.ACT_NONE, split_k=0):
        super().__init__()
        self.M, self.K, self.activation, self.split_k = int(M), int(K), int(activation), int(split_k)
        # offsets[G], read once here: the operator then checks `values` against it without touching device memory
        self.nnz = int(offsets[-1].item()) if offsets.numel() else 0
        if values.numel() < self.nnz:
            raise ValueError(f"values holds {values.numel()} halves, the offsets end at {self.nnz}")
        self.register_buffer("values", values)
        self.register_buffer("bitmaps", bitmaps)
        self.register_buffer("offsets", offsets)
        self.register_buffer("bias", bias)

    @classmethod
    def from_compressed(cls, compressed, device="cuda:0", bias=None, activation=A.ACT_NONE, split_k=0):
        """From the host encoder's output (`spmspm_amd.InitSparseMatrixA_bitmap`)."""
        vals = compressed.values if compressed.values.size else np.zeros(8, np.uint16)
        t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
        b = None
        if bias is not None:
            b = (torch.from_numpy(np.ascontiguousarray(bias, np.float16).view(np.int16)).view(torch.float16)
                 if isinstance(bias, np.ndarray) else bias).to(device).contiguous()
        return cls(compressed.M, compressed.K, t(vals.view(np.int16)), t(compressed.bitmaps.view(np.int64)),
                   t(compressed.offsets), b, activation, split_k)

    @classmethod
    def from_layer(cls, layer):
        """From a resident `spmspm_amd.SparseLinear` (shares its device arrays)."""
        b = None if layer.bias is None else layer.bias.view(torch.float16)
        return cls(layer.M, layer.K, layer.values, layer.bitmaps, layer.offsets, b, layer.activation, layer.split_k)

    def forward(self, x):
        return torch.ops.spmspm_amd.sparse_linear(x, self.values, self.bitmaps, self.offsets, self.bias, self.M,
                                                  self.split_k, self.activation, self.nnz)

    def extra_repr(self):
        return f"M={self.M}, K={self.K}, split_k={self.split_k}, activation={self.activation}"
