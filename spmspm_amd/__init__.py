"""MI355X (gfx950) bitmap-compressed SpMM: host layer over libSpMM_API.so.

The functions mirror the reference's public interface for this path
(csrc/SpMM_API.cuh): `InitSparseMatrixA_bitmap` (host encoder) and
`SpMM_SplitK_API` / `SpMM_SplitK_API_bitmap_v3` (device SpMM).
"""
from .api import (  # noqa: F401
    CompressedMatrix,
    InitSparseMatrixA_bitmap,
    InitSparseMatrixA_bitmap_device,
    InitSparseMatrixA_bitmap_device_onepass,
    Our_GenSparseMatrixBinFile,
    SparseLinear,
    ACT_GELU,
    ACT_NONE,
    ACT_RELU,
    NOALLOC_SCRATCH_BYTES,
    SpMM_SplitK_API,
    SpMM_SplitK_API_NoAlloc,
    SpMM_SplitK_API_Sized,
    SpMM_SplitK_API_BiasAct,
    SpMM_WorkspaceBytesBiasAct,
    SpMM_SplitK_API_bitmap_v3,
    SpMM_ReadWeightFiles,
    SpMM_SplitK_Auto,
    SpMM_SplitK_AutoNoAlloc,
    SpMM_SplitK_CostModel,
    SpMM_SplitK_TableSetMany,
    SpMM_SplitK_TableClear,
    SpMM_SplitK_TableLoad,
    SpMM_SplitK_TableSave,
    SpMM_SplitK_TableSet,
    SpMM_WorkspaceBytes,
    library,
    library_path,
    load_weight_files,
)
