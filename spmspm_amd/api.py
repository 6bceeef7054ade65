"""ctypes binding of libSpMM_API.so plus thin torch plumbing (device memory, streams).

Names, argument meaning and error behaviour follow the reference's interface
for this path (csrc/SpMM_API.cuh:47-53 and :112-120; call sites
kernel_benchmark/spmm_test.cu:316-388).  There is no CPU fallback: if the
library is missing or no GPU is present the SpMM calls raise.
"""
import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBPATH = os.path.join(_HERE, "lib", "libSpMM_API.so")
_lib = None

_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int)
_u64p = C.POINTER(C.c_uint64)

HIP_SUCCESS = 0
HIP_ERROR_INVALID_VALUE = 1
HIP_ERROR_UNKNOWN = 999


def library_path():
    return _LIBPATH


def library():
    """Load libSpMM_API.so (built in-tree by spmspm_amd/build.py).  Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIBPATH):
        raise RuntimeError(
            f"{_LIBPATH} is missing: build it with `python -m spmspm_amd.build` "
            "(or __graft_entry__.build()); there is no fallback path")
    L = C.CDLL(_LIBPATH)
    L.SpMM_SplitK_API.restype = C.c_int
    L.SpMM_SplitK_API.argtypes = [C.c_void_p] * 6 + [C.c_int] * 3 + [C.c_void_p, C.c_int]
    L.SpMM_SplitK_API_Sized.restype = C.c_int
    L.SpMM_SplitK_API_Sized.argtypes = [C.c_void_p] * 6 + [C.c_int] * 3 + [C.c_void_p, C.c_size_t, C.c_int]
    L.SpMM_SplitK_API_bitmap_v3.restype = C.c_int
    L.SpMM_SplitK_API_bitmap_v3.argtypes = [C.c_void_p] * 9 + [C.c_int] * 3 + [C.c_void_p, C.c_int]
    L.SpMM_SplitK_Auto.restype = C.c_int
    L.SpMM_SplitK_Auto.argtypes = [C.c_int] * 3
    L.SpMM_SplitK_TableSet.restype = C.c_int
    L.SpMM_SplitK_TableSet.argtypes = [C.c_int] * 4
    L.SpMM_SplitK_CostModel.restype = C.c_int
    L.SpMM_SplitK_CostModel.argtypes = [C.c_int] * 3
    L.SpMM_SplitK_AutoNoAlloc.restype = C.c_int
    L.SpMM_SplitK_AutoNoAlloc.argtypes = [C.c_int] * 3
    L.SpMM_SplitK_TableSetMany.restype = C.c_int
    L.SpMM_SplitK_TableSetMany.argtypes = [_i32p, C.c_int]
    L.SpMM_ReadWeightFiles.restype = C.c_int
    L.SpMM_ReadWeightFiles.argtypes = [C.c_char_p] * 6 + [C.c_int, C.c_int, C.POINTER(_u16p), C.POINTER(_i32p),
                                                         C.POINTER(_i32p), C.POINTER(_u64p), _i32p, _i32p]
    L.SpMM_LoadWeightFiles.restype = C.c_int
    L.SpMM_LoadWeightFiles.argtypes = [C.c_char_p] * 6 + [C.c_int, C.c_int] + [C.POINTER(C.c_void_p)] * 5 + [_i32p]
    L.SpMM_FreeWeights.restype = None
    L.SpMM_FreeWeights.argtypes = [C.c_void_p] * 5
    L.SpMM_SplitK_TableLoad.restype = C.c_int
    L.SpMM_SplitK_TableLoad.argtypes = [C.c_char_p]
    L.SpMM_SplitK_TableSave.restype = C.c_int
    L.SpMM_SplitK_TableSave.argtypes = [C.c_char_p]
    L.SpMM_SplitK_TableClear.restype = None
    L.SpMM_SplitK_TableClear.argtypes = []
    L.SpMM_SplitK_API_NoAlloc.restype = C.c_int
    L.SpMM_SplitK_API_NoAlloc.argtypes = [C.c_void_p] * 6 + [C.c_int] * 4
    L.SpMM_WorkspaceBytes.restype = C.c_size_t
    L.SpMM_WorkspaceBytes.argtypes = [C.c_int] * 4
    L.SpMM_SplitK_API_BiasAct.restype = C.c_int
    L.SpMM_SplitK_API_BiasAct.argtypes = [C.c_void_p] * 6 + [C.c_int] * 3 + [C.c_void_p, C.c_int, C.c_void_p, C.c_int]
    L.SpMM_WorkspaceBytesBiasAct.restype = C.c_size_t
    L.SpMM_WorkspaceBytesBiasAct.argtypes = [C.c_int] * 4
    L.SpMM_EncodeDevice_Bitmaps.restype = C.c_int
    L.SpMM_EncodeDevice_Bitmaps.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    L.SpMM_EncodeDevice_Values.restype = C.c_int
    L.SpMM_EncodeDevice_Values.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    L.SpMM_EncodeDevice_ScratchBytes.restype = C.c_size_t
    L.SpMM_EncodeDevice_ScratchBytes.argtypes = [C.c_int, C.c_int]
    L.SpMM_EncodeDevice_OnePass.restype = C.c_int
    L.SpMM_EncodeDevice_OnePass.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.c_size_t, C.c_void_p]
    L.InitSparseMatrixA_bitmap.restype = C.c_int
    L.InitSparseMatrixA_bitmap.argtypes = [C.c_void_p] + [C.c_int] * 8 + [
        C.POINTER(_u16p), C.POINTER(_i32p), C.POINTER(_i32p), C.POINTER(_i32p), C.POINTER(_u64p), _i32p]
    L.Our_GenSparseMatrixBinFile.restype = None
    L.Our_GenSparseMatrixBinFile.argtypes = [C.c_char_p, C.c_int, C.c_int] + [C.c_char_p] * 6
    L.SpMM_Version.restype = C.c_char_p
    L.SpMM_KernelName.restype = C.c_char_p
    L.SpMM_KernelName.argtypes = [C.c_int] * 4
    L.SpMM_ShaderClockProbe.restype = C.c_int
    L.SpMM_ShaderClockProbe.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
    L.SpMM_TimeNextCall.restype = None
    L.SpMM_TimeNextCall.argtypes = [C.c_void_p, C.c_void_p]
    _lib = L
    return L


_libc = C.CDLL(None)
_libc.free.argtypes = [C.c_void_p]


@dataclass
class CompressedMatrix:
    """Host-side TCA-BME arrays of one weight matrix, as the encoder returns them."""
    M: int
    K: int
    num_gtiles: int
    values: np.ndarray      # uint16 view of fp16, len == offsets[-1]
    tile_counts: np.ndarray  # int32, per 8x8 tile (the reference's `TileOffsets`)
    median: np.ndarray      # int32, 4 per group tile
    offsets: np.ndarray     # int32, num_gtiles + 1 (the reference's `TileOffsets_global`)
    bitmaps: np.ndarray     # uint64, 64 per group tile
    max_nnz: int            # largest padded per-group-tile count, not yet rounded

    @property
    def max_nnz_rounded(self):
        """Rounded up to a multiple of 64 as the reference's callers do (kernel_benchmark/spmm_test.cu:325-327)."""
        v = self.max_nnz
        return v if v % 64 == 0 else (v // 64 + 1) * 64

    def algorithmic_bytes(self, N):
        """Bytes one SpMM call must move: values + bitmaps + offsets + X + C."""
        return (2 * int(self.offsets[-1]) + 8 * self.bitmaps.size + 4 * self.offsets.size
                + 2 * self.K * N + 2 * self.M * N)


def InitSparseMatrixA_bitmap(A_h, M=None, K=None, tile_M=8, tile_M_median=16, tile_M_global=64,
                             tile_K=8, tile_K_median=64, tile_K_global=64):
    """Encode a dense row-major fp16 matrix (csrc/SpMM_API.cuh:112-241).

    `A_h`: numpy float16 (or uint16 bit patterns) of shape [M][K].  Returns a
    CompressedMatrix; raises MemoryError on the reference's -1, ValueError on
    tile sizes other than the reference's.
    """
    A = np.ascontiguousarray(A_h)
    if A.dtype == np.float16:
        A = A.view(np.uint16)
    if A.dtype != np.uint16:
        raise TypeError("A_h must be float16 (or its uint16 bit patterns)")
    if M is None or K is None:
        if A.ndim != 2:
            raise ValueError("give M and K for a flat array")
        M, K = A.shape
    if A.size != M * K:
        raise ValueError("A_h does not hold M*K elements")
    L = library()
    vals, cnt, med, glo, bmp = _u16p(), _i32p(), _i32p(), _i32p(), _u64p()
    mx = C.c_int(0)
    G = L.InitSparseMatrixA_bitmap(A.ctypes.data, M, K, tile_M, tile_M_median, tile_M_global, tile_K,
                                   tile_K_median, tile_K_global, C.byref(vals), C.byref(cnt), C.byref(med),
                                   C.byref(glo), C.byref(bmp), C.byref(mx))
    if G == -1:
        raise MemoryError("InitSparseMatrixA_bitmap: allocation failed")
    if G < 0:
        raise ValueError("InitSparseMatrixA_bitmap: only the reference tiling 8,16,64,8,64,64 is supported")
    T = (M // 8) * (K // 8)
    offsets = np.ctypeslib.as_array(glo, shape=(G + 1,)).copy()
    nnz = int(offsets[G])
    out = CompressedMatrix(
        M=M, K=K, num_gtiles=G,
        values=np.ctypeslib.as_array(vals, shape=(max(nnz, 1),))[:nnz].copy(),
        tile_counts=np.ctypeslib.as_array(cnt, shape=(max(T, 1),))[:T].copy(),
        median=np.ctypeslib.as_array(med, shape=(max(4 * G, 1),))[:4 * G].copy(),
        offsets=offsets,
        bitmaps=np.ctypeslib.as_array(bmp, shape=(max(T, 1),))[:T].copy(),
        max_nnz=mx.value)
    for p in (vals, cnt, med, glo, bmp):
        _libc.free(C.cast(p, C.c_void_p))
    return out


def Our_GenSparseMatrixBinFile(dense_path, M, K, values_path, global_path, median_path, bitmap_path,
                               max_nnz_path, sizes_path):
    """File-to-file encoder (csrc/SpMM_API.cuh:243-320).  Exits the process on I/O failure, like the reference."""
    enc = [os.fsencode(p) for p in (dense_path, values_path, global_path, median_path, bitmap_path,
                                    max_nnz_path, sizes_path)]
    library().Our_GenSparseMatrixBinFile(enc[0], M, K, *enc[1:])


def SpMM_ReadWeightFiles(values_path, global_path, median_path, bitmap_path, max_nnz_path, sizes_path, M, K):
    """The library's own reader of the six files (include/spmm_api.h) -> CompressedMatrix (per-tile counts from the
    bitmaps).  Raises OSError / ValueError on the library's -1 / -2."""
    enc = [os.fsencode(p) for p in (values_path, global_path, median_path, bitmap_path, max_nnz_path, sizes_path)]
    vals, glo, med, bmp = _u16p(), _i32p(), _i32p(), _u64p()
    mx, cnt = C.c_int(0), C.c_int(0)
    G = library().SpMM_ReadWeightFiles(*enc, M, K, C.byref(vals), C.byref(glo), C.byref(med), C.byref(bmp),
                                       C.byref(mx), C.byref(cnt))
    if G == -1:
        raise OSError("SpMM_ReadWeightFiles: a file is missing or has another length than the sizes file states")
    if G < 0:
        raise ValueError(f"SpMM_ReadWeightFiles: the files do not match M, K or each other ({G})")
    n = cnt.value
    bitmaps = np.ctypeslib.as_array(bmp, shape=(max(64 * G, 1),))[:64 * G].copy()
    out = CompressedMatrix(
        M=M, K=K, num_gtiles=G,
        values=np.ctypeslib.as_array(vals, shape=(max(n, 1),))[:n].copy(),
        tile_counts=_popcount64(bitmaps),
        median=np.ctypeslib.as_array(med, shape=(max(4 * G, 1),))[:4 * G].copy(),
        offsets=np.ctypeslib.as_array(glo, shape=(G + 1,)).copy(),
        bitmaps=bitmaps, max_nnz=mx.value)
    for p in (vals, glo, med, bmp):
        _libc.free(C.cast(p, C.c_void_p))
    return out


def load_weight_files(values_path, global_path, median_path, bitmap_path, max_nnz_path, sizes_path, M, K):
    """Read the six files back (layout of csrc/SpMM_API.cuh:304-319) into a CompressedMatrix."""
    sizes = np.fromfile(sizes_path, dtype=np.int32)
    if sizes.size != 4:
        raise ValueError("sizes file must hold 4 ints")
    val_count, g1, m4, l64 = (int(v) for v in sizes)
    G = g1 - 1
    if G != (M // 64) * (K // 64) or m4 != 4 * G or l64 != 64 * G:
        raise ValueError("sizes file does not match M, K")
    values = np.fromfile(values_path, dtype=np.uint16)
    offsets = np.fromfile(global_path, dtype=np.int32)
    median = np.fromfile(median_path, dtype=np.int32)
    bitmaps = np.fromfile(bitmap_path, dtype=np.uint64)
    max_nnz = int(np.fromfile(max_nnz_path, dtype=np.int32)[0])
    if values.size != val_count or offsets.size != g1 or median.size != m4 or bitmaps.size != l64:
        raise ValueError("file lengths do not match the sizes file")
    counts = np.array([bin(int(b)).count("1") for b in bitmaps], dtype=np.int32) if l64 <= 1 << 16 else \
        _popcount64(bitmaps)
    return CompressedMatrix(M=M, K=K, num_gtiles=G, values=values, tile_counts=counts, median=median,
                            offsets=offsets, bitmaps=bitmaps, max_nnz=max_nnz)


def _popcount64(a):
    a = a.copy()
    a = a - ((a >> np.uint64(1)) & np.uint64(0x5555555555555555))
    a = (a & np.uint64(0x3333333333333333)) + ((a >> np.uint64(2)) & np.uint64(0x3333333333333333))
    a = (a + (a >> np.uint64(4))) & np.uint64(0x0F0F0F0F0F0F0F0F)
    return ((a * np.uint64(0x0101010101010101)) >> np.uint64(56)).astype(np.int32)


def SpMM_SplitK_Auto(M, N, K):
    return library().SpMM_SplitK_Auto(M, N, K)


def SpMM_SplitK_TableSet(M, N, K, Split_K):
    """Record a measured Split_K for a shape; calls with Split_K <= 0 use it instead of the cost model."""
    rc = library().SpMM_SplitK_TableSet(M, N, K, Split_K)
    if rc != 0:
        raise ValueError(f"SpMM_SplitK_TableSet({M}, {N}, {K}, {Split_K}) -> {rc}")


def SpMM_SplitK_TableSetMany(entries):
    """Record several measured choices at once: an iterable of (M, N, K, Split_K)."""
    flat = np.ascontiguousarray(np.asarray(list(entries), dtype=np.int32).reshape(-1, 4))
    rc = library().SpMM_SplitK_TableSetMany(flat.ctypes.data_as(_i32p), flat.shape[0])
    if rc != 0:
        raise ValueError(f"SpMM_SplitK_TableSetMany refused its entries ({rc})")


def SpMM_SplitK_CostModel(M, N, K):
    """The built-in cost model's Split_K for a shape, whatever the table holds."""
    return library().SpMM_SplitK_CostModel(M, N, K)


def SpMM_SplitK_AutoNoAlloc(M, N, K):
    """The split SpMM_SplitK_API_NoAlloc uses for Split_K <= 0: the library's choice, held to what its array fits."""
    return library().SpMM_SplitK_AutoNoAlloc(M, N, K)


def SpMM_SplitK_TableLoad(path):
    """Add the "M N K Split_K" lines of a text file to the table; returns how many were read."""
    n = library().SpMM_SplitK_TableLoad(os.fsencode(path))
    if n < 0:
        raise OSError(f"{path}: " + ("cannot be opened" if n == -1 else "malformed line"))
    return n


def SpMM_SplitK_TableSave(path):
    n = library().SpMM_SplitK_TableSave(os.fsencode(path))
    if n < 0:
        raise OSError(f"{path}: cannot be written")
    return n


def SpMM_SplitK_TableClear():
    library().SpMM_SplitK_TableClear()


def SpMM_WorkspaceBytes(M, N, K, Split_K):
    return int(library().SpMM_WorkspaceBytes(M, N, K, Split_K))


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


def _stream_handle(stream):
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


def SpMM_SplitK_API(stream, values, bitmaps, offsets, X, C_out, M, N, K, workspace, Split_K):
    """C = W*X on the device (include/spmm_api.h).  Tensors or raw device addresses.  Returns the hipError_t."""
    return library().SpMM_SplitK_API(_stream_handle(stream), _ptr(values), _ptr(bitmaps), _ptr(offsets), _ptr(X),
                                     _ptr(C_out), M, N, K, _ptr(workspace), Split_K)


def SpMM_SplitK_API_Sized(stream, values, bitmaps, offsets, X, C_out, M, N, K, workspace, workspace_bytes, Split_K):
    """SpMM_SplitK_API that refuses (returns 1) a workspace smaller than the split it resolves to needs."""
    return library().SpMM_SplitK_API_Sized(_stream_handle(stream), _ptr(values), _ptr(bitmaps), _ptr(offsets),
                                           _ptr(X), _ptr(C_out), M, N, K, _ptr(workspace), int(workspace_bytes),
                                           Split_K)


NOALLOC_SCRATCH_BYTES = 32 << 20  # SPMM_NOALLOC_SCRATCH_BYTES of include/spmm_api.h


def SpMM_SplitK_API_NoAlloc(stream, values, bitmaps, offsets, X, C_out, M, N, K, Split_K):
    """SpMM_SplitK_API whose split-K partial sums live in the library's own device array: no workspace argument,
    no allocation (include/spmm_api.h).  Returns the hipError_t."""
    return library().SpMM_SplitK_API_NoAlloc(_stream_handle(stream), _ptr(values), _ptr(bitmaps), _ptr(offsets),
                                             _ptr(X), _ptr(C_out), M, N, K, Split_K)


ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2


def InitSparseMatrixA_bitmap_device(W, stream=None):
    """Device encoder: W is a contiguous [M][K] fp16 tensor in device memory.  Returns (values int16[offsets[G]],
    bitmaps int64[64*G], offsets int32[G+1]) on W's device, identical to the host encoder's arrays.  Synchronises
    once to read the number of values."""
    import torch
    if W.dtype != torch.float16 or W.dim() != 2 or not W.is_contiguous() or not W.is_cuda:
        raise ValueError("W must be a contiguous [M][K] fp16 tensor on the device")
    M, K = W.shape
    if M % 64 or K % 64:
        raise ValueError("M and K must be multiples of 64")
    G = (M // 64) * (K // 64)
    bitmaps = torch.empty(64 * G, dtype=torch.int64, device=W.device)
    offsets = torch.empty(G + 1, dtype=torch.int32, device=W.device)
    L = library()
    err = L.SpMM_EncodeDevice_Bitmaps(_stream_handle(stream), _ptr(W), M, K, _ptr(bitmaps), _ptr(offsets))
    if err != HIP_SUCCESS:
        raise RuntimeError(f"SpMM_EncodeDevice_Bitmaps failed with hipError_t {err}")
    if stream is not None:
        stream.synchronize()
    n = int(offsets[-1].item())
    values = torch.empty(max(n, 8), dtype=torch.int16, device=W.device)
    err = L.SpMM_EncodeDevice_Values(_stream_handle(stream), _ptr(W), M, K, _ptr(offsets), _ptr(values))
    if err != HIP_SUCCESS:
        raise RuntimeError(f"SpMM_EncodeDevice_Values failed with hipError_t {err}")
    return values[:n] if n else values[:0], bitmaps, offsets


def InitSparseMatrixA_bitmap_device_onepass(W, capacity=None, stream=None, values=None):
    """The device encoder in one pass over W (SpMM_EncodeDevice_OnePass): same arrays as
    InitSparseMatrixA_bitmap_device.  `values` needs room before the count is known: `capacity` halves (default M*K,
    which always suffices) are allocated, or a caller's int16 tensor `values` is used, and the result is a view of
    the first offsets[G] of them.  Synchronises once to read the count and the kernel's status word."""
    import torch
    if W.dtype != torch.float16 or W.dim() != 2 or not W.is_contiguous() or not W.is_cuda:
        raise ValueError("W must be a contiguous [M][K] fp16 tensor on the device")
    M, K = W.shape
    if M % 64 or K % 64:
        raise ValueError("M and K must be multiples of 64")
    G = (M // 64) * (K // 64)
    L = library()
    if values is None:
        values = torch.empty(max(int(capacity if capacity is not None else M * K), 8), dtype=torch.int16, device=W.device)
    elif values.dtype != torch.int16 or not values.is_contiguous() or values.device != W.device:
        raise ValueError("values must be a contiguous int16 tensor on W's device")
    bitmaps = torch.empty(64 * G, dtype=torch.int64, device=W.device)
    offsets = torch.empty(G + 1, dtype=torch.int32, device=W.device)
    scratch = torch.empty(L.SpMM_EncodeDevice_ScratchBytes(M, K) // 8 + 1, dtype=torch.int64, device=W.device)
    err = L.SpMM_EncodeDevice_OnePass(_stream_handle(stream), _ptr(W), M, K, _ptr(bitmaps), _ptr(offsets),
                                      _ptr(values), values.numel(), _ptr(scratch))
    if err != HIP_SUCCESS:
        raise RuntimeError(f"SpMM_EncodeDevice_OnePass failed with hipError_t {err}")
    if stream is not None:
        stream.synchronize()
    status = int(scratch.view(torch.int32)[1].item())
    n = int(offsets[-1].item())
    if status & 1:
        raise RuntimeError("SpMM_EncodeDevice_OnePass: a workgroup gave up waiting for its predecessors")
    if status & 2:
        raise ValueError(f"SpMM_EncodeDevice_OnePass: values holds {values.numel()} halves, the matrix needs {n}")
    return values[:n], bitmaps, offsets


def SpMM_WorkspaceBytesBiasAct(M, N, K, Split_K):
    return int(library().SpMM_WorkspaceBytesBiasAct(M, N, K, Split_K))


def SpMM_SplitK_API_BiasAct(stream, values, bitmaps, offsets, X, C_out, M, N, K, workspace, Split_K, bias, activation):
    """C = act(W*X + bias) with the tail applied in fp32 before the fp16 rounding (include/spmm_api.h)."""
    return library().SpMM_SplitK_API_BiasAct(_stream_handle(stream), _ptr(values), _ptr(bitmaps), _ptr(offsets),
                                             _ptr(X), _ptr(C_out), M, N, K, _ptr(workspace), Split_K, _ptr(bias),
                                             int(activation))


def SpMM_SplitK_API_bitmap_v3(stream, A, Compressed_A, TileOffsets, TileOffsets_Median, bitmap, max_nnz_intile, B,
                              C_out, M_Global, N_Global, K_Global, Reduction_Workspace, Split_K):
    """The reference's 14-argument call (kernel_benchmark/spmm_test.cu:375-388).  Returns the hipError_t."""
    return library().SpMM_SplitK_API_bitmap_v3(_stream_handle(stream), _ptr(A), _ptr(Compressed_A), _ptr(TileOffsets),
                                               _ptr(TileOffsets_Median), _ptr(bitmap), _ptr(max_nnz_intile), _ptr(B),
                                               _ptr(C_out), M_Global, N_Global, K_Global, _ptr(Reduction_Workspace),
                                               Split_K)


class SparseLinear:
    """One compressed weight matrix resident in HBM; `y = W x` for a batch of N activation columns.

    Takes the place of the reference's per-layer weight record plus its
    cublasMMWrapper::SpMM call (third_party/ft_spinfer.patch:599-610, :3722-3753).
    x: [N][K] fp16 on the device; returns [N][M] fp16.
    """

    def __init__(self, compressed, device="cuda:0", split_k=0, bias=None, activation=ACT_NONE):
        """bias: M fp16 values (numpy or tensor) added to every output column; activation: ACT_NONE/RELU/GELU.
        With either, calls go through SpMM_SplitK_API_BiasAct."""
        import torch
        self.M, self.K = compressed.M, compressed.K
        self.device = torch.device(device)
        self.activation = int(activation)
        if bias is None:
            self.bias = None
        elif isinstance(bias, np.ndarray):
            self.bias = torch.from_numpy(np.ascontiguousarray(bias, np.float16).view(np.int16)).to(self.device)
        else:
            self.bias = bias.to(self.device).contiguous()
        if self.bias is not None and self.bias.numel() != self.M:
            raise ValueError("bias must have M elements")
        nnz = compressed.values.size
        vals = compressed.values if nnz else np.zeros(8, np.uint16)
        self.values = torch.from_numpy(vals.view(np.int16)).to(self.device)
        self.bitmaps = torch.from_numpy(compressed.bitmaps.view(np.int64)).to(self.device)
        self.offsets = torch.from_numpy(compressed.offsets).to(self.device)
        self.nnz_padded = int(compressed.offsets[-1])
        self.split_k = split_k
        self._ws = None
        self._plans = {}

    def clone(self):
        """A second resident copy of the same weights (device-to-device), e.g. one per decoder layer."""
        c = object.__new__(SparseLinear)
        c.M, c.K, c.device, c.nnz_padded, c.split_k, c._ws = self.M, self.K, self.device, self.nnz_padded, self.split_k, None
        c._plans = {}
        c.activation, c.bias = self.activation, (None if self.bias is None else self.bias.clone())
        c.values, c.bitmaps, c.offsets = self.values.clone(), self.bitmaps.clone(), self.offsets.clone()
        return c

    def module(self):
        """The same resident weights as a `torch.nn.Module` whose forward is the registered operator
        `torch.ops.spmspm_amd.sparse_linear` (spmspm_amd/torch_ops.py): traceable by torch.compile, usable in
        nn.Sequential, capturable in graphs.  Shares this layer's device arrays."""
        from .torch_ops import SparseLinearModule
        return SparseLinearModule.from_layer(self)

    def bytes_per_call(self, N):
        return (2 * self.nnz_padded + 8 * self.bitmaps.numel() + 4 * self.offsets.numel()
                + 2 * self.K * N + 2 * self.M * N)

    def _plan(self, N):
        """(Split_K to pass, workspace bytes) for N columns.  An automatic Split_K is resolved here, once, and passed
        on as an explicit value: the workspace is then sized for exactly the split the call will use, whatever
        happens to the library's table afterwards, and the library is asked once per N instead of on every call."""
        plan = self._plans.get(N)
        if plan is None or plan[2] != self.split_k:
            fused = self.bias is not None or self.activation != ACT_NONE
            sk = self.split_k if self.split_k > 0 else SpMM_SplitK_Auto(self.M, N, self.K)
            need = (SpMM_WorkspaceBytesBiasAct if fused else SpMM_WorkspaceBytes)(self.M, N, self.K, sk)
            plan = self._plans[N] = (sk, need, self.split_k)
        return plan

    def replan(self):
        """Forget resolved splits (after the library's Split_K table has changed)."""
        self._plans = {}

    def workspace(self, N):
        import torch
        need = self._plan(N)[1]
        if need == 0:
            return None
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        return self._ws

    def __call__(self, x, out=None, stream=None):
        import torch
        N = x.shape[0]
        if x.dtype != torch.float16 or x.shape[1] != self.K or not x.is_contiguous():
            raise ValueError("x must be a contiguous [N][K] fp16 tensor")
        if out is None:
            out = torch.empty((N, self.M), dtype=torch.float16, device=self.device)
        sk = self._plan(N)[0]
        if self.bias is not None or self.activation != ACT_NONE:
            err = SpMM_SplitK_API_BiasAct(stream, self.values, self.bitmaps, self.offsets, x, out, self.M, N, self.K,
                                          self.workspace(N), sk, self.bias, self.activation)
        else:
            err = SpMM_SplitK_API(stream, self.values, self.bitmaps, self.offsets, x, out, self.M, N, self.K,
                                  self.workspace(N), sk)
        if err != HIP_SUCCESS:
            raise RuntimeError(f"SpMM call failed with hipError_t {err}")
        return out
