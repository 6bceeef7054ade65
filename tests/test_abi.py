"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares."""
import os
import re

import spmspm_amd as S

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "spmm_api.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    c_part = text.split('} /* extern "C" */')[0] if '} /* extern "C" */' in text else text
    c_part = c_part.split("#ifdef __cplusplus\n}")[0]
    return sorted(set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", c_part)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for n in ("SpMM_SplitK_API", "SpMM_SplitK_API_bitmap_v3", "InitSparseMatrixA_bitmap",
              "Our_GenSparseMatrixBinFile", "SpMM_SplitK_Auto", "SpMM_WorkspaceBytes", "SpMM_Version", "SpMM_TimeNextCall",
              "SpMM_SplitK_API_BiasAct", "SpMM_WorkspaceBytesBiasAct", "SpMM_EncodeDevice_Bitmaps",
              "SpMM_EncodeDevice_Values"):
        assert n in names


def test_library_exports_every_declared_symbol():
    L = S.library()
    for n in _declared_functions():
        assert hasattr(L, n), f"libSpMM_API.so does not export {n}"
    assert S.library().SpMM_Version().decode().startswith("spmm-gfx950")


def test_host_only_helpers():
    assert S.SpMM_SplitK_Auto(28672, 16, 7168) >= 1
    assert S.SpMM_WorkspaceBytes(4096, 16, 4096, 1) == 0
    assert S.SpMM_WorkspaceBytes(4096, 16, 4096, 4) == 4 * 4096 * 16 * 4
    sk = S.SpMM_SplitK_Auto(5120, 16, 5120)
    assert 1 <= sk <= 5120 // 64
    # Split_K <= 0: sized for the library's own choice
    assert S.SpMM_WorkspaceBytes(5120, 16, 5120, 0) == 4 * 5120 * 16 * sk
    # with bias/activation the partial sums always pass through the workspace
    assert S.SpMM_WorkspaceBytesBiasAct(4096, 16, 4096, 1) == 4 * 4096 * 16
    assert S.SpMM_WorkspaceBytesBiasAct(5120, 16, 5120, 0) == 4 * 5120 * 16 * sk
    assert S.SpMM_WorkspaceBytes(5120, 24, 5120, 0) == 0  # unsupported N: nothing to size


def test_shape_errors_are_reported_without_a_gpu(capfd):
    # argument checks run before anything touches the device
    assert S.SpMM_SplitK_API(0, 0, 0, 0, 0, 0, 64, 24, 64, 0, 1) == 999
    assert "Unsupported N dimension 24" in capfd.readouterr().out
    assert S.SpMM_SplitK_API(0, 0, 0, 0, 0, 0, 100, 16, 64, 0, 1) == 1
    assert S.SpMM_SplitK_API_bitmap_v3(0, 0, 0, 0, 0, 0, 0, 0, 0, 64, 16, 64, 0, 0) == 1
    assert S.SpMM_SplitK_API(0, 0, 0, 0, 0, 0, 128, 16, 128, 0, 2) == 1  # split-K without a workspace
    assert S.SpMM_SplitK_API_BiasAct(0, 0, 0, 0, 0, 0, 64, 24, 64, 0, 1, 0, 0) == 999
    assert S.SpMM_SplitK_API_BiasAct(0, 0, 0, 0, 0, 0, 64, 16, 64, 0, 1, 0, 3) == 1  # unknown activation
