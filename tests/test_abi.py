"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares."""
import os
import re

import spmspm_amd as S

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "spmm_api.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^[ \t]*#.*$", "", text, flags=re.M)  # preprocessor lines declare nothing
    c_part = text.split('} /* extern "C" */')[0] if '} /* extern "C" */' in text else text
    c_part = c_part.split("#ifdef __cplusplus\n}")[0]
    return sorted(set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", c_part)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for n in ("SpMM_SplitK_API", "SpMM_SplitK_API_bitmap_v3", "InitSparseMatrixA_bitmap",
              "Our_GenSparseMatrixBinFile", "SpMM_SplitK_Auto", "SpMM_WorkspaceBytes", "SpMM_Version", "SpMM_TimeNextCall",
              "SpMM_SplitK_API_BiasAct", "SpMM_WorkspaceBytesBiasAct", "SpMM_EncodeDevice_Bitmaps",
              "SpMM_EncodeDevice_Values", "SpMM_SplitK_TableSet", "SpMM_SplitK_TableLoad", "SpMM_SplitK_TableSave",
              "SpMM_SplitK_TableClear", "SpMM_SplitK_API_NoAlloc", "SpMM_SplitK_API_Sized", "SpMM_KernelName",
              "SpMM_SplitK_TableSetMany", "SpMM_SplitK_CostModel", "SpMM_SplitK_AutoNoAlloc", "SpMM_ReadWeightFiles",
              "SpMM_LoadWeightFiles", "SpMM_FreeWeights", "SpMM_ShaderClockProbe",
              "SpMM_EncodeDevice_OnePass", "SpMM_EncodeDevice_ScratchBytes"):
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
    capfd.readouterr()
    assert S.SpMM_SplitK_API_NoAlloc(0, 0, 0, 0, 0, 0, 64, 24, 64, 1) == 999
    assert S.SpMM_SplitK_API_NoAlloc(0, 0, 0, 0, 0, 0, 16384, 128, 4096, 8) == 1  # partial sums beyond the array
    assert "holds at most" in capfd.readouterr().out


def test_split_table_overrides_the_cost_model_and_round_trips_through_a_file(tmp_path):
    import pytest
    S.SpMM_SplitK_TableClear()
    model, model_n32 = S.SpMM_SplitK_Auto(28672, 16, 7168), S.SpMM_SplitK_Auto(28672, 32, 7168)
    other = model + 1
    try:
        S.SpMM_SplitK_TableSet(28672, 16, 7168, other)
        S.SpMM_SplitK_TableSet(5120, 16, 5120, 1000)  # more batches than group-tile columns: clamped when used
        assert S.SpMM_SplitK_Auto(28672, 16, 7168) == other
        assert S.SpMM_SplitK_Auto(5120, 16, 5120) == 5120 // 64
        assert S.SpMM_SplitK_Auto(28672, 32, 7168) == model_n32  # other N: not in the table
        assert S.SpMM_WorkspaceBytes(28672, 16, 7168, 0) == 4 * 28672 * 16 * other
        assert S.SpMM_WorkspaceBytesBiasAct(28672, 16, 7168, 0) == 4 * 28672 * 16 * other
        path = tmp_path / "splitk.txt"
        assert S.SpMM_SplitK_TableSave(path) == 2
        lines = [l for l in path.read_text().splitlines() if not l.startswith("#")]
        assert sorted(lines) == sorted(["28672 16 7168 %d" % other, "5120 16 5120 1000"])
        S.SpMM_SplitK_TableClear()
        assert S.SpMM_SplitK_Auto(28672, 16, 7168) == model
        path.write_text("# tuned on some day\n\n  28672 16 7168 %d\n4096 16 4096 2 trailing words are ignored\n" % other)
        assert S.SpMM_SplitK_TableLoad(path) == 2
        assert S.SpMM_SplitK_Auto(28672, 16, 7168) == other and S.SpMM_SplitK_Auto(4096, 16, 4096) == 2
        bad = tmp_path / "bad.txt"
        bad.write_text("28672 16 7168\n")
        with pytest.raises(OSError):
            S.SpMM_SplitK_TableLoad(bad)
        with pytest.raises(OSError):
            S.SpMM_SplitK_TableLoad(tmp_path / "missing.txt")
        with pytest.raises(ValueError):
            S.SpMM_SplitK_TableSet(100, 16, 64, 2)  # not a shape the library runs
        with pytest.raises(ValueError):
            S.SpMM_SplitK_TableSet(128, 16, 128, 0)
    finally:
        S.SpMM_SplitK_TableClear()


def test_shipped_split_table_loads_and_covers_the_decode_widths():
    """The measured table in spmspm_amd/tuned/ parses, lists the OPT-13B, OPT-30B and OPT-66B linears at N = 8, 16,
    32, 64 and 128, and takes precedence over the cost model once loaded."""
    path = os.path.join(ROOT, "spmspm_amd", "tuned", "splitk_mi355x.txt")
    try:
        S.SpMM_SplitK_TableClear()
        assert S.SpMM_SplitK_TableLoad(path) == 60
        for M, K in [(15360, 5120), (5120, 5120), (20480, 5120), (5120, 20480), (28672, 7168), (7168, 7168),
                     (21504, 7168), (7168, 28672), (27648, 9216), (9216, 9216), (36864, 9216), (9216, 36864)]:
            for N in (8, 16, 32):
                assert 1 <= S.SpMM_SplitK_Auto(M, N, K) <= 12
            for N in (64, 128):
                assert 1 <= S.SpMM_SplitK_Auto(M, N, K) <= 32
        table = {}
        for line in open(path):
            if line.strip() and not line.startswith("#"):
                m, n, k, sk = map(int, line.split())
                table[(m, n, k)] = sk
        assert all(S.SpMM_SplitK_Auto(m, n, k) == sk for (m, n, k), sk in table.items())
    finally:
        S.SpMM_SplitK_TableClear()
    # at least one listed shape is a case where the measurement overrules the cost model
    assert any(S.SpMM_SplitK_Auto(m, n, k) != sk for (m, n, k), sk in table.items())


def test_split_table_file_named_in_the_environment_is_loaded_on_first_use(tmp_path):
    import subprocess
    import sys
    path = tmp_path / "t.txt"
    path.write_text("28672 16 7168 7\n")
    code = "import spmspm_amd as S; print(S.SpMM_SplitK_Auto(28672, 16, 7168), S.SpMM_SplitK_Auto(4096, 16, 4096))"
    env = dict(os.environ, SPMM_SPLITK_TABLE=str(path), PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True).stdout.split()
    assert out[0] == "7" and int(out[1]) >= 1
    env["SPMM_SPLITK_TABLE"] = str(tmp_path / "missing.txt")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True)
    assert "cannot be opened" in r.stdout and int(r.stdout.split()[-2]) >= 1


def test_shipped_table_is_loaded_by_default_and_an_empty_variable_switches_it_off():
    """Without SPMM_SPLITK_TABLE the library finds tuned/splitk_mi355x.txt beside its own directory on first use; with
    the variable set to an empty string the cost model stands alone."""
    import subprocess
    import sys
    path = os.path.join(ROOT, "spmspm_amd", "tuned", "splitk_mi355x.txt")
    table = {}
    for line in open(path):
        if line.strip() and not line.startswith("#"):
            m, n, k, sk = map(int, line.split())
            table[(m, n, k)] = sk
    code = ("import spmspm_amd as S\n"
            "for m, n, k in %r:\n"
            "    print(m, n, k, S.SpMM_SplitK_Auto(m, n, k), S.SpMM_SplitK_CostModel(m, n, k))" % (sorted(table),))
    env = {k: v for k, v in os.environ.items() if k != "SPMM_SPLITK_TABLE"}
    env["PYTHONPATH"] = ROOT
    rows = [tuple(map(int, l.split())) for l in
            subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True).stdout.splitlines()]
    assert len(rows) == len(table)
    assert all(auto == table[(m, n, k)] for m, n, k, auto, _ in rows)
    assert any(auto != model for _, _, _, auto, model in rows)  # the table does overrule the model somewhere
    env["SPMM_SPLITK_TABLE"] = ""
    rows = [tuple(map(int, l.split())) for l in
            subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True).stdout.splitlines()]
    assert all(auto == model for _, _, _, auto, model in rows)


def test_table_set_many_records_all_or_nothing():
    import pytest
    S.SpMM_SplitK_TableClear()
    try:
        S.SpMM_SplitK_TableSetMany([(4096, 16, 4096, 3), (8192, 32, 4096, 5)])
        assert S.SpMM_SplitK_Auto(4096, 16, 4096) == 3 and S.SpMM_SplitK_Auto(8192, 32, 4096) == 5
        with pytest.raises(ValueError):
            S.SpMM_SplitK_TableSetMany([(4096, 8, 4096, 7), (100, 16, 64, 2)])  # second entry is no shape the library runs
        assert S.SpMM_SplitK_Auto(4096, 8, 4096) == S.SpMM_SplitK_CostModel(4096, 8, 4096)
        S.SpMM_SplitK_TableSetMany([])
        # many updates in a row leave one table, not one copy per update alive
        for i in range(2000):
            S.SpMM_SplitK_TableSet(4096, 16, 4096, 1 + i % 7)
        assert S.SpMM_SplitK_Auto(4096, 16, 4096) == 1 + 1999 % 7
    finally:
        S.SpMM_SplitK_TableClear()


def test_no_alloc_entry_point_clamps_its_own_split_and_refuses_an_explicit_one(capfd):
    """With Split_K <= 0 the library's choice gives way to the largest split whose fp32 partial sums fit the 32 MiB
    array; an explicit Split_K beyond it is refused before anything touches the device."""
    M, N, K = 20480, 128, 5120
    S.SpMM_SplitK_TableClear()
    try:
        S.SpMM_SplitK_TableSet(M, N, K, 6)  # 4*M*N*6 = 60 MiB of partial sums
        assert S.SpMM_SplitK_Auto(M, N, K) == 6
        fit = S.SpMM_SplitK_AutoNoAlloc(M, N, K)
        assert fit == 3 and 4 * M * N * fit <= S.NOALLOC_SCRATCH_BYTES < 4 * M * N * (fit + 1)
        capfd.readouterr()
        rc = S.library().SpMM_SplitK_API_NoAlloc(None, None, None, None, None, None, M, N, K, 0)
        out = capfd.readouterr().out
        assert "holds at most" not in out  # not refused for its size; without a GPU the device look-up fails instead
        assert rc != 1 or "scratch array" in out
        assert S.library().SpMM_SplitK_API_NoAlloc(None, None, None, None, None, None, M, N, K, 6) == 1
        assert "holds at most" in capfd.readouterr().out
        # a single slab beyond the array: the automatic call runs unsplit
        assert S.SpMM_SplitK_AutoNoAlloc(36864, 256, 9216) == 1
        assert S.SpMM_SplitK_AutoNoAlloc(5120, 16, 5120) == S.SpMM_SplitK_Auto(5120, 16, 5120)
    finally:
        S.SpMM_SplitK_TableClear()


def test_tuner_candidates_and_presets():
    from spmspm_amd import tuner
    assert tuner.candidate_splits(5120) == list(range(1, 13))
    assert tuner.candidate_splits(256) == [1] and tuner.candidate_splits(512) == [1, 2]
    assert (28672, 7168) in tuner.PRESETS["opt30b"] and len(tuner.PRESETS["opt13b"]) == 4


def test_null_and_misaligned_pointers_are_refused_on_the_host(capfd):
    """Addresses the kernels cannot use (null, or off the 16-byte grid their loads and stores assume) never reach the
    device: every entry point returns hipErrorInvalidValue before it launches anything."""
    a = 1 << 20  # a plausible, aligned, never dereferenced address
    ok = dict(values=a, bitmaps=a, offsets=a, X=a, C=a)
    for name, bad in (("values", 0), ("values", a + 2), ("bitmaps", a + 4), ("offsets", a + 2), ("X", a + 8), ("C", a + 4), ("X", 0)):
        p = dict(ok, **{name: bad})
        capfd.readouterr()
        assert S.SpMM_SplitK_API(0, p["values"], p["bitmaps"], p["offsets"], p["X"], p["C"], 64, 16, 64, 0, 1) == 1, name
        assert "null or misaligned" in capfd.readouterr().out
        assert S.SpMM_SplitK_API_NoAlloc(0, p["values"], p["bitmaps"], p["offsets"], p["X"], p["C"], 64, 16, 64, 1) == 1
    assert S.SpMM_SplitK_API(0, a, a, a, a, a, 128, 16, 128, a + 4, 2) == 1  # a workspace off the grid
    assert S.SpMM_SplitK_API_BiasAct(0, a, a, a, a, a, 64, 16, 64, a, 1, a + 1, 0) == 1  # an odd bias address


def test_sized_entry_point_refuses_a_small_workspace_without_a_gpu(capfd):
    """The size check comes before anything touches the device: a too-small workspace returns
    hipErrorInvalidValue for an explicit split and for the library's own choice, also after the table has changed
    that choice behind the caller's back."""
    M, N, K = 4096, 16, 4096
    need4 = S.SpMM_WorkspaceBytes(M, N, K, 4)

    def call(m, n, k, ws_bytes, sk):  # raw C call: null stream and null pointers, nothing is launched
        return S.library().SpMM_SplitK_API_Sized(None, None, None, None, None, None, m, n, k, None, ws_bytes, sk)

    assert call(M, N, K, need4 - 1, 4) == 1
    assert "workspace" in capfd.readouterr().out
    S.SpMM_SplitK_TableClear()
    try:
        small = S.SpMM_WorkspaceBytes(M, N, K, 0)
        sk0 = S.SpMM_SplitK_Auto(M, N, K)
        S.SpMM_SplitK_TableSet(M, N, K, sk0 + 3)           # the choice grows after the buffer was sized
        assert S.SpMM_WorkspaceBytes(M, N, K, 0) > small
        assert call(M, N, K, small, 0) == 1
    finally:
        S.SpMM_SplitK_TableClear()
    # shape errors keep their own codes
    assert call(M, 24, K, 1 << 30, 1) == 999
    assert call(M + 1, N, K, 1 << 30, 1) == 1


def test_kernel_name_follows_the_dispatch():
    name = lambda *a: (S.library().SpMM_KernelName(*a) or b"").decode()
    assert name(28672, 16, 7168, 4) == "spmm::spmm_bitmap_rows<1, true>"
    assert name(28672, 8, 7168, 1) == "spmm::spmm_bitmap_rows<1, false>"
    assert name(28672, 32, 7168, 1) == "spmm::spmm_bitmap_rows<2, false>"
    assert name(9216, 64, 36864, 14) == "spmm::spmm_bitmap_wide<4, true>"
    assert name(28672, 64, 7168, 4) == "spmm::spmm_bitmap_wide<4, true>"
    assert name(5120, 64, 5120, 3) == "spmm::spmm_bitmap_rows<4, true>"  # too few tiles for one round of long batches
    assert name(128, 64, 4096, 2) == "spmm::spmm_bitmap_rows<4, true>"   # fewer than 256 rows
    assert name(9216, 256, 36864, 7) == "spmm::spmm_bitmap_wide<8, true>"
    assert name(9216, 24, 36864, 1) == "" and name(100, 16, 64, 1) == ""
    # the name is that of SpMM_SplitK_API / _Sized / _NoAlloc: fp32 partial sums exactly when K is split
    assert name(5120, 16, 5120, 1).endswith("false>") and name(5120, 16, 5120, 2).endswith("true>")


def test_row_count_limit_is_reported(capfd):
    """Row blocks are the z dimension of the launch grid: more than 65535 of them is refused before any launch."""
    L = S.library()
    assert L.SpMM_SplitK_API(None, None, None, None, None, None, 64 * 65536, 16, 64, None, 1) == 1
    assert "65535" in capfd.readouterr().out
