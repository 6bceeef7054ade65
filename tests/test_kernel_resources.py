"""No kernel of the library spills registers or uses scratch memory (checked on the compiler's own record of the
gfx950 code, no GPU needed).  A spill inside the tile loop costs a large factor and fails no numerical test."""
import pytest

from spmspm_amd import build


@pytest.mark.parametrize("source", ["spmm_api.hip", "encoder_device.hip"])
def test_no_kernel_spills(source):
    res = build.kernel_resources(source)
    assert res, "no kernels found in " + source
    for name, r in res.items():
        assert r["vgpr_spill"] == 0 and r["sgpr_spill"] == 0 and r["scratch_bytes"] == 0, (name, r)


def test_main_kernel_occupancy_budget():
    """Registers decide how many workgroups a CU holds: at most 128 for the 16-column kernel (four workgroups per
    CU), 168 for 32 columns (three), 256 for 64 (two)."""
    res = build.kernel_resources("spmm_api.hip")
    limit = {"ILi1E": 128, "ILi2E": 168, "ILi4E": 256}
    seen = 0
    for name, r in res.items():
        if "spmm_bitmap_rows" in name:
            key = next(k for k in limit if k in name)
            assert r["vgpr"] <= limit[key], (name, r)
            seen += 1
    assert seen == 6
