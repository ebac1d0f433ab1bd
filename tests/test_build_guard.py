"""The build refuses a register-staged kernel that spills: its loads into registers are inline assembly with
hand-placed waits, and a spill would store such a register before its data has arrived."""

import pytest

from iree_turbine_amd import build

REMARK = "x.hip:1:1: remark: {} [-Rpass-analysis=kernel-resource-usage]"


def _remarks(name, scratch):
    return "\n".join([
        REMARK.format(f"Function Name: {name}"),
        "    1 | void k() {",
        "      | ^",
        REMARK.format("    VGPRs: 256"),
        REMARK.format(f"    ScratchSize [bytes/lane]: {scratch}"),
        REMARK.format("    VGPRs Spill: 3"),
        "x.hip:7:3: warning: something else",
    ])


def test_staged_kernel_with_scratch_is_refused():
    with pytest.raises(RuntimeError, match="spills"):
        build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_stagedItLb1EEEv", 36))


def test_other_kernels_may_use_scratch_and_warnings_pass_through():
    rest = build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_genericItLb1EEEv", 36))
    assert rest == ["x.hip:7:3: warning: something else"]
    rest = build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_stagedItLb1EEEv", 0))
    assert rest == ["x.hip:7:3: warning: something else"]
