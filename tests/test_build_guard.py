"""The build refuses a register-staged kernel that spills: its loads into registers are inline assembly with
hand-placed waits, and a spill would store such a register before its data has arrived."""

import pytest

from iree_turbine_amd import build

REMARK = "x.hip:1:1: remark: {} [-Rpass-analysis=kernel-resource-usage]"


def _remarks(name, scratch, vgpr_spill=0, occupancy=1):
    return "\n".join([
        REMARK.format(f"Function Name: {name}"),
        "    1 | void k() {",
        "      | ^",
        REMARK.format("    VGPRs: 256"),
        REMARK.format(f"    ScratchSize [bytes/lane]: {scratch}"),
        REMARK.format(f"    Occupancy [waves/SIMD]: {occupancy}"),
        REMARK.format("    SGPRs Spill: 2"),
        REMARK.format(f"    VGPRs Spill: {vgpr_spill}"),
        "x.hip:7:3: warning: something else",
    ])


def test_staged_kernel_with_scratch_is_refused():
    with pytest.raises(RuntimeError, match="spills"):
        build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_stagedItLb1EEEv", 36))


def test_staged_kernel_with_a_register_spill_or_another_occupancy_is_refused():
    with pytest.raises(RuntimeError, match="spills 3 vector registers"):
        build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_stagedItLb1EEEv", 0, vgpr_spill=3))
    with pytest.raises(RuntimeError, match="2 waves per SIMD, expected 1"):
        build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_stagedItLb1EEEv", 0, occupancy=2))
    with pytest.raises(RuntimeError, match="expected 7"):
        build._check_resource_remarks(_remarks("_ZN5mi35518gemm_f16_nt_skinnyIfLb1EEEv", 0, occupancy=8))
    build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp4_skinnyIfEEv", 0, occupancy=2))


def test_other_kernels_may_use_scratch_and_warnings_pass_through():
    rest = build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_genericItLb1EEEv", 36, vgpr_spill=3, occupancy=4))
    assert rest == ["x.hip:7:3: warning: something else"]
    rest = build._check_resource_remarks(_remarks("_ZN5mi35517gemm_mxfp8_stagedItLb1EEEv", 0))
    assert rest == ["x.hip:7:3: warning: something else"]


def test_remarks_with_the_location_behind_the_word_remark_are_read_too():
    """With preprocessed sources (-save-temps) the compiler prints 'remark: file:line:col: Field: N'."""
    located = "remark: /x/gemm_mxfp8.hip:597:0: {} [-Rpass-analysis=kernel-resource-usage]"
    text = "\n".join([
        located.format("Function Name: _ZN5mi35517gemm_mxfp8_streamItLb1EEEvPKhS2_S2_S2_PT_iiiiiif"),
        located.format("    VGPRs: 199"),
        located.format("    ScratchSize [bytes/lane]: 0"),
        located.format("    Occupancy [waves/SIMD]: 1"),
        located.format("    VGPRs Spill: 0"),
    ])
    assert build._check_resource_remarks(text) == []
    with pytest.raises(RuntimeError, match="spills \\(16 bytes"):
        build._check_resource_remarks(text.replace("ScratchSize [bytes/lane]: 0", "ScratchSize [bytes/lane]: 16"))
    with pytest.raises(RuntimeError, match="2 waves per SIMD, expected 1"):
        build._check_resource_remarks(text.replace("Occupancy [waves/SIMD]: 1", "Occupancy [waves/SIMD]: 2"))
