"""The build refuses tile kernels that spill registers: their s_waitcnt vmcnt values are counted by hand, and a spill's
scratch accesses would add to the count."""
from amct_amd import build


REMARKS = """x.hip:1:1: remark: Function Name: _ZN4amct17w4a16_tile_wide16ILb1EEEvNS_9W4A16ArgsE [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark:     ScratchSize [bytes/lane]: 72 [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark:     VGPRs Spill: 17 [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark: Function Name: _ZN4amct12w4a16_decodeILi1EEEvNS_9W4A16ArgsE [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark:     VGPRs Spill: 3 [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark: Function Name: _ZN4amct15w8a8_tile_mix16ILi2EEEvNS_8W8A8ArgsENS_7MixPlanE [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
x.hip:1:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
"""


def test_spilling_tile_kernels_are_reported_and_others_are_not():
    bad = build._spilling_kernels(REMARKS)
    assert len(bad) == 2 and all("w4a16_tile_wide16" in b for b in bad)
    assert any("VGPRs Spill: 17" in b for b in bad) and any("ScratchSize [bytes/lane]: 72" in b for b in bad)
    assert build._spilling_kernels(REMARKS.split("x.hip:1:1: remark: Function Name: _ZN4amct12")[1]) == []
