"""The build's check that kernels with load requests in flight across their loop use no scratch memory: the parser
of the compiler's resource report, on a report written out here (no compiler run)."""
from helpers import pkg

B = pkg("build")

REPORT = """\
a.hip:10:1: remark: Function Name: _ZN2mi17a16_rows32_kernelILi0EEEvNS_10Rows32ArgsE [-Rpass-analysis=kernel-resource-usage]
a.hip:10:1: remark:     VGPRs: 118 [-Rpass-analysis=kernel-resource-usage]
a.hip:10:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:10:1: remark:     LDS Size [bytes/block]: 65536 [-Rpass-analysis=kernel-resource-usage]
a.hip:90:1: remark: Function Name: _ZN2mi20a16_rows16_w4_kernelILi1ELi2ELi4ELb1EEEvNS_12Rows32W4ArgsE [-Rpass-analysis=kernel-resource-usage]
a.hip:90:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
a.hip:90:1: remark:     ScratchSize [bytes/lane]: 64 [-Rpass-analysis=kernel-resource-usage]
a.hip:200:1: remark: Function Name: _ZN2mi15a16_other_kernelEv [-Rpass-analysis=kernel-resource-usage]
a.hip:200:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]
"""


def test_spilling_ring_kernels_are_named_and_others_left_alone():
    bad = B._spilling_kernels(REPORT, ("rows32", "rows16"))
    assert len(bad) == 1 and "a16_rows16_w4_kernelILi1ELi2ELi4ELb1" in bad[0] and "64 bytes/lane" in bad[0]
    assert B._spilling_kernels(REPORT, ("wide",)) == []
    assert B._spilling_kernels("", ("rows32",)) == []


def test_every_guarded_file_is_a_source_of_the_library():
    assert set(B.NO_SPILL) <= set(B.SOURCES)
