"""The build refuses kernels that spill registers (CPU only; nothing is compiled here).

Kernels that issue loads as inline assembly and wait for them by hand are only correct
while the compiler spills nothing; llaminar_amd.build parses the compiler's
kernel-resource-usage remarks and fails the build otherwise.
"""
import pytest

from llaminar_amd import build as b

REMARKS = """\
gemv_quad.h:702:1: remark: Function Name: _ZN6llamql16gemv_quad_kernelINS_7Q4KQuadELi1ELi{u}ELi0EEEvNS_8QuadArgsE [-Rpass-analysis=kernel-resource-usage]
  702 |     {{
      | ^
gemv_quad.h:702:1: remark:     TotalSGPRs: 48 [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     ScratchSize [bytes/lane]: {scratch} [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     Dynamic Stack: False [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     Occupancy [waves/SIMD]: 4 [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     VGPRs Spill: {spill} [-Rpass-analysis=kernel-resource-usage]
gemv_quad.h:702:1: remark:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
"""


def test_clean_kernels_pass_and_are_reported():
    text = REMARKS.format(u=3, scratch=0, spill=0) + REMARKS.format(u=2, scratch=0, spill=0)
    usage = b.check_kernel_resources(text, "gemv.hip")
    assert len(usage) == 2
    assert all(u["VGPRs"] == 128 and u["VGPRs Spill"] == 0 for u in usage.values())


@pytest.mark.parametrize("scratch,spill", [(60, 38), (4, 0), (0, 1)])
def test_a_spilling_kernel_fails_the_build(scratch, spill):
    text = REMARKS.format(u=3, scratch=0, spill=0) + REMARKS.format(u=4, scratch=scratch, spill=spill)
    with pytest.raises(b.SpillError) as e:
        b.check_kernel_resources(text, "gemv.hip")
    assert "Li4E" in str(e.value) and "Li3E" not in str(e.value)


def test_remarks_do_not_reach_the_build_log():
    lines = (REMARKS.format(u=3, scratch=0, spill=0) + "x.hip:1:1: warning: something real\n").splitlines()
    assert b._drop_resource_remarks(lines) == ["x.hip:1:1: warning: something real"]


def test_compile_command_asks_for_the_remarks():
    assert b.RESOURCE_FLAG == "-Rpass-analysis=kernel-resource-usage"
