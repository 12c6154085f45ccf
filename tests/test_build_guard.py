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


# with -save-temps (which the build uses, for the assembly check below) the backend runs as a step of
# its own and prints the position AFTER "remark:", with column 0 and no source excerpt
REMARKS_SAVE_TEMPS = """\
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0: Function Name: _ZN6llamql11gemm_kernelINS_9Q4KTraitsELb{d}EEEvNS_8GemmArgsE [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     TotalSGPRs: 68 [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     ScratchSize [bytes/lane]: {scratch} [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     Dynamic Stack: False [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     Occupancy [waves/SIMD]: 4 [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     VGPRs Spill: {spill} [-Rpass-analysis=kernel-resource-usage]
remark: /root/repo/llaminar_amd/csrc/gemm.hip:195:0:     LDS Size [bytes/block]: 0 [-Rpass-analysis=kernel-resource-usage]
"""


def test_the_layout_of_the_remarks_under_save_temps_is_read_too():
    """A build that keeps the intermediate files prints 'remark: file:line:col: field', not 'file:line:col:
    remark: field'; a guard that only knew the second form let two spilling kernels through."""
    clean = REMARKS_SAVE_TEMPS.format(d=1, scratch=0, spill=0)
    usage = b.check_kernel_resources(clean, "gemm.hip")
    assert len(usage) == 1 and next(iter(usage.values()))["VGPRs"] == 128
    with pytest.raises(b.SpillError) as e:
        b.check_kernel_resources(clean + REMARKS_SAVE_TEMPS.format(d=0, scratch=44, spill=10), "gemm.hip")
    assert "Lb0E" in str(e.value) and "44 B/lane" in str(e.value) and "Lb1E" not in str(e.value)
    assert b._drop_resource_remarks(clean.splitlines()) == []


def test_remarks_do_not_reach_the_build_log():
    lines = (REMARKS.format(u=3, scratch=0, spill=0) + "x.hip:1:1: warning: something real\n").splitlines()
    assert b._drop_resource_remarks(lines) == ["x.hip:1:1: warning: something real"]


def test_compile_command_asks_for_the_remarks():
    assert b.RESOURCE_FLAG == "-Rpass-analysis=kernel-resource-usage"


# ---- the second check: registers of hand-issued loads touched before their wait ----------

_PROLOGUE = """\
\t.text
_ZN6llamql4demoEv:
\ts_load_dwordx2 s[0:1], s[4:5], 0x0
"""


def _asm(body: str) -> str:
    return _PROLOGUE + body + "\ts_endpgm\n"


def test_inflight_check_accepts_use_after_wait():
    from llaminar_amd.build import check_inflight_registers

    asm = _asm("""\
\t;;#ASMSTART
\tglobal_load_dwordx4 v[8:11], v[2:3], off
\t;;#ASMEND
\t;;#ASMSTART
\tglobal_load_dwordx4 v[12:15], v[2:3], off offset:16
\t;;#ASMEND
\tv_add_u32_e32 v20, v21, v22
\t;;#ASMSTART
\ts_waitcnt vmcnt(1)
\t;;#ASMEND
\tv_and_b32_e32 v4, 0xf0f0f0f, v8
\t;;#ASMSTART
\ts_waitcnt vmcnt(0)
\t;;#ASMEND
\tv_and_b32_e32 v5, 0xf0f0f0f, v12
""")
    assert check_inflight_registers(asm, "demo.hip") == 2


def test_inflight_check_refuses_a_copy_before_the_wait():
    from llaminar_amd.build import InFlightRegisterError, check_inflight_registers

    asm = _asm("""\
\t;;#ASMSTART
\tglobal_load_dwordx4 v[8:11], v[2:3], off
\t;;#ASMEND
\tv_mov_b64_e32 v[20:21], v[8:9]
\t;;#ASMSTART
\ts_waitcnt vmcnt(0)
\t;;#ASMEND
""")
    with pytest.raises(InFlightRegisterError, match="v8"):
        check_inflight_registers(asm, "demo.hip")


def test_inflight_check_refuses_partial_wait_and_reuse_as_address():
    from llaminar_amd.build import InFlightRegisterError, check_inflight_registers

    # vmcnt(1) retires the older load only: the newer one's registers are still in flight
    asm = _asm("""\
\t;;#ASMSTART
\tglobal_load_dwordx4 v[8:11], v[2:3], off
\t;;#ASMEND
\t;;#ASMSTART
\tglobal_load_dwordx2 v[12:13], v[2:3], off offset:16
\t;;#ASMEND
\t;;#ASMSTART
\ts_waitcnt vmcnt(1)
\t;;#ASMEND
\tv_add_u32_e32 v4, v8, v12
""")
    with pytest.raises(InFlightRegisterError, match="v12"):
        check_inflight_registers(asm, "demo.hip")
    # the destination of a load in flight handed out as an address of the next load
    asm = _asm("""\
\t;;#ASMSTART
\tglobal_load_dwordx2 v[8:9], v[2:3], off
\t;;#ASMEND
\t;;#ASMSTART
\tglobal_load_dwordx4 v[16:19], v[8:9], off
\t;;#ASMEND
""")
    with pytest.raises(InFlightRegisterError, match="in flight"):
        check_inflight_registers(asm, "demo.hip")


def test_inflight_check_counts_other_memory_operations_and_resets_at_jumps():
    from llaminar_amd.build import check_inflight_registers

    # a compiler-issued store after the load is one more entry of vmcnt: vmcnt(1) then means
    # "the hand-issued load has landed"; after an unconditional branch nothing is assumed in flight
    asm = _asm("""\
\t;;#ASMSTART
\tglobal_load_dwordx4 v[8:11], v[2:3], off
\t;;#ASMEND
\tglobal_store_dword v[30:31], v32, off
\t;;#ASMSTART
\ts_waitcnt vmcnt(1)
\t;;#ASMEND
\tv_mov_b32_e32 v4, v8
\t;;#ASMSTART
\tglobal_load_dwordx4 v[12:15], v[2:3], off
\t;;#ASMEND
\ts_branch .LBB0_2
.LBB0_1:
\tv_mov_b32_e32 v5, v12
.LBB0_2:
\ts_waitcnt vmcnt(0)
""")
    assert check_inflight_registers(asm, "demo.hip") == 2
