"""The build's checks on hand-pipelined kernels (slang_amd/build.py), on synthetic compiler output."""
import pytest

from slang_amd import build

ASM_OK = """
_ZN2cv12_GLOBAL__N_113mlpWideKernelILi2ELi2EEEvNS_7MlpArgsE:
	global_load_dwordx4 v[96:99], v0, s[22:23] nt
	v_add_u32_e32 v1, v2, v3
	global_store_dwordx2 v[4:5], v[0:1], off
	s_waitcnt vmcnt(1)
	v_mov_b32_e32 v4, v98
	global_load_dwordx4 v[96:99], v0, s[4:5] nt
	global_load_dwordx4 v[100:103], v0, s[6:7] nt
	s_waitcnt vmcnt(1)
	v_mov_b32_e32 v5, v97
	s_waitcnt vmcnt(0)
.Lfunc_end0:
_ZN2cv5otherEv:
	global_load_dwordx4 v[8:11], v0, s[4:5] nt
	v_mov_b32_e32 v1, v9
.Lfunc_end1:
"""


def test_pending_register_scan_accepts_clean_code():
    assert build._check_inflight_registers("x.hip", "mlpWideKernel", ASM_OK) == 3


@pytest.mark.parametrize("bad", ["\tv_mov_b32_e32 v1, v97\n", "\tv_pk_max_f16 v96, v1, v2\n", "\tglobal_store_dwordx2 v[4:5], v[98:99], off\n",
                                 "\tv_mfma_f32_32x32x16_f16 v[0:15], v[92:97], v[20:23], 0\n"])
def test_pending_register_scan_rejects_a_touch(bad):
    asm = ASM_OK.replace("\tv_add_u32_e32 v1, v2, v3\n", bad, 1)
    with pytest.raises(RuntimeError, match="pending"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", asm)


def test_pending_register_scan_ignores_a_wait_that_does_not_cover_the_load():
    # vmcnt(3) after only one younger vector-memory instruction can return while the load is on its way: the scan goes
    # on to the wait that does cover it, and sees the touch in between
    asm = ASM_OK.replace("\ts_waitcnt vmcnt(1)\n\tv_mov_b32_e32 v4, v98\n", "\ts_waitcnt vmcnt(3)\n\tv_mov_b32_e32 v4, v98\n\ts_waitcnt vmcnt(0)\n", 1)
    with pytest.raises(RuntimeError, match="pending"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", asm)


LOOP_ASM = """
_ZN2cv12_GLOBAL__N_113mlpWideKernelILi2ELi2EEEvNS_7MlpArgsE:
	global_load_dwordx4 v[96:99], v0, s[22:23] nt
.LBB0_1:
	s_waitcnt vmcnt(0)
	v_mov_b32_e32 v4, v98
	global_load_dwordx4 v[96:99], v0, s[4:5] nt
%s	v_add_u32_e32 v1, v2, v3
	s_cbranch_scc1 .LBB0_1
	s_endpgm
.Lfunc_end0:
"""


def test_pending_register_scan_follows_the_loop_back_edge():
    # the refill's covering wait sits at the top of the next round of the loop
    assert build._check_inflight_registers("x.hip", "mlpWideKernel", LOOP_ASM % "") == 2
    with pytest.raises(RuntimeError, match="pending"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", LOOP_ASM % "\tv_mov_b32_e32 v5, v99\n")


def test_pending_register_scan_fails_closed():
    # an instruction form the scan does not know, registers it cannot parse, a load without a covering wait
    with pytest.raises(RuntimeError, match="does not know the instruction form"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", LOOP_ASM % "\timage_sample v[0:3], v[4:5], s[0:7], s[8:11]\n")
    with pytest.raises(RuntimeError, match="cannot parse"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", LOOP_ASM % "\tv_mov_b32_e32 v5, v[96\n")
    open_ended = LOOP_ASM.replace("\ts_cbranch_scc1 .LBB0_1\n\ts_endpgm\n", "") % ""
    with pytest.raises(RuntimeError, match="runs off the end"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", open_ended)
    with pytest.raises(RuntimeError, match="indirect control flow"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", LOOP_ASM % "\ts_setpc_b64 s[0:1]\n")


def test_pending_register_scan_takes_both_sides_of_a_branch():
    # a touch that only one side of a conditional branch reaches is still found
    asm = LOOP_ASM % "\ts_cbranch_execz .LBB0_2\n\tv_mov_b32_e32 v7, v96\n.LBB0_2:\n"
    with pytest.raises(RuntimeError, match="pending"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", asm)
    ok = LOOP_ASM % "\ts_cbranch_execz .LBB0_2\n\tglobal_store_dwordx2 v[8:9], v[0:1], off\n.LBB0_2:\n"
    assert build._check_inflight_registers("x.hip", "mlpWideKernel", ok) == 2


def test_pending_register_scan_must_find_its_loads():
    with pytest.raises(RuntimeError, match="no hand-issued load"):
        build._check_inflight_registers("x.hip", "mlpWideKernel", "_ZN2cv5otherEv:\n\ts_endpgm\n.Lfunc_end0:\n")


REMARKS = """x.h:1:1: remark: Function Name: _ZN2cv13mlpWideKernelILi2EEEv [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     VGPRs: 156 [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     ScratchSize [bytes/lane]: %d [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     VGPRs Spill: %d [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark: Function Name: _ZN2cv5otherEv [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     VGPRs Spill: 7 [-Rpass-analysis=kernel-resource-usage]
"""


def test_spill_check():
    build._check_no_spills("x.hip", "mlpWideKernel", REMARKS % (0, 0))      # another kernel's spills do not matter
    with pytest.raises(RuntimeError, match="VGPRs Spill"):
        build._check_no_spills("x.hip", "mlpWideKernel", REMARKS % (0, 4))
    with pytest.raises(RuntimeError, match="ScratchSize"):
        build._check_no_spills("x.hip", "mlpWideKernel", REMARKS % (20, 0))
