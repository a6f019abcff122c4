"""Host-side checks of the build helpers (no GPU, no compiler run)."""

from cornserve_amd.build import check_hand_managed_acc_registers

_CLEAN = """
_Z6kernelv:
	v_add_u32_e32 v1, v2, v3
	;;#ASMSTART
	v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]
	;;#ASMEND
	ds_read_b128 v[8:11], v12
	;;#ASMSTART
	v_accvgpr_read_b32 v5, a[7]
	;;#ASMEND
	s_endpgm
"""

_SPILL = _CLEAN.replace("\tds_read_b128 v[8:11], v12\n", "\tv_accvgpr_write_b32 a17, v5\n\tds_read_b128 v[8:11], v12\n")
_STAGED = _CLEAN.replace("\tds_read_b128 v[8:11], v12\n", "\tglobal_load_dwordx4 a[0:3], v172, s[8:9] offset:256\n")
_COMPILER_ONLY = """
_Z7kernel2v:
	v_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]
	v_accvgpr_read_b32 v5, a1
	s_endpgm
"""


def test_clean_kernel_passes():
    assert check_hand_managed_acc_registers(_CLEAN) == []


def test_compiler_spill_into_accumulation_register_is_reported():
    out = check_hand_managed_acc_registers(_SPILL)
    assert len(out) == 1 and out[0].startswith("_Z6kernelv")


def test_compiler_load_into_accumulation_register_is_reported():
    assert len(check_hand_managed_acc_registers(_STAGED)) == 1


def test_kernels_without_inline_accumulators_are_not_checked():
    # a kernel whose accumulators the compiler manages itself may use the registers freely
    assert check_hand_managed_acc_registers(_COMPILER_ONLY) == []
    assert len(check_hand_managed_acc_registers(_COMPILER_ONLY + _SPILL)) == 1
