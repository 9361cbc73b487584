"""The kernels' device code holds no place where an instruction inside (or next to) an inline-assembly
statement reads a register sooner than the hardware allows after the instruction that wrote it.

The compiler does not apply its hazard rules to inline assembly; hipkittens_amd/isa_check.py states the
rules checked (vector-ALU write of a scalar register -> vector-memory read: five wait states; scalar
write of M0 -> global->LDS load: one; result of a matrix instruction -> any other use: its passes + 4;
data registers of a store of more than 64 bits -> vector-ALU write: two). Compiles every csrc/*.hip to assembly: about two minutes
on eight cores, no GPU needed.
"""
import shutil

import pytest

from hipkittens_amd import isa_check


def test_scanner_reports_the_two_hazards_and_accepts_enough_wait_states():
    bad = """
_Z3fooPi:
	v_readlane_b32 s4, v254, 3
	s_mov_b32 s5, s9
	;;#ASMSTART
	buffer_load_dwordx4 v[0:3], v9, s[4:7], s12 offen offset:16
	;;#ASMEND
	s_mov_b32 m0, s20
	buffer_load_dwordx4 v9, s[4:7], s12 offen lds
	v_readfirstlane_b32 s12, v1
	s_nop 3
	buffer_store_dword v0, v9, s[4:7], s12 offen
"""
    found = isa_check.scan(bad)
    assert [(f.register, f.wait_states, f.needed) for f in found] == [
        ("s4", 1, 5), ("s4", 3, 5), ("m0", 0, 1), ("s12", 4, 5)]
    good = """
_Z3fooPi:
	v_readlane_b32 s4, v254, 3
	s_nop 4
	buffer_load_dwordx4 v[0:3], v9, s[4:7], s12 offen
	v_readlane_b32 s12, v254, 4
	s_mov_b32 s12, s13
	s_mov_b32 m0, s20
	s_nop 0
	buffer_load_dwordx4 v9, s[4:7], s12 offen lds
"""
    assert isa_check.scan(good) == []
    # along a taken branch only: the fall-through path has the nops, the branch skips them
    branch = """
_Z3barPi:
	v_readfirstlane_b32 s8, v3
	s_cbranch_scc1 .LBB0_2
	s_nop 4
.LBB0_2:
	global_load_dword v1, v2, s[8:9]
	s_endpgm
"""
    assert [(f.register, f.wait_states) for f in isa_check.scan(branch)] == [("s8", 1)]


def test_scanner_matrix_results():
    # 8-pass FP8 instruction: its result may be touched 12 wait states after it issues; a second matrix
    # instruction waits 8 for the pipe, which counts towards the first one's 12
    text = """
_Z3bazPi:
	v_mfma_f32_16x16x128_f8f6f4 a[0:3], v[0:7], v[8:15], a[0:3]
	v_mfma_f32_16x16x128_f8f6f4 a[4:7], v[0:7], v[8:15], a[4:7]
	v_accvgpr_read_b32 v20, a0
	s_nop 2
	v_accvgpr_read_b32 v20, a1
	s_nop 5
	v_accvgpr_read_b32 v21, a4
	s_nop 1
	v_mov_b32_e32 v22, 0
	v_accvgpr_write_b32 a5, v22
	v_mfma_scale_f32_16x16x128_f8f6f4 a[8:11], v[0:3], v[8:11], a[8:11], v30, v31 op_sel_hi:[0,0,0] cbsz:4 blgp:4
	s_nop 6
	v_accvgpr_read_b32 v23, a8
	v_accvgpr_read_b32 v23, a9
	s_endpgm
"""
    found = [(f.line, f.register, f.wait_states, f.needed) for f in isa_check.scan(text)]
    assert found == [(5, "a0", 8, 12), (9, "a4", 11, 12), (15, "a8", 7, 8)]
    assert isa_check.mfma_passes("v_mfma_f32_16x16x32_bf16", "") == 4
    assert isa_check.mfma_passes("v_mfma_scale_f32_16x16x128_f8f6f4", "cbsz:4") == 8   # fp4 x fp8
    assert isa_check.mfma_passes("v_mfma_f32_32x32x64_f8f6f4", "") == 16


def test_scanner_wide_store_data():
    text = """
_Z3quxPi:
	buffer_store_dwordx4 v[4:7], v9, s[4:7], 0 offen
	v_mov_b32_e32 v5, 0
	global_store_dwordx4 v[10:11], v[12:15], off
	s_nop 0
	v_add_f32_e32 v15, v1, v2
	buffer_store_dwordx4 v[4:7], v9, s[4:7], 0 offen
	s_nop 1
	v_mov_b32_e32 v5, 0
	buffer_store_dwordx2 v[4:5], v9, s[4:7], 0 offen
	v_mov_b32_e32 v5, 0
	s_endpgm
"""
    found = [(f.line, f.register, f.wait_states, f.needed) for f in isa_check.scan(text)]
    assert found == [(4, "v5", 0, 2), (7, "v15", 1, 2)]


def test_scanner_scalar_load_destinations():
    text = """
_Z3quuPi:
	s_load_dword s20, s[4:5], s9
	s_load_dwordx4 s[24:27], s[4:5], 0x10
	s_waitcnt vmcnt(0) lgkmcnt(1)
	v_writelane_b32 v254, s20, 3
	s_add_u32 s4, s4, 8
	s_waitcnt lgkmcnt(0)
	v_writelane_b32 v254, s25, 4
	s_endpgm
"""
    found = [(f.line, f.register) for f in isa_check.scan(text)]
    assert found == [(6, "s20 (scalar load in flight)")]


def test_kernel_resources_and_scratch_rule():
    meta = """
amdhsa.kernels:
  - .agpr_count:     16
    .args:
      - .address_space:  global
        .offset:         0
        .size:           8
    .group_segment_fixed_size: 1024
    .name:           _Z1kPi
    .private_segment_fixed_size: 0
    .sgpr_count:     40
    .sgpr_spill_count: 3
    .vgpr_count:     48
    .vgpr_spill_count: 0
  - .agpr_count:     0
    .args:           []
    .group_segment_fixed_size: 0
    .name:           _Z1sPi
    .private_segment_fixed_size: 72
    .sgpr_count:     20
    .sgpr_spill_count: 0
    .vgpr_count:     256
    .vgpr_spill_count: 18
"""
    res = isa_check.kernel_resources(meta)
    assert res["_Z1kPi"] == {"agprs": 16, "lds_bytes": 1024, "scratch_bytes": 0, "sgprs": 40, "sgpr_spills": 3,
                             "vgprs": 48, "vgpr_spills": 0}
    assert [f.function for f in isa_check.memory_spills(meta)] == ["_Z1sPi"]


@pytest.fixture(scope="module")
def assembly():
    if shutil.which("hipcc") is None:
        pytest.skip("needs hipcc")
    return isa_check.assembly_of_sources()


def test_no_unseen_wait_state_violation_in_any_kernel(assembly):
    findings = isa_check.check_texts(assembly)
    assert not findings, "\n".join(str(f) for f in findings)


# Scalar registers the compiler keeps in lanes of vector registers, per kernel family: the most any instantiation
# has today. A restore (v_readlane) next to a hand-written load is what the wait-state rule above guards against, and
# every restore is an issue slot of a SIMD's only wave; the counts may go down, not up. Kernels not listed: none.
SCALAR_SPILL_CEILINGS = {
    r"moe_mxfp4_stream4_kernel": 101,
    r"moe_mxfp4_gemm_kernel": 56,
    r"moe_fp8blk_stream_kernel": 19,
    r"moe_fp8blk_gemm_kernel": 44,
}


def test_scalar_register_spills_do_not_grow(assembly):
    import re

    over = []
    for src, text in assembly.items():
        for name, res in isa_check.kernel_resources(text).items():
            ceiling = next((c for pat, c in SCALAR_SPILL_CEILINGS.items() if re.search(pat, name)), 0)
            if res.get("sgpr_spills", 0) > ceiling:
                over.append(f"{src} {name}: {res['sgpr_spills']} scalar registers spilled (ceiling {ceiling})")
    assert not over, "\n".join(over)
