"""The build-time check of hand-issued loads: flags a register that is read or overwritten while
its load is still in flight, follows forward branches, and accepts the pipelined pattern."""
from tritium_amd import check_isa

HEAD = "_Z14tk_gemm_kernelILi4ELi1ELb0EEv9TkProblemPKS0_PKi:\n"
TAIL = ".Lfunc_end0:\n"


def run(body):
    return check_isa.check_text(HEAD + body + TAIL)


def test_copy_of_a_register_in_flight_is_flagged():
    bad = run("""
	global_load_dwordx4 v[66:69], v[104:105], off offset:512
	global_load_lds_dwordx4 v100, s[6:7]
	v_mov_b32_e32 v5, v66
	s_waitcnt vmcnt(0)
	v_mov_b32_e32 v66, v5
""")
    (name, hz), = bad.items()
    assert [(h[2], h[1].split()[0]) for h in hz] == [(66, "v_mov_b32_e32")]
    assert "v66" in check_isa.report(bad)


def test_overwrite_and_partial_waits():
    # vmcnt(1) retires the older load only: v[10:13] may be used, v[20:23] not yet
    ok = run("""
	global_load_dwordx4 v[10:13], v[2:3], off
	global_load_dwordx4 v[20:23], v[2:3], off offset:512
	s_waitcnt vmcnt(1)
	v_and_b32_e32 v30, 0x3030303, v10
	s_waitcnt vmcnt(0)
	v_and_b32_e32 v31, 0x3030303, v20
""")
    assert ok == {}
    bad = run("""
	global_load_dwordx4 v[10:13], v[2:3], off
	global_load_dwordx4 v[20:23], v[2:3], off offset:512
	s_waitcnt vmcnt(1)
	v_mov_b32_e32 v21, 0
""")
    assert list(bad.values())[0][0][2] == 21


def test_lds_reads_one_step_ahead():
    # lgkmcnt(2) retires all but the two youngest LDS reads: the pair read first may feed the matrix
    # instruction, the pair read ahead may not be touched until its own wait
    ok = run("""
	ds_read_b128 v[10:13], v2
	ds_read_b128 v[14:17], v2 offset:512
	ds_read_b128 v[20:23], v2 offset:4096
	ds_read_b128 v[24:27], v2 offset:4608
	s_waitcnt lgkmcnt(2)
	v_mfma_i32_32x32x32_i8 v[40:55], v[10:13], v[30:33], v[40:55]
	s_waitcnt lgkmcnt(0)
	v_mfma_i32_32x32x32_i8 v[40:55], v[20:23], v[30:33], v[40:55]
""")
    assert ok == {}
    bad = run("""
	ds_read_b128 v[10:13], v2
	ds_read_b128 v[20:23], v2 offset:4096
	s_waitcnt lgkmcnt(1)
	v_mov_b32_e32 v5, v22
	s_waitcnt lgkmcnt(0)
""")
    assert list(bad.values())[0][0][2] == 22
    # a vmcnt wait does not retire LDS reads
    bad = run("""
	ds_read_b128 v[10:13], v2
	s_waitcnt vmcnt(0)
	v_mov_b32_e32 v5, v10
""")
    assert list(bad.values())[0][0][2] == 10


def test_branch_targets_start_from_the_state_at_the_jump():
    # the zero-fill path is entered by a jump taken before the loads were issued
    ok = run("""
	s_cbranch_scc0 .LBB0_2
	global_load_dwordx4 v[82:85], v[6:7], off offset:512
	s_branch .LBB0_3
.LBB0_2:
	v_mov_b32_e32 v82, 0
.LBB0_3:
	s_waitcnt vmcnt(0)
	v_and_b32_e32 v1, 0x3030303, v82
""")
    assert ok == {}


def test_other_kernels_are_not_scanned():
    text = "_Z14tk_flow_kernelILi1EEvv:\n\tglobal_load_dwordx4 v[1:4], v[8:9], off\n\tv_mov_b32_e32 v0, v1\n.Lfunc_end1:\n"
    assert check_isa.check_text(text) == {}


def test_register_budgets():
    """A kernel over its budget, one that spills, and one missing from the assembly are all reported."""
    meta = """
amdhsa.kernels:
  - .name:           _Z5alphaILi1EEvv
    .vgpr_count:     128
    .vgpr_spill_count: 0
  - .name:           _Z4betaILi2EEvv
    .vgpr_count:     169
    .vgpr_spill_count: 0
  - .name:           _Z5gammaILi3EEvv
    .vgpr_count:     100
    .vgpr_spill_count: 4
"""
    budgets = (("alphaILi1E", 128), ("betaILi2E", 168), ("gammaILi3E", 128), ("deltaILi4E", 64))
    bad = check_isa.check_budgets(meta, budgets)
    assert ("_Z4betaILi2EEvv", 169, 168) in bad and ("_Z5gammaILi3EEvv", 10100, 128) in bad and ("deltaILi4E", None, 64) in bad
    assert not any("alpha" in b[0] for b in bad) and len(bad) == 3


def test_static_lds_rule():
    """A listed kernel with static LDS in front of its dynamic array, and a listed kernel missing from the
    assembly, are reported; one with an empty fixed segment is not."""
    meta = """
amdhsa.kernels:
  - .agpr_count:     0
    .group_segment_fixed_size: 0
    .name:           _Z5alphaILi1EEvv
    .vgpr_count:     100
  - .agpr_count:     0
    .group_segment_fixed_size: 144
    .name:           _Z4betaILi2EEvv
    .vgpr_count:     100
"""
    bad = check_isa.check_static_lds(meta, ("alpha", "beta", "gamma"))
    assert bad == [("_Z4betaILi2EEvv", 144), ("gamma", None)]
