"""Scalar-register hazards around the asm blocks of the kernels (no GPU needed: hipcc cross-compiles).

A memory instruction or an MFMA inside an asm block is invisible to the compiler's hazard pass, so
the assembly of every kernel source is checked for (1) a vector-memory instruction reading a scalar
register that a vector-ALU instruction wrote fewer than 5 slots earlier, (2) a global->LDS copy
reading M0 right after the scalar instruction that wrote it, (3) an MFMA result touched fewer than 11
slots after the MFMA, (4) an MFMA operand written by the vector ALU fewer than 2 slots before and
(5) a dot-product result read by another vector-ALU opcode fewer than 3 slots later (or overwritten
by one fewer than 4 slots later).
The checker itself is pinned on hand-written listings."""
import isa_lint

HAZ_VMEM = """
	v_readfirstlane_b32 s17, v210
	v_readfirstlane_b32 s16, v211
	;;#ASMSTART
	global_load_dwordx4 v[152:155], v212, s[16:17]
	;;#ASMEND
"""
OK_NOPS = HAZ_VMEM.replace(";;#ASMSTART", "s_nop 4\n\t;;#ASMSTART")
SHORT_NOPS = HAZ_VMEM.replace(";;#ASMSTART", "s_nop 2\n\t;;#ASMSTART")
OK_SALU = HAZ_VMEM.replace(";;#ASMSTART", "s_mov_b64 s[16:17], s[16:17]\n\t;;#ASMSTART")
OK_OTHER_REG = HAZ_VMEM.replace("s[16:17]", "s[18:19]")
HAZ_CMP = """
	v_cmp_lt_u32_e64 s[4:5], v1, v2
	v_mov_b32_e32 v3, 0
	buffer_load_dword v4, v5, s[4:7], 0 offen
"""
HAZ_M0 = """
	s_add_i32 m0, s38, 0x2000
	global_load_lds_dwordx4 v191, s[26:27]
"""
OK_M0 = HAZ_M0.replace("\tglobal_load_lds", "\ts_nop 0\n\tglobal_load_lds")
OK_M0_PLAIN_LOAD = HAZ_M0.replace("global_load_lds_dwordx4 v191", "global_load_dwordx4 v[0:3], v191")


MFMA = "\tv_mfma_f32_32x32x16_f16 v[32:47], v[6:9], v[116:119], v[32:47]\n"
MFMA_READ_EARLY = MFMA + "\tv_add_f32_e32 v1, v2, v3\n" * 9 + "\tv_exp_f32_e32 v0, v33\n"
MFMA_READ_OK = MFMA + "\tv_add_f32_e32 v1, v2, v3\n" * 11 + "\tv_exp_f32_e32 v0, v33\n"
MFMA_READ_NOPS = MFMA + "\ts_nop 7\n\ts_nop 2\n\tv_exp_f32_e32 v0, v33\n"
MFMA_CHAIN_OK = MFMA + "\tv_mfma_f32_32x32x16_f16 v[32:47], v[10:13], v[120:123], v[32:47]\n"
MFMA_AS_OPERAND = MFMA + "\tv_mfma_f32_32x32x16_f16 v[48:63], v[32:35], v[120:123], v[48:63]\n"
VALU_THEN_MFMA = "\tv_cvt_pkrtz_f16_f32 v6, v1, v2\n" + MFMA
VALU_THEN_MFMA_OK = "\tv_cvt_pkrtz_f16_f32 v6, v1, v2\n\ts_nop 1\n" + MFMA


def test_checker_on_matrix_core_listings():
    assert len(isa_lint.lint(MFMA_READ_EARLY)) == 1
    assert isa_lint.lint(MFMA_READ_OK) == []
    assert isa_lint.lint(MFMA_READ_NOPS) == []
    assert isa_lint.lint(MFMA_CHAIN_OK) == []
    assert len(isa_lint.lint(MFMA_AS_OPERAND)) == 1
    assert len(isa_lint.lint(VALU_THEN_MFMA)) == 1
    assert isa_lint.lint(VALU_THEN_MFMA_OK) == []


def test_checker_on_transcendental_results():
    assert len(isa_lint.lint("\tv_exp_f32_e32 v1, v2\n\tv_mul_f32_e32 v3, v1, v4\n")) == 1
    assert isa_lint.lint("\tv_exp_f32_e32 v1, v2\n\tv_exp_f32_e32 v3, v1\n") == []
    assert isa_lint.lint("\tv_exp_f32_e32 v1, v2\n\tv_mul_f32_e32 v1, v5, v4\n") == []
    assert isa_lint.lint("\tv_exp_f32_e32 v1, v2\n\ts_nop 0\n\tv_mul_f32_e32 v3, v1, v4\n") == []


def test_checker_on_dot_product_results():
    dot = "\tv_dot2_f32_f16 v80, v24, s36, 0\n"
    acc = "\tv_dot2_f32_f16 v80, v25, s36, v80\n"
    # the same opcode accumulating into its own result is forwarded
    assert isa_lint.lint(dot + acc) == []
    # another opcode reading the sum: three idle slots needed
    assert len(isa_lint.lint(dot + acc + "\tv_cmp_nge_f32_e32 vcc, s37, v80\n")) == 1
    assert len(isa_lint.lint(dot + acc + "\ts_nop 1\n\tv_cmp_nge_f32_e32 vcc, s37, v80\n")) == 1
    assert isa_lint.lint(dot + acc + "\ts_nop 2\n\tv_cmp_nge_f32_e32 vcc, s37, v80\n") == []
    # the two-operand form accumulating into the result of the three-operand form is another opcode
    assert len(isa_lint.lint(dot + "\tv_dot2c_f32_f16_e32 v80, s36, v25\n")) == 1
    assert isa_lint.lint("\tv_dot2c_f32_f16_e32 v80, s36, v24\n\tv_dot2c_f32_f16_e32 v80, s36, v25\n") == []
    # the same opcode taking the sum as a multiplicand
    assert len(isa_lint.lint(dot + "\tv_dot2_f32_f16 v81, v80, s36, 0\n")) == 1
    # overwritten by another opcode within four slots
    assert len(isa_lint.lint(dot + "\tv_add_f32_e32 v1, v2, v3\n" * 3 + "\tv_mov_b32_e32 v80, 0\n")) == 1
    assert isa_lint.lint(dot + "\tv_add_f32_e32 v1, v2, v3\n" * 4 + "\tv_mov_b32_e32 v80, 0\n") == []


def test_checker_on_hand_written_listings():
    assert len(isa_lint.lint(HAZ_VMEM)) == 1
    assert len(isa_lint.lint(SHORT_NOPS)) == 1
    assert isa_lint.lint(OK_NOPS) == []
    assert isa_lint.lint(OK_SALU) == []
    assert isa_lint.lint(OK_OTHER_REG) == []
    assert len(isa_lint.lint(HAZ_CMP)) == 1
    assert len(isa_lint.lint(HAZ_M0)) == 1
    assert isa_lint.lint(OK_M0) == []
    assert isa_lint.lint(OK_M0_PLAIN_LOAD) == []


def test_kernel_sources_have_no_scalar_register_hazards():
    report = isa_lint.analyse_sources()
    assert set(report) == set(isa_lint._build.SOURCES)
    assert {s: h for s, (h, _) in report.items() if h} == {}
    # the hand-scheduled kernels keep everything in registers: a reload would make the compiler wait for
    # every memory operation in flight, the stage copies included, in the middle of the schedule
    for src in ("fta_fwd1.hip", "fta_fwd2.hip", "fta_bwd_dq1.hip", "fta_bwd_dkdv1.hip"):
        spilling = dict(report[src][1])
        if src == "fta_fwd2.hip":
            # known: the tail-masking instances of the two-slab D=64 forward (template arguments <T, 2, true>)
            # keep five bias registers of a row's last tile in scratch (three reloads per row)
            spilling = {k: v for k, v in spilling.items() if "Li2ELb1E" not in k}
        if src == "fta_bwd_dkdv1.hip":
            # known: the D=64 instances for 384 queries per launch (template arguments <T, 64, 12, 4, ...>) use
            # every vector and accumulation register and keep one loop-invariant pair in scratch (one
            # reload per row; three accesses per kernel); still 2.5x the general kernel's rate at that length
            assert all(v <= 3 for k, v in spilling.items() if "Li64ELi12ELi4E" in k)
            spilling = {k: v for k, v in spilling.items() if "Li64ELi12ELi4E" not in k}
        assert spilling == {}, f"{src}: kernels that spill registers"


def test_checker_counts_the_scratch_accesses_of_a_kernel():
    listing = ("_Zspills:\n\tscratch_store_dword off, v51, off offset:4\n\tv_mov_b32 v1, v2\n\tscratch_load_dword v88, off, off offset:4\n"
               "\t.end_amdhsa_kernel\n_Zclean:\n\tv_mov_b32 v1, v2\n\t.end_amdhsa_kernel\n")
    assert isa_lint.scratch_ops(listing) == {"_Zspills": 2}


def test_checker_on_wide_store_data():
    bad = "global_store_dwordx4 v131, v[34:37], s[10:11]\nv_mul_f32_e32 v34, v8, v38\n"
    late = "global_store_dwordx4 v131, v[34:37], s[10:11]\ns_nop 1\nv_mul_f32_e32 v34, v8, v38\n"
    other = "global_store_dwordx4 v131, v[34:37], s[10:11]\nv_mul_f32_e32 v40, v8, v38\nv_mul_f32_e32 v131, v8, v38\n"
    narrow = "global_store_dwordx2 v131, v[34:35], s[10:11]\nv_mul_f32_e32 v34, v8, v38\n"
    assert len(isa_lint.lint(bad)) == 1
    assert isa_lint.lint(late) == [] and isa_lint.lint(other) == [] and isa_lint.lint(narrow) == []
