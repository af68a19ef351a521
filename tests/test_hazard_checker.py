"""The build-time checker of the inline-assembly MFMAs (csrc/check_pw_hazards.py) on small synthetic
assembly texts: each rule must fire on a violation and stay quiet on the repaired sequence."""
import importlib.util
import os

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location(
    "check_pw_hazards", os.path.join(HERE, "..", "megafold_amd", "csrc", "check_pw_hazards.py"))
chk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(chk)

HEAD = "_ZN2mf22evo_bwd_dqkv_pw_kernelIDF16bLi3EEEvNS_9EvoParamsEii:\n"


def run(tmp_path, body):
    f = tmp_path / "k.s"
    f.write_text(HEAD + body)
    return chk.check(str(f))


def asm(inst):
    return ";;#ASMSTART\n%s\n;;#ASMEND\n" % inst


MFMA_V = "v_mfma_f32_32x32x16_bf16 v[0:15], a[0:3], a[4:7], v[0:15]"
MFMA_A = "v_mfma_f32_32x32x16_bf16 a[16:31], a[0:3], v[20:23], a[16:31]"
MFMA_C = "v_mfma_f32_32x32x16_bf16 v[0:15], a[0:3], a[4:7], v[32:47]"


def test_operand_written_right_before_the_product(tmp_path):
    bad = "v_cvt_pk_bf16_f32 v20, v40, v41\n" + asm(MFMA_A)
    assert any("writes an operand" in e for e in run(tmp_path, bad))
    good = "v_cvt_pk_bf16_f32 v20, v40, v41\ns_nop 1\n" + asm(MFMA_A)
    assert run(tmp_path, good) == []


def test_c_operand_rewritten_while_the_product_runs(tmp_path):
    bad = asm(MFMA_C) + "v_mov_b32_e32 v33, v50\n" + "s_nop 15\n"
    assert any("rewrites the C operand" in e for e in run(tmp_path, bad))
    good = asm(MFMA_C) + "s_nop 12\nv_mov_b32_e32 v33, v50\n"
    assert run(tmp_path, good) == []


def test_vector_result_read_or_rewritten_too_early(tmp_path):
    early_read = asm(MFMA_V) + "v_mul_f32_e32 v60, v61, v3\n"
    assert any("reads the result" in e for e in run(tmp_path, early_read))
    early_write = asm(MFMA_V) + "s_nop 3\nv_accvgpr_read_b32 v15, a63\n"
    assert any("overwrites the result" in e for e in run(tmp_path, early_write))
    ok = asm(MFMA_V) + "s_nop 15\ns_nop 3\nv_accvgpr_read_b32 v15, a63\nv_mul_f32_e32 v60, v61, v15\n"
    assert run(tmp_path, ok) == []
    # a register rewritten late no longer holds the result: reading it afterwards is no finding
    late = asm(MFMA_V) + "s_nop 15\nv_mov_b32_e32 v3, v70\n" + "v_add_f32_e32 v71, v3, v3\n" * 2
    assert run(tmp_path, late) == []


def test_accumulation_register_result_read_by_other_units(tmp_path):
    bad = asm(MFMA_A) + "ds_write_b128 v90, a[16:19]\n"
    assert any("reads the result" in e for e in run(tmp_path, bad))
    good = asm(MFMA_A) + "s_nop 15\ns_nop 3\nds_write_b128 v90, a[16:19]\n"
    assert run(tmp_path, good) == []


def test_conditional_branch_both_continuations_are_followed(tmp_path):
    """A reader inside a conditionally skipped region is separated from the product by the region's own
    instructions; a reader behind the branch target is not (the branch may be taken)."""
    filler = "v_add_f32_e32 v80, v81, v82\n" * 10 + "s_nop 1\ns_nop 1\n"
    inside = asm(MFMA_V) + "s_cbranch_scc1 .LBB0_9\n" + filler + "v_mul_f32_e32 v60, v61, v3\n.LBB0_9:\ns_endpgm\n"
    assert run(tmp_path, inside) == []
    behind = asm(MFMA_V) + "s_cbranch_scc1 .LBB0_9\n" + filler + ".LBB0_9:\nv_mul_f32_e32 v60, v61, v3\ns_endpgm\n"
    assert any("reads the result" in e for e in run(tmp_path, behind))


def test_bias_gradient_ring_kernel_is_checked(tmp_path):
    f = tmp_path / "k.s"
    f.write_text("_ZN2mf25evo_bwd_dbias_ring_kernelIDF16bLi4EEEvNS_9EvoParamsEii:\n" + asm(MFMA_V) + "v_mul_f32_e32 v60, v61, v3\n")
    assert any("reads the result" in e for e in chk.check(str(f)))
