"""The build-time check for hand-written DPP instructions (rust-model-inference_amd/csrc/check_dpp_hazards.py)
flags what it is there to flag.  The compiler's hazard recogniser does not look into inline asm: a DPP operand read
within two wait states of the vector instruction that wrote it, or within five of a vector write of EXEC, returns
stale data on the GPU without any error, so the check must not pass such code."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CHECK = os.path.join(HERE, "..", "rust-model-inference_amd", "csrc", "check_dpp_hazards.py")

FMAC = "v_fmac_f32_dpp v10, v3, v7 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf"


def _run(tmp_path, body, *args):
    f = tmp_path / "k.s"
    f.write_text("\t.text\nkernel:\n" + "".join("\t%s\n" % line for line in body) + "\ts_endpgm\n")
    return subprocess.run([sys.executable, CHECK, str(f), *args], capture_output=True, text=True)


def test_clean_code_passes(tmp_path):
    r = _run(tmp_path, ["v_mul_f32_e32 v3, v1, v2", "v_add_u32_e32 v20, v21, v22", "v_cvt_f32_i32_e32 v7, v8", FMAC], "1")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "1 v_fmac_f32_dpp), 0 hazards" in r.stdout


def test_write_right_before_the_dpp_read_fails(tmp_path):
    r = _run(tmp_path, ["v_mul_f32_e32 v3, v1, v2", FMAC])
    assert r.returncode == 1 and "hazard: 0 wait state(s)" in r.stdout
    r = _run(tmp_path, ["v_mul_f32_e32 v3, v1, v2", "v_cvt_f32_i32_e32 v7, v8", FMAC])
    assert r.returncode == 1 and "hazard: 1 wait state(s)" in r.stdout
    r = _run(tmp_path, ["v_pk_mul_lo_u16 v[2:3], v[4:5], v[6:7]", FMAC])  # a register pair that holds the operand
    assert r.returncode == 1


def test_s_nop_counts_its_wait_states(tmp_path):
    assert _run(tmp_path, ["v_mul_f32_e32 v3, v1, v2", "s_nop 0", FMAC]).returncode == 1
    assert _run(tmp_path, ["v_mul_f32_e32 v3, v1, v2", "s_nop 1", FMAC]).returncode == 0


def test_other_registers_and_non_dpp_sources_do_not_matter(tmp_path):
    # v7 is the plain second factor and v10 the accumulator: neither goes through the DPP path
    assert _run(tmp_path, ["v_cvt_f32_i32_e32 v7, v8", FMAC]).returncode == 0
    assert _run(tmp_path, ["v_mul_f32_e32 v10, v1, v2", FMAC]).returncode == 0


def test_vector_write_of_exec_fails(tmp_path):
    r = _run(tmp_path, ["v_cmpx_lt_u32_e32 v1, v2", "s_nop 2", FMAC])
    assert r.returncode == 1
    assert _run(tmp_path, ["v_cmpx_lt_u32_e32 v1, v2", "s_nop 4", FMAC]).returncode == 0


def test_missing_instructions_fail(tmp_path):
    """The build names how many v_fmac_f32_dpp it expects: a compile that silently dropped them does not pass."""
    assert _run(tmp_path, ["v_mul_f32_e32 v3, v1, v2"], "1000").returncode == 1


def test_every_matching_function_must_hold_the_instruction(tmp_path):
    """With a regular expression instead of a count the functions that must hold a v_fmac_f32_dpp are the build's
    own instantiations: one of them without it, or no match at all, fails."""
    two = ["v_add_u32_e32 v20, v21, v22", "v_cvt_f32_i32_e32 v7, v8", FMAC, "s_endpgm", "kernel_b:", "v_add_u32_e32 v20, v21, v22"]
    r = _run(tmp_path, two, "kernel")
    assert r.returncode == 1 and "kernel_b" in r.stdout
    assert _run(tmp_path, two, "kernel$").returncode == 0  # only the first function is named
    assert _run(tmp_path, two + ["s_nop 1", FMAC], "kernel").returncode == 0
    assert _run(tmp_path, two, "no_such_function").returncode == 1


def test_hazard_across_a_branch_fails(tmp_path):
    """The write sits in front of a branch and the DPP read behind its target: text order alone would not see it."""
    body = ["v_mul_f32_e32 v3, v1, v2", "s_cbranch_scc1 .LBB0_2", "s_nop 7", "s_nop 7", "s_branch .LBB0_3",
            ".LBB0_2:", FMAC, ".LBB0_3:"]
    r = _run(tmp_path, body)
    assert r.returncode == 1 and "hazard: 1 wait state(s)" in r.stdout, r.stdout
    body[0:2] = ["v_mul_f32_e32 v3, v1, v2", "s_nop 0", "s_cbranch_scc1 .LBB0_2"]  # two wait states: enough
    assert _run(tmp_path, body).returncode == 0


def test_loop_back_edge_is_followed(tmp_path):
    body = [".LBB0_1:", FMAC, "v_add_u32_e32 v20, v21, v22", "v_mul_f32_e32 v3, v1, v2", "s_cbranch_vccnz .LBB0_1"]
    assert _run(tmp_path, body).returncode == 1
    body = [".LBB0_1:", FMAC, "v_mul_f32_e32 v3, v1, v2", "v_add_u32_e32 v20, v21, v22", "s_cbranch_vccnz .LBB0_1"]
    assert _run(tmp_path, body).returncode == 0


def test_indirect_jump_is_refused(tmp_path):
    assert _run(tmp_path, ["s_setpc_b64 s[30:31]"]).returncode == 1


def test_reading_a_matrix_core_result_too_early_fails(tmp_path):
    """An instruction (an asm statement's, for the compiler spaces its own) that reads a 4x4x4 matrix-core result
    sooner than five wait states after it; a matrix-core shape the script has no rule for is refused."""
    mfma = "v_mfma_f32_4x4x4_16b_f16 v[8:11], v[4:5], v[6:7], 0"
    use = "v_fmac_f32_dpp v20, v3, v9 row_ror:12 row_mask:0xf bank_mask:0xf"
    pad = "v_add_u32_e32 v30, v31, v32"
    assert _run(tmp_path, [mfma, pad, pad, use]).returncode == 1
    assert _run(tmp_path, [mfma, pad, pad, pad, pad, pad, use]).returncode == 0
    assert _run(tmp_path, [mfma, "s_nop 4", use]).returncode == 0
    assert _run(tmp_path, [mfma, "s_nop 3", use]).returncode == 1
    assert _run(tmp_path, [mfma, "v_mov_b32_e32 v9, v1", use]).returncode == 0  # v9 is another value by then
    assert _run(tmp_path, ["v_mfma_i32_32x32x32_i8 v[0:15], v[16:19], v[20:23], 0"]).returncode == 1
