"""The build-time check of inline-assembly MFMAs (fast_ops_amd/asm_lint.py) on small hand-written listings: it has to
flag the two hazards it exists for, and leave hazard-free code alone."""
from fast_ops_amd.asm_lint import lint_function

MFMA = "v_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]"


def _lint(text):
    return lint_function(text.strip().splitlines(), "k")


def test_valu_write_right_before_mfma_source_is_flagged():
    assert _lint(f"v_mov_b32_e32 v4, v9\n{MFMA}")                       # zero wait states
    assert _lint(f"v_mov_b32_e32 v1, v9\ns_nop 0\n{MFMA}")               # one wait state
    assert not _lint(f"v_mov_b32_e32 v1, v9\ns_nop 1\n{MFMA}")           # two: enough
    assert not _lint(f"v_mov_b32_e32 v1, v9\nv_add_f32 v20, v21, v22\nv_add_f32 v23, v21, v22\n{MFMA}")
    assert _lint(f"v_accvgpr_write_b32 a3, v9\n{MFMA}")                  # the accumulator is a source too
    assert not _lint(f"ds_read_b128 v[0:3], v30\ns_waitcnt lgkmcnt(0)\n{MFMA}")   # LDS data is not a VALU write
    assert not _lint(f"v_mov_b32_e32 v40, v9\n{MFMA}")                   # unrelated register


def test_mfma_right_after_a_label_is_flagged():
    assert _lint(f".LBB0_1:\n{MFMA}")
    assert not _lint(f".LBB0_1:\ns_nop 1\n{MFMA}")


def test_reading_an_mfma_result_too_early_is_flagged():
    assert _lint(f"{MFMA}\nv_accvgpr_read_b32 v50, a7")
    assert _lint(f"{MFMA}\ns_nop 7\nv_accvgpr_read_b32 v50, a7")         # 8 wait states: not yet
    assert not _lint(f"{MFMA}\ns_nop 7\ns_nop 7\nv_accvgpr_read_b32 v50, a7")
    # a dependent MFMA may follow at once; a reader after it waits for the second one
    second = "v_mfma_f32_32x32x16_bf16 a[0:15], v[8:11], v[4:7], a[0:15]"
    assert not _lint(f"{MFMA}\n{second}")
    assert _lint(f"{MFMA}\n{second}\ns_nop 7\nv_accvgpr_read_b32 v50, a0")
    # results in VGPRs are covered the same way
    to_v = "v_mfma_f32_32x32x16_f16 v[16:31], v[0:3], v[4:7], 0"
    assert _lint(f"{to_v}\nv_mul_f32_e32 v40, v41, v17")
    assert not _lint(f"{to_v}\ns_nop 7\ns_nop 7\nv_mul_f32_e32 v40, v41, v17")
