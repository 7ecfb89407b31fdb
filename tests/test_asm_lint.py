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


def test_lds_dma_right_after_an_m0_write_is_flagged():
    from fast_ops_amd.asm_lint import lint_m0_function

    lint = lambda text: lint_m0_function(text.strip().splitlines(), "k")
    dma = "global_load_lds_dwordx4 v2, s[6:7]"
    assert lint(f"s_mov_b32 m0, s5\n{dma}")                              # no wait state
    assert lint(f"s_add_u32 m0, s5, 0x400\n{dma}")                       # any scalar write of M0 counts
    assert lint(f"s_mov_b32 m0, s5\n.LBB0_3:\n{dma}")                    # a label in between changes nothing
    assert lint("s_mov_b32 m0, s5\nbuffer_load_dword v1, s[8:11], 0 offen lds")
    assert not lint(f"s_mov_b32 m0, s5\ns_nop 0\n{dma}")                 # one wait state: enough
    assert not lint(f"s_mov_b32 m0, s5\nv_add_u32_e32 v2, v2, v3\n{dma}")
    assert not lint(f"s_mov_b32 s4, s5\n{dma}")                          # not M0
    assert not lint("s_mov_b32 m0, s5\nbuffer_load_dword v1, s[8:11], 0 offen")   # not an LDS-DMA
    assert not lint("s_mov_b32 m0, s5\nds_read_b128 v[0:3], v30")
