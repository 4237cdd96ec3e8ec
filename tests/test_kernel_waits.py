"""The static check of MFMA wait states (flashbias_amd/csrc/check_mfma_waits.py): on hand-made instruction
sequences, and on the compiled code of the two units in which the compiler's own count fell short before
(the window backward, whose first version read a score block across a loop branch after two slots, and the
general dq kernel, where a short-circuit condition gave the block after the last MFMA two ways out)."""
import importlib.util
import os
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "flashbias_amd", "csrc")
spec = importlib.util.spec_from_file_location("check_mfma_waits", os.path.join(CSRC, "check_mfma_waits.py"))
waits = importlib.util.module_from_spec(spec)
spec.loader.exec_module(waits)

MFMA = "v_mfma_f32_32x32x16_bf16 v[0:15], v[16:19], v[20:23], v[0:15]"
OTHER = "v_mfma_f32_32x32x16_bf16 v[32:47], v[16:19], v[20:23], v[32:47]"


def early(*lines):
    return waits.check("kernel:\n" + "\n".join(lines) + "\ns_endpgm\n")


def test_straight_line():
    assert early(MFMA, "s_nop 10", "v_mul_f32_e32 v60, v0, v61")            # 11 slots: one short
    assert not early(MFMA, "s_nop 11", "v_mul_f32_e32 v60, v0, v61")
    assert not early(MFMA, "s_nop 4", "v_mul_f32_e32 v60, v61, v62", "s_nop 5", "v_mul_f32_e32 v60, v15, v61")
    assert early(MFMA, "s_nop 7", "ds_write_b64 v50, v[14:15]")             # LDS and memory instructions count too
    assert early(MFMA, "s_nop 7", "v_mov_b32_e32 v3, 0")                    # and so does overwriting a result register


def test_the_matrix_pipe_takes_one_instruction_at_a_time():
    # a second, independent MFMA leaves the first one's eight passes behind it before it issues
    assert not early(MFMA, OTHER, "s_nop 2", "v_mul_f32_e32 v60, v0, v61")
    # ... but its own result is as young as before
    assert early(MFMA, OTHER, "s_nop 2", "v_mul_f32_e32 v60, v32, v61")
    # accumulating into the same registers is the hardware's business, reading them as A or B is not
    assert not early(MFMA, MFMA)
    assert early(MFMA, "v_mfma_f32_32x32x16_bf16 v[32:47], v[0:3], v[20:23], v[32:47]")


def test_every_path_counts():
    # the branch skips four scalar instructions: twelve slots along the fall-through path, eight along the other
    lines = [MFMA, "s_cbranch_vccnz .LBB0_1", "s_add_i32 s0, s1, 31", "s_cmp_gt_i32 s0, s2", "s_cselect_b64 s[4:5], -1, 0",
             "s_and_b64 s[4:5], s[6:7], s[4:5]", ".LBB0_1:", "s_nop 5", "v_mul_f32_e32 v60, v0, v61"]
    found = early(*lines)
    assert found and found[0][3] == 7
    lines[7] = "s_nop 10"
    assert not early(*lines)
    # a loop whose body starts with the reader and ends with the MFMA
    assert early(".LBB0_2:", "v_mul_f32_e32 v60, v0, v61", "s_nop 11", MFMA, "s_cbranch_scc1 .LBB0_2")
    assert not early(".LBB0_2:", "v_mul_f32_e32 v60, v0, v61", "s_nop 11", MFMA, "s_nop 10", "s_cbranch_scc1 .LBB0_2")


@pytest.mark.skipif(shutil.which("hipcc") is None or shutil.which("make") is None, reason="needs hipcc and make")
def test_compiled_kernels():
    units = ["build/asm/fb_bwd_win_bf16_2.s", "build/asm/fb_bwd_dq_bf16_2.s"]
    subprocess.run(["make", "-j2"] + units, cwd=CSRC, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    for unit in units:
        with open(os.path.join(CSRC, unit)) as f:
            text = f.read()
        assert text.count("v_mfma_f32_32x32x16") > 100, unit
        assert waits.check(text) == [], unit
