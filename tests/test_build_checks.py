"""The build's check of the hand-issued matrix instructions (moba_amd/asm_check.py): the checker itself on
small assembly texts, and the generated code of the dK/dV kernel when hipcc is at hand.  CPU only."""

import os

import pytest

from moba_amd import asm_check, build

_FN = """
_ZN4moba14bwd_dkv_kernelINS_4Bf16EEEvNS_9BwdParamsIT_EE:
\ts_load_dword s0, s[4:5], 0x0
\tv_mfma_f32_32x32x16_bf16 v[0:15], a[0:3], a[4:7], 0
\tv_mfma_f32_32x32x16_bf16 v[0:15], a[8:11], a[12:15], v[0:15]
%s
\ts_endpgm
.Lfunc_end0:
"""


def _asm(body):
    return _FN % "\n".join("\t" + l for l in body)


def test_checker_counts_instructions_to_the_first_use():
    body = ["v_add_f32_e32 v40, v41, v42"] * 5 + ["v_fma_f32 v50, s0, v3, -v51"]
    dist, count, where = asm_check.min_result_distance(_asm(body), "bwd_dkv_kernelINS_4Bf16")
    assert (dist, count) == (5, 2) and "v_fma_f32" in where


def test_checker_follows_branches_and_counts_nops():
    # the fall-through path is long, the taken branch reaches a write of v7 after two instructions
    body = ["s_cbranch_scc1 .LBB0_2"] + ["v_mov_b32_e32 v60, v61"] * 30 + [".LBB0_2:", "v_mov_b32_e32 v7, 0"]
    body = [l if l.endswith(":") else l for l in body]
    text = _FN % "\n".join(l if l.endswith(":") else "\t" + l for l in body)
    assert asm_check.min_result_distance(text, "bwd_dkv_kernelINS_4Bf16")[0] == 1
    body = ["s_nop 15", "v_mov_b32_e32 v7, 0"]
    assert asm_check.min_result_distance(_asm(body), "bwd_dkv_kernelINS_4Bf16")[0] == 16


def test_checker_rejects_an_early_use():
    text = _asm(["v_exp_f32_e32 v20, v2"]) + (_FN % "\tv_exp_f32_e32 v20, v2").replace("4Bf16", "3F16")
    with pytest.raises(RuntimeError, match="touched 0 instructions later"):
        asm_check.check_dkv_kernel(text)


@pytest.mark.skipif(not os.path.exists(build.HIPCC), reason="needs hipcc")
def test_generated_dkv_kernel_keeps_its_distance():
    asm = asm_check.device_assembly(build.HIPCC, build.FLAGS, os.path.join(build.CSRC, "bwd.hip"))
    symbols = asm_check.dkv_kernel_symbols(asm)
    assert len(symbols) == 4        # two element types x (plain, batched) layouts
    for sym in symbols:
        dist, count, where = asm_check.min_result_distance(asm, sym)
        assert count == 80          # 2 chains x 8 steps in each of the five places phase A is instantiated
        assert dist >= asm_check.MIN_DISTANCE, where
