"""The scanner of the kernels' assembly (`make -C nanovllm-voxcpm_amd/csrc check`) on hand-written
snippets: it reports an MFMA whose result is read too soon behind a branch and nothing else."""

import importlib.util
import pathlib

ROOT = pathlib.Path(__file__).resolve().parents[1]


def _scanner():
    spec = importlib.util.spec_from_file_location("check_mfma_reads", ROOT / "nanovllm-voxcpm_amd" / "csrc" / "check_mfma_reads.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


HEAD = "_Z6kernelv:\n"
RUN = (
    "\tv_mfma_f32_16x16x32_bf16 v[46:49], v[74:77], v[98:101], v[46:49]\n"
    "\ts_cbranch_vccnz .LBB0_2\n"
    "\tds_read_b128 v[74:77], v172 offset:8896\n"
    "\ts_waitcnt lgkmcnt(0)\n"
    "\tv_mfma_f32_16x16x32_bf16 v[42:45], v[74:77], v[98:101], v[42:45]\n"
)


def _count(tmp_path, text):
    f = tmp_path / "k.s"
    f.write_text(text)
    return _scanner().scan(str(f))


def test_result_read_two_instructions_behind_the_branch_is_reported(tmp_path, capsys):
    join = ".LBB0_2:\n\ts_nop 0\n\tv_mov_b64_e32 v[100:101], v[48:49]\n\ts_endpgm\n"
    assert _count(tmp_path, HEAD + RUN + join) == 1
    assert "read after 2 wait states" in capsys.readouterr().out


def test_a_store_of_the_result_counts_as_a_read(tmp_path):
    join = ".LBB0_2:\n\tglobal_store_dwordx4 v[40:41], v[46:49], off\n\ts_endpgm\n"
    assert _count(tmp_path, HEAD + RUN + join) == 1


def test_idle_cycles_at_the_join_clear_it(tmp_path):
    join = ".LBB0_2:\n\ts_nop 7\n\ts_nop 7\n\tv_mov_b64_e32 v[100:101], v[48:49]\n\ts_endpgm\n"
    assert _count(tmp_path, HEAD + RUN + join) == 0


def test_other_registers_and_later_mfmas_are_not_reported(tmp_path):
    join = ".LBB0_2:\n\tv_mov_b64_e32 v[100:101], v[50:51]\n\tv_mfma_f32_16x16x32_bf16 v[46:49], v[74:77], v[98:101], v[46:49]\n\ts_endpgm\n"
    assert _count(tmp_path, HEAD + RUN + join) == 0


def test_a_branch_a_few_instructions_behind_the_mfma_is_followed(tmp_path):
    run = (
        "\tv_mfma_f32_16x16x32_bf16 v[46:49], v[74:77], v[98:101], v[46:49]\n"
        "\ts_and_b64 vcc, exec, s[0:1]\n"
        "\tv_add_u32_e32 v1, v2, v3\n"
        "\ts_cbranch_vccnz .LBB0_2\n"
        "\ts_endpgm\n"
    )
    join = ".LBB0_2:\n\tds_write_b128 v144, v[46:49] offset:64\n\ts_endpgm\n"
    assert _count(tmp_path, HEAD + run + join) == 1


def test_a_wait_instruction_behind_the_branch_is_not_taken_for_a_delay(tmp_path):
    """A wait that finds its counter at zero returns at once: the read behind it is as early as
    without it."""
    join = ".LBB0_2:\n\ts_waitcnt vmcnt(0)\n\tv_mov_b64_e32 v[100:101], v[48:49]\n\ts_endpgm\n"
    assert _count(tmp_path, HEAD + RUN + join) == 1


def test_the_distance_asked_for_follows_from_the_variant(tmp_path):
    """Seven wait states behind the branch are too few for a 16x16 variant (never less than eight
    are asked for); a 32x32 variant (8 passes + 3) asks for eleven, an unknown one for the most."""
    sc = _scanner()
    assert sc.need_of("v_mfma_f32_16x16x32_bf16") == 8 and sc.need_of("v_mfma_f32_16x16x16_bf16") == 8
    assert sc.need_of("v_mfma_f32_32x32x16_bf16") == 11 and sc.need_of("v_mfma_f32_unknown") == sc.NEED_MAX
    for nops, found in ((5, 1), (6, 0)):  # the branch itself is one state
        join = f".LBB0_2:\n\ts_nop {nops}\n\tv_mov_b64_e32 v[100:101], v[48:49]\n\ts_endpgm\n"
        assert _count(tmp_path, HEAD + RUN + join) == found, nops
