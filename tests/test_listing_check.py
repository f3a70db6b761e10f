"""The build's check of the assembly listings: reads of an MFMA result that sit too close behind the MFMA are found,
along straight code and across branches, and idle states or enough MFMAs in between clear them."""
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))
import __graft_entry__ as ge  # noqa: E402

ge._package()
from triton_tenstorrent_amd import listing_check as lc  # noqa: E402

MFMA = "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[30:33], v[62:65], a[0:15]"
OTHER = "\tv_mfma_f32_32x32x16_bf16 a[16:31], v[22:25], v[62:65], a[16:31]"


def kernel(*body):
    return ["k:", *body, "\ts_endpgm", ".Lfunc_end0:"]


def test_a_copy_directly_behind_the_mfma_is_found():
    h = lc.mfma_result_hazards(kernel(MFMA, "\ts_nop 0", "\tv_accvgpr_read_b32 v177, a15"))
    assert len(h) == 1 and "v_accvgpr_read_b32 v177, a15" in h[0]


def test_idle_states_inside_the_statement_clear_it():
    assert lc.mfma_result_hazards(kernel(MFMA, "\ts_nop 7", "\ts_nop 2", "\tv_accvgpr_read_b32 v177, a15")) == []
    assert len(lc.mfma_result_hazards(kernel(MFMA, "\ts_nop 7", "\ts_nop 1", "\tv_accvgpr_read_b32 v177, a15"))) == 1


def test_one_mfma_in_between_is_not_enough_two_are():
    assert len(lc.mfma_result_hazards(kernel(MFMA, OTHER, "\tv_accvgpr_read_b32 v1, a3"))) == 1
    assert lc.mfma_result_hazards(kernel(MFMA, OTHER, OTHER.replace("16:31", "32:47"), "\tv_accvgpr_read_b32 v1, a3")) == []


def test_other_registers_and_the_addend_of_a_later_mfma_are_fine():
    assert lc.mfma_result_hazards(kernel(MFMA, "\tv_accvgpr_read_b32 v1, a16", "\tv_add_f32_e32 v2, v30, v62")) == []
    assert lc.mfma_result_hazards(kernel(MFMA, MFMA)) == []
    # as a multiplicand the result is a read like any other
    assert len(lc.mfma_result_hazards(kernel("\tv_mfma_f32_32x32x16_bf16 v[0:15], v[30:33], v[62:65], v[0:15]",
                                             "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[62:65], a[0:15]"))) == 1


def test_both_sides_of_a_branch_are_followed():
    body = [MFMA, "\ts_cbranch_vccz .LBB0_2", "\tv_mov_b32_e32 v1, v2", "\ts_branch .LBB0_3", ".LBB0_2:",
            "\tv_accvgpr_mov_b32 a128, a0", ".LBB0_3:", "\tv_accvgpr_read_b32 v9, a1"]
    h = lc.mfma_result_hazards(kernel(*body))
    assert any("v_accvgpr_mov_b32 a128, a0" in m for m in h) and any("v_accvgpr_read_b32 v9, a1" in m for m in h)


def test_the_window_follows_the_passes_of_the_form():
    short = "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[30:33], v[62:65], a[0:3]"
    assert lc.passes("v_mfma_f32_16x16x32_bf16") == 4 and lc.passes("v_mfma_f32_32x32x64_f8f6f4") == 16
    assert lc.mfma_result_hazards(kernel(short, "\ts_nop 6", "\tv_accvgpr_read_b32 v1, a0")) == []
    assert len(lc.mfma_result_hazards(kernel(short, "\ts_nop 5", "\tv_accvgpr_read_b32 v1, a0"))) == 1


def test_kernels_of_a_listing_are_checked_one_by_one():
    text = "\n".join(kernel(MFMA, "\tv_accvgpr_read_b32 v1, a0") + ["clean:", MFMA, "\ts_endpgm", ".Lfunc_end1:"])
    assert list(lc.check_listing(text)) == ["k"]


def test_compiler_waits_for_memory_inside_an_mfma_loop_are_counted():
    loop = [".LBB0_1:"] + [MFMA] * 32
    asm_wait = ["\t;;#ASMSTART", "\ts_waitcnt vmcnt(16) lgkmcnt(0)", "\t;;#ASMEND"]
    assert lc.vmcnt_waits_in_mfma_blocks(kernel(*loop, *asm_wait)) == 0
    assert lc.vmcnt_waits_in_mfma_blocks(kernel(*loop, *asm_wait, "\ts_waitcnt vmcnt(0)")) == 1
    # outside the loops (a block with few MFMAs) the compiler may wait as it likes
    assert lc.vmcnt_waits_in_mfma_blocks(kernel(*loop, ".LBB0_2:", MFMA, "\ts_waitcnt vmcnt(0)")) == 0


def test_a_register_file_copy_right_in_front_of_the_mfma_that_reads_it_is_found():
    mfma = "\tv_mfma_f32_32x32x16_bf16 v[2:17], v[34:37], a[132:135], v[2:17]"
    mf = ["\t;;#ASMSTART", mfma, "\t;;#ASMEND"]
    padded = ["\t;;#ASMSTART", "\ts_nop 1", mfma, "\t;;#ASMEND"]
    assert len(lc.valu_writes_in_front_of_an_mfma(kernel("\tv_accvgpr_read_b32 v37, a191", *mf))) == 1
    assert len(lc.valu_writes_in_front_of_an_mfma(kernel("\tv_accvgpr_write_b32 a133, v9", "\ts_nop 0", *mf))) == 1
    assert lc.valu_writes_in_front_of_an_mfma(kernel("\tv_accvgpr_read_b32 v37, a191", *padded)) == []
    # other registers, an operand that comes from LDS, another block, the compiler's own MFMA
    assert lc.valu_writes_in_front_of_an_mfma(kernel("\tv_accvgpr_read_b32 v38, a191", *mf)) == []
    assert len(lc.valu_writes_in_front_of_an_mfma(kernel("\tv_cvt_pk_bf16_f32 v37, v1, v2", *mf))) == 1
    assert lc.valu_writes_in_front_of_an_mfma(kernel("\tds_read_b128 v[34:37], v5", "\ts_waitcnt lgkmcnt(0)", *mf)) == []
    assert lc.valu_writes_in_front_of_an_mfma(kernel("\tv_accvgpr_read_b32 v37, a191", ".LBB0_1:", *mf)) == []
    assert lc.valu_writes_in_front_of_an_mfma(kernel("\tv_accvgpr_read_b32 v37, a191", mfma)) == []
    assert list(lc.check_listing("\n".join(kernel("\tv_accvgpr_read_b32 v37, a191", *mf)))) == ["k"]


def test_the_build_reads_the_listing_of_its_own_compilation(monkeypatch, tmp_path):
    """build_code_object hands hipcc -save-temps, checks the listing that lands beside it and refuses the code object
    when the check finds something (the compiler stands in here: it writes a listing and an object)."""
    from triton_tenstorrent_amd import build as b

    def compiler(body):
        def run(cmd, cwd=None):
            assert "-save-temps" in cmd and cwd is not None
            out = Path(cmd[cmd.index("-o") + 1])
            out.write_bytes(b"\x7fELF")
            Path(cwd, f"probe-hip-amdgcn-amd-amdhsa-{b.ARCH}.s").write_text("\n".join(kernel(*body)))
        return run

    monkeypatch.setattr(b, "BUILD", tmp_path)
    monkeypatch.setattr(b, "hipcc", lambda: "hipcc")
    monkeypatch.setattr(b, "_run", compiler([MFMA, "\ts_nop 7", "\ts_nop 2", "\tv_accvgpr_read_b32 v177, a15"]))
    assert b.build_code_object("probe") == tmp_path / "probe.hsaco" and (tmp_path / "probe.hsaco").exists()
    monkeypatch.setattr(b, "_run", compiler([MFMA, "\tv_accvgpr_read_b32 v177, a15"]))
    try:
        b.build_code_object("probe")
    except RuntimeError as e:
        assert "touched too early" in str(e) and "k:" in str(e)
    else:
        raise AssertionError("a listing with a read right behind an MFMA passed the build")
    assert not (tmp_path / "probe.hsaco").exists()
