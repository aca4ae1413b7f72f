"""The check of the generated code around inline-asm MFMAs (wmma_extension_amd/isa_check.py).

A vector-ALU write of a register directly in front of an MFMA that reads it is a hazard the
hardware does not interlock (one-wave probe on gfx950, wmmae_mfma_source_hazard_probe, run by
tests/test_gpu_primitives.py: `v_mov_b32` or `v_accvgpr_read_b32` into a source register, then
the MFMA: the MFMA multiplies the old contents, every time; with `s_nop 0` or any instruction
in between, the new ones).  The compiler spaces its own MFMAs,
but it does not look into asm statements, and its register allocator may reload a fragment
register from an AGPR copy right at the statement.  Snippets below are shaped like the compiler's
output."""
import os

import pytest

from wmma_extension_amd import _lib, isa_check

ASM_MFMA = """
	;;#ASMSTART
	v_mfma_f32_16x16x32_bf16 a[0:3], v[6:9], v[0:3], a[0:3]
	;;#ASMEND
"""


def _kinds(text):
    return [f["kind"] for f in isa_check.scan(text)]


def test_reload_in_front_of_an_asm_mfma_is_found():
    text = "\tv_accvgpr_read_b32 v8, a248\n\tv_accvgpr_read_b32 v9, a249\n" + ASM_MFMA
    found = isa_check.scan(text)
    assert [f["kind"] for f in found] == ["valu-write-before-asm-mfma"] * 2
    assert sorted(f["wait_states"] for f in found) == [0, 1]
    assert "v_accvgpr_read_b32 v9, a249" in isa_check.format_findings(found)
    # the accumulator counts as a source too (zeroed right before its first product)
    assert _kinds("\tv_accvgpr_write_b32 a2, 0\n" + ASM_MFMA) == ["valu-write-before-asm-mfma"]
    # a wide move into the B fragment
    assert _kinds("\tv_mov_b64_e32 v[2:3], v[20:21]\n" + ASM_MFMA) == ["valu-write-before-asm-mfma"]


def test_two_wait_states_or_other_registers_are_clean():
    assert _kinds("\tv_accvgpr_read_b32 v9, a249\n\ts_nop 1\n" + ASM_MFMA) == []
    assert _kinds("\tv_accvgpr_read_b32 v9, a249\n\tds_read_b128 v[20:23], v2\n\ts_add_u32 s1, s1, 4\n"
                  + ASM_MFMA) == []
    assert _kinds("\tv_accvgpr_read_b32 v10, a249\n" + ASM_MFMA) == []        # v10 is not read
    assert _kinds("\tds_read_b128 v[6:9], v2\n\ts_waitcnt lgkmcnt(0)\n" + ASM_MFMA) == []   # LDS data: a counter
    # an MFMA in front of an MFMA on the same accumulator is what the matrix core chains
    assert _kinds(ASM_MFMA + ASM_MFMA) == []
    # the compiler's own MFMAs are its own business
    assert _kinds("\tv_accvgpr_read_b32 v9, a249\n\tv_mfma_f32_16x16x32_bf16 a[0:3], v[6:9], v[0:3], a[0:3]\n") == []


def test_result_touched_before_the_matrix_core_has_written_it():
    assert _kinds(ASM_MFMA + "\tv_accvgpr_read_b32 v40, a3\n") == ["asm-mfma-result-touched-early"]
    assert _kinds(ASM_MFMA + "\tv_accvgpr_write_b32 a0, 0\n") == ["asm-mfma-result-touched-early"]
    # what the kernels do before their epilogue
    assert _kinds(ASM_MFMA + "\ts_nop 15\n\ts_nop 15\n\tv_accvgpr_read_b32 v40, a3\n") == []
    # other accumulators and the operands may be touched at once
    assert _kinds(ASM_MFMA + "\tv_accvgpr_read_b32 v40, a7\n\tds_read_b128 v[6:9], v2\n") == []


def test_check_file_raises_with_the_place(tmp_path):
    bad = tmp_path / "bad.s"
    bad.write_text("\tv_accvgpr_read_b32 v9, a249\n" + ASM_MFMA)
    with pytest.raises(RuntimeError) as e:
        isa_check.check_file(str(bad))
    assert "line 4" in str(e.value) and "line 1: v_accvgpr_read_b32 v9" in str(e.value)
    good = tmp_path / "good.s"
    good.write_text("\ts_nop 1\n" + ASM_MFMA)
    assert isa_check.check_file(str(good)) == 0


def test_built_library_is_clean():
    """The assembly build() kept of the GEMM translation unit (absent when the library was
    built elsewhere: then build() made this check there)."""
    for name in _lib.ASM_MFMA_SOURCES:
        path = _lib.device_asm_path(name)
        if not os.path.exists(path):
            pytest.skip("no device assembly beside the library")
        with open(path) as f:
            text = f.read()
        assert text.count("v_mfma") > 1000
        assert isa_check.scan(text) == []
