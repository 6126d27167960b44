"""The GEMM's MFMAs and the int8 -> fp16 conversions are inline assembly, invisible to the compiler's hazard
recogniser: the compiled kernels must keep every read of an accumulator register far enough behind the last such
MFMA, and every conversion far enough ahead of the MFMA that reads it. Checked on the assembly hipcc produces
(no GPU needed)."""
import os
import sys
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "hexagon-mlir_amd"))
import check_mfma_hazards as chk  # noqa: E402


def _scan(tmp_path, text):
    p = tmp_path / "k.s"
    p.write_text(textwrap.dedent(text))
    return chk.scan(str(p))


def test_scanner_flags_an_early_accumulator_read(tmp_path):
    bad = _scan(tmp_path, """\
        _Zkernel:
        \t;;#ASMSTART
        \tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
        \t;;#ASMEND
        \ts_nop 3
        \tv_accvgpr_read_b32 v9, a2
        \ts_endpgm
        """)
    assert list(bad) == ["_Zkernel"] and bad["_Zkernel"][0][0] == 4


def test_scanner_accepts_spent_wait_states_builtin_mfmas_and_other_paths(tmp_path):
    bad = _scan(tmp_path, """\
        _Zkernel:
        \t;;#ASMSTART
        \tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
        \t;;#ASMEND
        \t;;#ASMSTART
        \ts_nop 15
        \ts_nop 15
        \t;;#ASMEND
        \tv_accvgpr_read_b32 v9, a2
        \tv_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]
        \tv_accvgpr_read_b32 v9, a2
        \t;;#ASMSTART
        \tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]
        \t;;#ASMEND
        \ts_branch .LBB0_1
        .LBB0_9:
        \tv_accvgpr_mov_b32 a1, a0
        """)
    assert bad == {}


def test_scanner_flags_a_hidden_write_one_slot_ahead_of_its_mfma(tmp_path):
    text = """\
        _Zkernel:
        \t;;#ASMSTART
        \tv_cvt_f16_i16_sdwa v41, sext(v8) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2
        \tv_cvt_f16_i16_sdwa v41, sext(v8) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3
        \t;;#ASMEND
        \ts_nop 0
        \tv_mfma_f32_16x16x32_f16 v[2:5], v[40:43], v[14:17], v[2:5]
        \ts_endpgm
        """
    p = tmp_path / "k.s"
    p.write_text(textwrap.dedent(text))
    bad = chk.scan_conversions(str(p))
    assert list(bad) == ["_Zkernel"] and bad["_Zkernel"][0][0] == 1       # the second conversion: one slot
    p.write_text(textwrap.dedent(text).replace("s_nop 0", "s_nop 1"))
    assert chk.scan_conversions(str(p)) == {}
    # another register is no reader
    p.write_text(textwrap.dedent(text).replace("v[40:43]", "v[44:47]"))
    assert chk.scan_conversions(str(p)) == {}
    # a write the compiler can see, read by an MFMA it can see: its own business
    p.write_text(textwrap.dedent(text).replace("\t;;#ASMSTART\n", "").replace("\t;;#ASMEND\n", ""))
    assert chk.scan_conversions(str(p)) == {}
    # a write the compiler can see, read by an assembly MFMA
    p.write_text(textwrap.dedent("""\
        _Zkernel:
        \tv_mov_b32_e32 v40, v9
        \t;;#ASMSTART
        \tv_mfma_f32_16x16x32_f16 a[0:3], v[40:43], v[14:17], a[0:3]
        \t;;#ASMEND
        \ts_endpgm
        """))
    assert chk.scan_conversions(str(p))["_Zkernel"][0][0] == 0


def test_scanner_flags_scratch_among_the_copies_of_a_kernel_with_counted_waits(tmp_path):
    p = tmp_path / "k.s"
    p.write_text(textwrap.dedent("""\
        _ZN5hexmi16w8a16_mid_kernelILi8ELi1EEEvPKh:
        \tscratch_store_dword off, v1, off
        \tglobal_load_lds_dwordx4 v[2:3], off
        \tscratch_load_dword v1, off, off
        \tglobal_load_lds_dwordx4 v[2:3], off nt
        \tscratch_load_dword v1, off, off
        \ts_endpgm
        _ZN5hexmi10row_kernelIfEEvPKf:
        \tglobal_load_lds_dwordx4 v[2:3], off
        \tscratch_load_dword v1, off, off
        \tglobal_load_lds_dwordx4 v[2:3], off
        \ts_endpgm
        """))
    assert chk.scan_scratch(str(p)) == {"_ZN5hexmi16w8a16_mid_kernelILi8ELi1EEEvPKh": [4]}


@pytest.mark.timeout(600)
def test_compiled_kernels_keep_their_distance():
    assert chk.main() == 0
