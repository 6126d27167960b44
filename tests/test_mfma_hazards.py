"""The GEMM's MFMAs are inline assembly, invisible to the compiler's hazard recogniser: the compiled kernels must keep
every read of an accumulator register far enough behind the last of them. Checked on the assembly hipcc produces
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


@pytest.mark.timeout(600)
def test_compiled_gemm_kernels_keep_their_distance():
    assert chk.main() == 0
