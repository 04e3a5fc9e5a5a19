"""Every kernel that uses the matrix cores is compiled to gfx950 assembly (hipcc cross-compiles without
a GPU) and scanned for readers of a matrix instruction's result that sit in another basic block closer
than the instruction's latency (tests/isa_hazards.py says why the compiler does not pad those). One such
reader existed in the streaming kernel's masked path at head dim 256 - the fourth register of a score
tile was read 3 wait states after the last matrix instruction - and showed as keys 3, 7, 11 of a partial
16-key unit taking slightly wrong weights at some page sizes; `mfma_settle` (common.hpp) closes it."""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

import isa_hazards

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "espetero_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"
SOURCES = ["attn_stream.hip", "attn_tiled.hip", "attn_tiled512.hip", "head_gate.hip"]


def test_scanner_flags_a_reader_behind_a_branch_and_not_a_padded_one():
    bad = """
_Z1kv:
	v_mfma_f32_16x16x32_f16 a[64:67], v[0:3], v[4:7], a[64:67]
	s_cbranch_vccz .LBB0_2
	s_mov_b64 s[0:1], 0
.LBB0_2:
	s_mov_b64 s[2:3], -1
	v_accvgpr_read_b32 v69, a67
	s_endpgm
"""
    (name, lines), = isa_hazards.kernels(bad)
    v = isa_hazards.violations(lines)
    assert len(v) == 1 and v[0][4] < 7
    good = bad.replace("	s_cbranch_vccz .LBB0_2\n", "	s_nop 7\n	s_cbranch_vccz .LBB0_2\n")
    (name, lines), = isa_hazards.kernels(good)
    assert isa_hazards.violations(lines) == []
    same_block = bad.replace("	s_cbranch_vccz .LBB0_2\n", "").replace(".LBB0_2:\n", "")
    (name, lines), = isa_hazards.kernels(same_block)
    assert isa_hazards.violations(lines) == []          # in one block the compiler pads; not this check's business


def _product_flags():
    """The flags the library is built with (csrc/Makefile's HIPFLAGS): the scan is of the code that ships."""
    text = open(os.path.join(CSRC, "Makefile")).read().replace("\\\n", " ")
    line = next(l for l in text.splitlines() if l.startswith("HIPFLAGS"))
    flags = line.split("=", 1)[1].replace("$(ARCH)", "gfx950").split()
    assert "-amdgpu-mfma-vgpr-form=1" in flags and "--offload-arch=gfx950" in flags, flags
    return [f for f in flags if f != "-fPIC"]


def _assembly(src, out_dir):
    out = os.path.join(out_dir, src.replace(".hip", ".s"))
    subprocess.run([HIPCC, *_product_flags(), "-S", "--cuda-device-only", "-o", out, os.path.join(CSRC, src)],
                   check=True, capture_output=True)
    return open(out).read()


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_no_matrix_result_is_read_across_a_block_boundary_too_early(tmp_path):
    with ThreadPoolExecutor(len(SOURCES)) as pool:
        texts = list(pool.map(lambda s: _assembly(s, str(tmp_path)), SOURCES))
    n_kernels, n_mfma, bad = 0, 0, []
    for src, text in zip(SOURCES, texts):
        for name, lines in isa_hazards.kernels(text):
            n_kernels += 1
            n_mfma += sum(1 for l in lines if l[0] == "ins" and l[1].startswith("v_mfma"))
            bad += [(src, name[:80]) + v for v in isa_hazards.violations(lines)]
    assert n_kernels >= 30 and n_mfma > 2000          # the listing really was parsed
    assert not bad, bad[:5]
