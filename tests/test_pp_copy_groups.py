"""Copy groups of the hand-scheduled K block (gen_pp_phase.py) and of the C++ copy helpers (grouped_gemm.hip).

A global -> LDS copy adds its immediate offset to the LDS address (m0) AND to the global address.  The operand copies
come in groups that share one write of m0 and use offsets 0, 1024, 2048, 3072; their per-lane source offsets carry
`kBias - i * 1024` and their base pointers point kBias bytes in front of the tensor, so that offset and bias cancel.
A scale copy has neither: its base pointer is the tensor's and its lanes' offsets are plain.  Put into a group with
an immediate offset it would read up to 3 KB beside the bytes it is meant to read (in front of the scale tensor for a
group that starts at its first K block).  So: every scale copy writes m0 itself and carries no offset, every copy with
an offset reads through a biased base, and the offsets of a group are i * 1024 below the bias.  No GPU, no compiler.
"""
import os
import re

import pytest

from tests.test_pp_lds_waits import _statements

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIASED = {"%[ap]": "%[la]", "%[wp]": "%[lw]"}     # base operand -> the LDS operand its group writes to m0
PLAIN = {"%[sp]": "%[ls]"}
K_BIAS = 3072


@pytest.mark.parametrize("name,lines", _statements(), ids=lambda v: v if isinstance(v, str) else "")
def test_scale_copies_never_share_an_offset_group_with_operand_copies(name, lines):
    m0, in_group, copies = None, 0, 0
    for line in lines:
        if line.startswith("s_mov_b32 m0,"):
            m0, in_group = line.split(",")[1].strip(), 0
            continue
        if not line.startswith("global_load_lds"):
            continue
        copies += 1
        m = re.fullmatch(r"global_load_lds_dword(x4)? (%\[\w+\]), (%\[\w+\])(?: offset:(\d+))?", line)
        assert m, line
        base, off = m.group(3), int(m.group(4) or 0)
        if base in PLAIN:
            assert m0 == PLAIN[base] and in_group == 0 and off == 0, f"{name}: scale copy inside an offset group: {line}"
        else:
            assert base in BIASED and m0 == BIASED[base], f"{name}: {line} under m0 = {m0}"
            assert off == in_group * 1024 and off <= K_BIAS, f"{name}: {line} is copy {in_group} of its group"
        in_group += 1
    assert copies >= 6


def test_cxx_copy_helpers_keep_the_same_rule():
    """grouped_gemm.hip: the grouped helper (dma16xn, immediate offsets) is only ever called with a pointer that has
    kBias taken off, the single-copy helpers (dma16, dma4: no offset) only with plain pointers; kBias covers the
    largest immediate offset."""
    src = open(os.path.join(ROOT, "expert_specialization_moe_amd", "csrc", "grouped_gemm.hip")).read()
    assert set(re.findall(r"constexpr int kBias = (\d+);", src)) == {str(K_BIAS)}
    offsets = [int(v) for v in re.findall(r"ESMOE_DMAO\(\d, (\d+),", src)]
    assert offsets and max(offsets) == K_BIAS
    biased = set(re.findall(r"const uint8_t\* (\w+) = [^;]*- kBias;", src))
    assert {"a_ptr", "w_ptr"} <= biased
    grouped = re.findall(r"dma16xn<\w+>\([^,]+, (\w+)", src)
    assert grouped and all(p in biased for p in grouped), grouped
    for call in re.findall(r"\bdma(?:16|4)\(([^;]*);", src):
        ptr = call.split(",")[0].strip()
        if ptr.startswith("const void*"):
            continue   # the helpers' own definitions
        assert not any(re.search(rf"\b{b}\b", ptr) for b in biased), f"plain copy through a biased pointer: dma({call}"
