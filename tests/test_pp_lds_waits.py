"""LDS waits of the hand-scheduled K block (gen_pp_phase.py: memory_phase, mx_memory_phase).

LDS answers a wavefront's reads in order, so `s_waitcnt lgkmcnt(n)` means "all but the last n reads have answered".  The
barrier that ends the memory phase must not be passed with a read of a weight slot outstanding: the weight slots (MXFP8:
with the weight rows' scale tiles behind them) are the one region that wavefronts of the other group refill.  Reads of
the group's own token slots and scale buffers may be out at that barrier and must all have answered before the first MFMA.
This test reads the generated statements and checks exactly that, and the counted waits of the matrix phase's rolling
token reads.  No GPU, no compiler.
"""
import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
WEIGHT_OPERANDS = ("%[wl]", "%[wh]", "%[sfwl]")     # fragment and scale reads that address a weight slot


def _gen():
    spec = importlib.util.spec_from_file_location("gen_pp_phase", os.path.join(ROOT, "expert_specialization_moe_amd", "csrc", "gen_pp_phase.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _statements():
    g = _gen()
    out = []
    for mtw in (4, 6):
        for fuse in (False, True):
            p = g.Plan(mtw, fuse)
            out.append((f"fp8 mtw={mtw} fuse={fuse}", g.memory_phase(p) + g.matrix_phase(p)))
            q = g.MxPlan(mtw, fuse)
            out.append((f"mx mtw={mtw} fuse={fuse}", g.mx_memory_phase(q) + g.mx_matrix_phase(q)))
    return out


def _written(line):
    """Vector registers an LDS read or an MFMA writes / an MFMA reads, as sets of register numbers."""
    def span(tok):
        m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.fullmatch(r"v(\d+)", tok)
        return {int(m.group(1))} if m else set()
    op, rest = line.split(None, 1)
    toks = [t.strip().split()[0] for t in rest.split(",")]
    return op, [span(t) for t in toks]


@pytest.mark.parametrize("name,lines", _statements(), ids=lambda v: v if isinstance(v, str) else "")
def test_barrier_waits_for_weight_slot_reads_and_mfmas_for_their_operands(name, lines):
    outstanding = []        # LDS reads in flight, oldest first: (line, registers written)
    barriers = 0
    for line in lines:
        if line.startswith("ds_read"):
            _, spans = _written(line)
            outstanding.append((line, spans[0]))
        elif line.startswith("s_waitcnt lgkmcnt("):
            n = int(line.split("(")[1].split(")")[0])
            assert n <= 15, f"{name}: lgkmcnt is a 4-bit counter"
            outstanding = outstanding[max(len(outstanding) - n, 0):] if n else []
        elif line == "s_barrier":
            barriers += 1
            left = [l for l, _ in outstanding if any(w in l for w in WEIGHT_OPERANDS)]
            assert not left, f"{name}: barrier {barriers} passed with weight-slot reads outstanding: {left}"
            if barriers == 2:
                assert not outstanding, f"{name}: the matrix phase ends with LDS reads outstanding"
        elif line.startswith("v_mfma"):
            _, spans = _written(line)
            used = set().union(*spans[1:])          # operands, accumulator / scale registers
            late = [l for l, regs in outstanding if regs & used]
            assert not late, f"{name}: {line.split(',')[0]} reads registers of reads that have not answered: {late}"
        elif line.startswith("v_mul_f32") or line.startswith("v_fmac_f32"):
            _, spans = _written(line)
            used = set().union(*spans)
            late = [l for l, regs in outstanding if regs & used]
            assert not late, f"{name}: {line} uses registers of reads that have not answered: {late}"
    assert barriers == 2


@pytest.mark.parametrize("name,lines", _statements(), ids=lambda v: v if isinstance(v, str) else "")
def test_reads_left_out_at_the_first_barrier_are_the_groups_own(name, lines):
    outstanding = []
    for line in lines:
        if line.startswith("ds_read"):
            outstanding.append(line)
        elif line.startswith("s_waitcnt lgkmcnt("):
            n = int(line.split("(")[1].split(")")[0])
            outstanding = outstanding[max(len(outstanding) - n, 0):] if n else []
        elif line == "s_barrier":
            own = ("%[al]", "%[ah]", "%[sal]", "%[sbl]", "%[sfa")
            assert outstanding, f"{name}: nothing is left out at the barrier (the wait in front of it is the old, full one)"
            assert all(any(o in l for o in own) for l in outstanding), f"{name}: {outstanding}"
            break


def test_every_statement_raises_the_priority_for_its_matrix_phase_only():
    """The generated header: one `s_setprio 3` right after the barrier that ends the memory phase (and the wait for the
    group's own reads), one `s_setprio 0` in front of the wait and barrier that end the matrix phase, so that the
    wavefront leaves every statement, and with it the K loop, at priority 0."""
    text = open(os.path.join(ROOT, "expert_specialization_moe_amd", "csrc", "pp_phase.h")).read()
    bodies = re.findall(r"#define (\w+_BODY\w*) \\\n((?:  \".*\n)+)", text)
    assert len(bodies) == 16
    for name, body in bodies:
        lines = [l.strip().strip("\\").strip().strip('"').replace("\\n\\t", "") for l in body.splitlines()]
        prio = [(i, l) for i, l in enumerate(lines) if l.startswith("s_setprio")]
        barriers = [i for i, l in enumerate(lines) if l == "s_barrier"]
        mfma = [i for i, l in enumerate(lines) if l.startswith("v_mfma")]
        assert [l for _, l in prio] == ["s_setprio 3", "s_setprio 0"], name
        assert len(barriers) == 2, name
        assert barriers[0] < prio[0][0] < mfma[0], name
        assert mfma[-1] < prio[1][0] < barriers[1], name


def test_committed_header_is_what_the_generator_writes():
    import subprocess
    import sys
    csrc = os.path.join(ROOT, "expert_specialization_moe_amd", "csrc")
    out = subprocess.run([sys.executable, os.path.join(csrc, "gen_pp_phase.py")], capture_output=True, text=True, check=True).stdout
    assert out == open(os.path.join(csrc, "pp_phase.h")).read(), "pp_phase.h is stale: python gen_pp_phase.py > pp_phase.h"
