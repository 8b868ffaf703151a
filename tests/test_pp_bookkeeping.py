"""The K-loop bookkeeping that the hand-scheduled K block advances itself (gen_pp_phase.py: bookkeeping, mx_bookkeeping).

The statement of a tall tile keeps, as in/out operands, every address that changes from one K block to the next (ring
slots, LDS read addresses, the copies' source offsets) and advances them with a few scalar and vector instructions
behind its MFMAs.  This test interprets exactly those generated instructions on plain integers, K block after K block,
and compares every operand with the closed form that the ring design prescribes (token stage kb in slot kb % 2,
weight stage kb in slot kb % 3, copies fetching token stage kb + 1 and weight stage kb + 2, clamped at the last K block).
No GPU, no compiler.
"""
import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
M32 = 0xFFFFFFFF


def _gen():
    spec = importlib.util.spec_from_file_location("gen_pp_phase", os.path.join(ROOT, "expert_specialization_moe_amd", "csrc", "gen_pp_phase.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _run(lines, env):
    """Interpret the bookkeeping instructions on env (operand name -> 32-bit value); 'scc' and 'vcc_lo' live in env too."""
    def val(tok):
        tok = tok.strip()
        m = re.fullmatch(r"%\[(\w+)\]", tok)
        if m:
            return env[m.group(1)]
        if tok == "vcc_lo":
            return env["vcc_lo"]
        return int(tok, 0) & M32

    def dst(tok):
        tok = tok.strip()
        m = re.fullmatch(r"%\[(\w+)\]", tok)
        return m.group(1) if m else tok

    for line in lines:
        op, rest = line.split(None, 1)
        a = [t.strip() for t in rest.split(",")]
        if op in ("s_add_u32", "v_add_u32"):
            env[dst(a[0])] = (val(a[1]) + val(a[2])) & M32
        elif op == "s_sub_u32":
            env[dst(a[0])] = (val(a[1]) - val(a[2])) & M32
        elif op == "v_xor_b32":
            env[dst(a[0])] = val(a[1]) ^ val(a[2])
        elif op == "s_cmp_lg_u32":
            env["scc"] = int(val(a[0]) != val(a[1]))
        elif op == "s_cmp_ge_u32":
            env["scc"] = int(val(a[0]) >= val(a[1]))
        elif op == "s_cselect_b32":
            env[dst(a[0])] = val(a[1]) if env["scc"] else val(a[2])
        else:
            raise AssertionError("instruction the test does not know: " + line)


@pytest.mark.parametrize("mx", [False, True])
@pytest.mark.parametrize("mtw", [4, 6])
@pytest.mark.parametrize("kb_count", [1, 2, 3, 4, 5, 7, 12, 56, 57])
def test_statement_advances_its_operands_as_the_ring_prescribes(mx, mtw, kb_count):
    gen = _gen()
    plan = gen.MxPlan(mtw) if mx else gen.Plan(mtw, False)
    atoms, late = (gen.mx_bookkeeping if mx else gen.bookkeeping)(plan)
    lines = [l for group in atoms + late for l in group]
    kW = 256 * 128 + (1024 if mx else 0)           # bytes of a weight slot (mxfp8: plus its scale tiles)
    kT = mtw * 16 * 128 + (1024 if mx else 0)      # bytes of a group's token slot
    t_dst, w_dst, afrag, wfrag, sfw_rd = 0x19000, 0x40, 0x19a30, 0x2a0, 0x8010
    for role in ((0, 1, 2) if mx else (None,)):
        s_dst = {0: 0x8000, 1: 0x1c000, 2: 0x27000, None: 0}[role]
        kbt0, kbw0 = min(1, kb_count - 1), min(2, kb_count - 1)
        env = {"la": t_dst + kT, "td": kT, "lw": w_dst + 2 * kW, "woff": 0, "lwbase": w_dst, "lwend": w_dst + 3 * kW,
               "rem": kb_count - 1, "wl": wfrag, "wh": wfrag ^ 64, "al": afrag, "ah": afrag ^ 64, "wfrag": wfrag, "scc": 0, "vcc_lo": 0}
        for i in range(plan.ntc):
            env[f"va{i}"] = 1000 * i + kbt0 * 128
        for i in range(4):
            env[f"vw{i}"] = 77 * i + kbw0 * 128
        if mx:
            env.update({"ls": s_dst + (2 * kW if role == 0 else kT if role == 1 else 0),
                        "lsinc": kW if role == 0 else kT if role == 1 else 0,
                        "lsend": s_dst + 3 * kW if role == 0 else s_dst + 2 * kT if role == 1 else M32,
                        "lswrap": 3 * kW if role == 0 else 2 * kT if role == 1 else 0,
                        "sthr": 3 if role == 0 else 2, "vs": 5 + (kbw0 if role == 0 else kbt0) * 512,
                        "sfwl": sfw_rd, "sfwrd": sfw_rd})
            for mt in range(mtw):
                env[f"sfa{mt}"] = 0x30000 + 16 * mt
        for kb in range(kb_count):
            tslot, wslot = kb % 2, kb % 3
            kbt, kbw = min(kb + 1, kb_count - 1), min(kb + 2, kb_count - 1)
            assert env["la"] == t_dst + (tslot ^ 1) * kT and env["lw"] == w_dst + ((kb + 2) % 3) * kW
            assert env["al"] == afrag + tslot * kT and env["ah"] == env["al"] ^ 64
            assert env["wl"] == wfrag + wslot * kW and env["wh"] == env["wl"] ^ 64
            assert all(env[f"va{i}"] == 1000 * i + kbt * 128 for i in range(plan.ntc))
            assert all(env[f"vw{i}"] == 77 * i + kbw * 128 for i in range(4))
            if mx:
                want_ls = s_dst + (((kb + 2) % 3) * kW if role == 0 else (tslot ^ 1) * kT if role == 1 else 0)
                assert env["ls"] == want_ls and env["vs"] == 5 + (kbw if role == 0 else kbt) * 512
                assert env["sfwl"] == sfw_rd + wslot * kW
                assert all(env[f"sfa{mt}"] == 0x30000 + 16 * mt + tslot * kT for mt in range(mtw))
            _run(lines, env)


def test_bookkeeping_sits_behind_mfmas_and_token_addresses_move_last():
    """The token fragment addresses are still read by the rolling fragment reads of the matrix phase: they may only
    move behind the last of those reads, and the sign of the token-slot step flips after its last use."""
    gen = _gen()
    for plan, phase in ((gen.Plan(6, False), gen.matrix_phase), (gen.Plan(4, False), gen.matrix_phase),
                        (gen.MxPlan(6), gen.mx_matrix_phase), (gen.MxPlan(4), gen.mx_matrix_phase)):
        lines = phase(plan)
        last_roll = max(i for i, l in enumerate(lines) if l.startswith("ds_read_b128") and ("%[al]" in l or "%[ah]" in l))
        move_al = next(i for i, l in enumerate(lines) if l.startswith("v_add_u32 %[al]"))
        flip = next(i for i, l in enumerate(lines) if l.startswith("s_sub_u32 %[td], 0"))
        uses_td = [i for i, l in enumerate(lines) if "%[td]" in l]
        first_mfma = next(i for i, l in enumerate(lines) if l.startswith("v_mfma"))
        assert move_al > last_roll and flip == max(uses_td)
        assert all(i > first_mfma for i, l in enumerate(lines) if re.match(r"[sv]_(add|sub|xor|cmp|cselect)", l))
