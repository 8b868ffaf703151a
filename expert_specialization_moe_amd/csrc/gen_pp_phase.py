"""Writes pp_phase.h: one K block of a tall fp8-blockwise tile as ONE inline-asm statement.

    python gen_pp_phase.py > pp_phase.h

The eight wavefronts of a tile form two groups of four (one wavefront of each group per SIMD); group 0 owns the upper
half of the tile's token rows, group 1 the lower half, and every wavefront owns 64 of the 256 weight rows.  The groups
run half a K block apart.  A K block of a wavefront is

    memory phase   copies of coming stages global -> LDS, weight fragments and the first two token fragments
                   LDS -> registers, the block's scales; waits for the weight fragments only
    s_barrier
    matrix phase   (at wave priority MATRIX_PRIO) waits for the token fragments and the scales, sa * sb;
                   MTW x 4 MFMAs; the fp32 promotion of MFMA j - 3 (four v_fmac) behind MFMA j; token fragment
                   mt + 2 read from LDS behind the first MFMA of row tile mt (three fragment buffers)
    s_barrier
    the last three promotions (in the shadow of the other group's first MFMAs)

and the statement also advances, behind its first three MFMAs (which have no promotions to issue yet), what changes from
one K block to the next of token slot, weight slot and copy sources (bookkeeping): between two statements those
instructions would delay the next memory phase's copies.

so while one group's wavefront keeps its SIMD's matrix pipe busy, the other group's wavefront on that SIMD moves data.
Written as a statement, not as C++ with scheduling fences: the compiler neither keeps such an order nor tracks the
asynchronous copies (its own waits would land in the loop), and every register that lives only inside the K block
(fragments, MFMA results, scales) is a fixed register named as a clobber, which leaves the compiler nothing to spill.

Ring (see gemm_tile_pp): weight stages in 3 slots shared by both groups, token stages in 2 slots per group (each
group copies and reads only its own token rows), activation scales in 3 chunk buffers of 4 K blocks per group.
Copies issued in the memory phase of K block kb, oldest first:  one 16-row piece of scale chunk kb/4 + 2,  the
group's token rows of K block kb + 1,  the wavefront's weight rows of K block kb + 2.  Waits (per wavefront, own copies):
    end of the memory phase   vmcnt(nT + 5): everything older than this phase's copies, i.e. weights kb + 1
    end of the matrix phase   vmcnt(4):      also the scale piece and the tokens of kb + 1; weights kb + 2 stay in flight
Every barrier certifies to the other wavefronts what the waits before it completed.

Hazards the assembler does not see (no hardware interlock between an MFMA's result and a vector-ALU read of it):
a promotion follows its MFMA by three MFMAs and twelve v_fmac (at least 15 issue slots, 11 needed); the tail
promotions follow the barrier; a fragment buffer is overwritten by a read that issues behind a later MFMA than
the last one that used it, and LDS data returns much later than an MFMA reads its operands; s_nop 0 separates
a write of m0 from the copy that uses it.
"""

NT = 4
MATRIX_PRIO = 3   # wave priority during the matrix phase (the memory phase runs at 0): where both wavefronts of a SIMD
                  # have an instruction ready, the one that feeds the matrix core goes first (one large expert,
                  # 12288 x 4096 x 7168: MXFP8 -1.7 %, FP8-blockwise -0.6 %; the memory phase first instead: +1.7 %, +0.3 %)


def with_prio(lines, level, before):
    """`lines` run at wave priority `level`, back to 0 in front of the first line that starts with `before`."""
    if not level:
        return lines
    i = next(k for k, l in enumerate(lines) if l.startswith(before))
    return [f"s_setprio {level}"] + lines[:i] + ["s_setprio 0"] + lines[i:]


def regs(lo, n):
    return f"v[{lo}:{lo + n - 1}]"


class Plan:
    def __init__(self, mtw, fuse):
        self.mtw, self.fuse = mtw, fuse
        # fixed registers, from the top of the file down
        self.w = [224 + 8 * n for n in range(4)]          # weight fragments
        self.a = [200, 208, 216]                          # token fragment buffers
        self.t = [184, 188, 192, 196]                     # MFMA results awaiting promotion
        self.sa = (184 - (mtw + 2)) // 2 * 2              # sa[0..mtw-1] (sa * sb after the memory phase), sb, sb_up
        self.sb = self.sa + mtw
        self.sbu = self.sb + 1
        self.scu = (self.sa - mtw) // 2 * 2 if fuse else None    # fused form: products sa * sb_up of the up half
        self.lowest = self.scu if fuse else self.sa
        self.ntc = mtw // 2                               # token copies per wavefront and K block

    def clobbers(self):
        return [f'"v{i}"' for i in range(self.lowest, 256)] + ['"memory"', '"m0"', '"scc"', '"vcc"']


def read_line(d, a, off):
    if a is None:
        return d          # a whole instruction
    return f"ds_read_b128 {d}, %[{a}]" + (f" offset:{off}" if off else "")


def scale_reads(p):
    L = [f"ds_read_b32 v{p.sa + mt}, %[sal]" + (f" offset:{mt * 256}" if mt else "") for mt in range(p.mtw)]
    L.append(f"ds_read_b32 v{p.sb}, %[sbl]")
    if p.fuse:
        L.append(f"ds_read_b32 v{p.sbu}, %[sbl] offset:1024")
    return L


def scale_products(p):
    L = []
    if p.fuse:
        L += [f"v_mul_f32 v{p.scu + mt}, v{p.sa + mt}, v{p.sbu}" for mt in range(p.mtw)]
    return L + [f"v_mul_f32 v{p.sa + mt}, v{p.sa + mt}, v{p.sb}" for mt in range(p.mtw)]


def memory_phase(p):
    L = []
    rd = []   # LDS reads to interleave with the copies: (dst, addr, offset)
    for n in range(4):
        rd.append((regs(p.w[n], 4), "wl", n * 2048))
        rd.append((regs(p.w[n] + 4, 4), "wh", n * 2048))
    for mt in range(2):
        rd.append((regs(p.a[mt], 4), "al", mt * 2048))
        rd.append((regs(p.a[mt] + 4, 4), "ah", mt * 2048))
    copies = [("s", None)] + [("t", i) for i in range(p.ntc)] + [("w", i) for i in range(4)]
    per = (len(rd) + len(copies) - 1) // len(copies)
    for kind, i in copies:
        if kind == "s":
            L += ["s_mov_b32 m0, %[ls]", "s_nop 0", "global_load_lds_dword %[vs], %[sp]"]
        elif kind == "t":
            if i == 0:
                L += ["s_mov_b32 m0, %[la]", "s_nop 0"]
            L.append(f"global_load_lds_dwordx4 %[va{i}], %[ap]" + (f" offset:{i * 1024}" if i else ""))
        else:
            if i == 0:
                L += ["s_mov_b32 m0, %[lw]", "s_nop 0"]
            L.append(f"global_load_lds_dwordx4 %[vw{i}], %[wp]" + (f" offset:{i * 1024}" if i else ""))
        for _ in range(per):
            if rd:
                L.append(read_line(*rd.pop(0)))
    L += [read_line(*r) for r in rd]
    sr = scale_reads(p)
    L += sr
    # LDS answers in order.  In front of the barrier a wavefront waits for its weight fragments only: the weight slots
    # are the one region that wavefronts of the other group refill, and they may do so once this barrier has passed
    # for the second time.  The token fragments and the scales come from the group's own slots and buffers, which
    # its own wavefronts refill after the barrier that ends the matrix phase, and every wavefront of the group has
    # waited for these reads before it gets there.  So the barrier is not kept waiting for them
    # (one large expert, 12288 x 4096 x 7168 FP8-blockwise: -3.4 %).
    L.append(f"s_waitcnt lgkmcnt({4 + len(sr)})")
    L.append(f"s_waitcnt vmcnt({p.ntc + 5}) ; explicit")
    L.append("s_barrier")
    L.append("s_waitcnt lgkmcnt(0)")
    L += scale_products(p)
    return L


def promotion(p, j):
    mt, nt = divmod(j, NT)
    sc = p.scu + mt if (p.fuse and nt >= NT // 2) else p.sa + mt
    return [f"v_fmac_f32 %[c{nt}_{mt}_{i}], v{p.t[j % 4] + i}, v{sc}" for i in range(4)]


def bookkeeping(p):
    """The part of the K loop's bookkeeping that this statement advances itself, behind its MFMAs (see mx_bookkeeping
    for the scheme and the reason): token slot, weight slot and the copies' source offsets.  What goes with the scale
    chunks (a four-K-block rhythm with an irregular last chunk) stays with the caller."""
    S = 256 * 128
    A = []
    A.append(["s_sub_u32 %[la], %[la], %[td]"])
    A.append([f"s_add_u32 %[lw], %[lw], {S}", "s_cmp_lg_u32 %[lw], %[lwend]", "s_cselect_b32 %[lw], %[lw], %[lwbase]"])
    A.append([f"s_add_u32 %[woff], %[woff], {S}", f"s_cmp_lg_u32 %[woff], {3 * S}", "s_cselect_b32 %[woff], %[woff], 0"])
    A.append(["v_add_u32 %[wl], %[woff], %[wfrag]", "v_xor_b32 %[wh], 64, %[wl]"])
    A.append(["s_cmp_ge_u32 %[rem], 2", "s_cselect_b32 vcc_lo, 128, 0"] + [f"v_add_u32 %[va{i}], vcc_lo, %[va{i}]" for i in range(p.ntc)])
    A.append(["s_cmp_ge_u32 %[rem], 3", "s_cselect_b32 vcc_lo, 128, 0"] + [f"v_add_u32 %[vw{i}], vcc_lo, %[vw{i}]" for i in range(4)]
             + ["s_sub_u32 %[rem], %[rem], 1"])
    late = [["v_add_u32 %[al], %[td], %[al]", "v_xor_b32 %[ah], 64, %[al]"], ["s_sub_u32 %[td], 0, %[td]"]]
    return A, late


def matrix_phase(p):
    L = []
    total = p.mtw * NT
    lag = 3
    atoms, late = bookkeeping(p)
    last_roll = (p.mtw - 3) * NT      # MFMA behind which the last rolling token read issues
    for j in range(total):
        mt, nt = divmod(j, NT)
        if nt == 0 and mt >= 2:
            L.append("s_waitcnt lgkmcnt(2)" if mt + 1 < p.mtw else "s_waitcnt lgkmcnt(0)")
        L.append(f"v_mfma_f32_16x16x128_f8f6f4 {regs(p.t[j % 4], 4)}, {regs(p.w[nt], 8)}, {regs(p.a[mt % 3], 8)}, 0")
        if nt == 0 and mt + 2 < p.mtw:
            b = p.a[(mt + 2) % 3]
            L.append(f"ds_read_b128 {regs(b, 4)}, %[al] offset:{(mt + 2) * 2048}")
            L.append(f"ds_read_b128 {regs(b + 4, 4)}, %[ah] offset:{(mt + 2) * 2048}")
        if j >= lag:
            L += promotion(p, j - lag)
        # bookkeeping behind the first three MFMAs, which have no promotions to issue yet (two groups each); the
        # token-slot group once the last rolling read has used al and ah
        if j < lag:
            for _ in range(2):
                if atoms:
                    L += atoms.pop(0)
        if j > last_roll and not atoms and late:
            L += late.pop(0)
    assert not atoms and not late, "more bookkeeping than MFMAs"
    L.append("s_waitcnt vmcnt(4) ; explicit")
    L.append("s_barrier")
    for j in range(total - lag, total):
        L += promotion(p, j)
    return L


def print_body(name, lines):
    """The statement, and its form for weight rows that no other tile reads (non-temporal hint on the weight copies)."""
    for suffix, hint in (("", ""), ("_NT", " nt")):
        print(f"#define {name}_BODY{suffix} \\")
        for i, l in enumerate(lines):
            last = i + 1 == len(lines)
            if l.startswith("global_load_lds_dwordx4 %[vw"):
                l += hint
            print('  "%s%s"%s' % (l, "" if last else "\\n\\t", "" if last else " \\"))


def emit(name, mtw, fuse):
    p = Plan(mtw, fuse)
    lines = memory_phase(p) + with_prio(matrix_phase(p), MATRIX_PRIO, "s_waitcnt vmcnt(4)")
    print_body(name, lines)
    outs = [f'[c{nt}_{mt}_{i}] "+v"(acc[{nt}][{mt}][{i}])' for mt in range(mtw) for nt in range(NT) for i in range(4)]
    outs += [f'[va{i}] "+v"(va[{i}])' for i in range(p.ntc)] + [f'[vw{i}] "+v"(vw[{i}])' for i in range(4)]
    outs += ['[wl] "+v"(wl)', '[wh] "+v"(wh)', '[al] "+v"(al)', '[ah] "+v"(ah)']
    outs += ['[la] "+s"(la)', '[lw] "+s"(lw)', '[td] "+s"(td)', '[woff] "+s"(woff)', '[rem] "+s"(rem)']
    print(f"#define {name}_OUTS " + ", ".join(outs))
    ins = ['[vs] "v"(vsq)', '[sal] "v"(sal)', '[sbl] "v"(sbl)', '[wfrag] "v"(wfrag)',
           '[ls] "s"(ls)', '[ap] "s"(a_ptr)', '[wp] "s"(w_ptr)', '[sp] "s"(sp)', '[lwbase] "s"(lwbase)', '[lwend] "s"(lwend)']
    print(f"#define {name}_INS " + ", ".join(ins))
    print(f"#define {name}_CLOBBERS " + ", ".join(p.clobbers()))
    print(f"#define {name}_LOWEST_FIXED_VGPR {p.lowest}")


# ---- mxfp8 form ----------------------------------------------------------------------------------------------------
# Same ring and phases with the hardware-scaled MFMA accumulating straight into the accumulators: no promotions, no
# result buffers, and the K loop's bookkeeping inside the statement (mx_bookkeeping).  The E8M0 scale bytes travel with the stages as verbatim 512-byte scale tiles (2 for the weight
# rows behind a weight stage, 2 for the group's token rows behind its token stage); every wavefront issues one
# 1 KB scale copy per K block so that the counted waits are the same for all (wavefront 0: weight scales of K block
# kb + 2, wavefronts 1 and 5: their group's token scales of kb + 1, the others re-read one line into a spare area).
# A lane reads, of the scale dword of its row, the byte of its K sub-block (lane / 16).
class MxPlan:
    def __init__(self, mtw, fuse=False):
        self.mtw = mtw
        self.fuse = fuse                    # gate_up weights: n-tiles 0, 1 are gate rows, 2, 3 the matching up rows
        self.w = [224 + 8 * n for n in range(4)]
        self.a = [200, 208, 216]
        self.sfw = 196                      # 4 weight-row scale registers
        self.sfa = 196 - mtw - (mtw % 2)    # mtw token-row scale registers
        self.lowest = self.sfa
        self.ntc = mtw // 2

    def clobbers(self):
        return [f'"v{i}"' for i in range(self.lowest, 256)] + ['"memory"', '"m0"', '"scc"', '"vcc"']


def mx_memory_phase(p):
    L, rd = [], []
    for n in range(4):
        rd.append((regs(p.w[n], 4), "wl", n * 2048))
        rd.append((regs(p.w[n] + 4, 4), "wh", n * 2048))
    # the scale bytes of the weight rows right behind the weight fragments: both live in the weight slot, the region that
    # has to be read in front of the barrier (memory_phase)
    for nt in range(4):
        # plain: n-tiles 2, 3 are the next 32-row quarter of the same scale tile; gate_up: the second tile (up rows)
        off = (nt & 1) * 256 + (nt >> 1) * (512 if p.fuse else 4)
        rd.append((f"ds_read_u8 v{p.sfw + nt}, %[sfwl]" + (f" offset:{off}" if off else ""), None, None))
    for mt in range(2):
        rd.append((regs(p.a[mt], 4), "al", mt * 2048))
        rd.append((regs(p.a[mt] + 4, 4), "ah", mt * 2048))
    copies = [("s", None)] + [("t", i) for i in range(p.ntc)] + [("w", i) for i in range(4)]
    per = (len(rd) + len(copies) - 1) // len(copies)
    for kind, i in copies:
        if kind == "s":
            L += ["s_mov_b32 m0, %[ls]", "s_nop 0", "global_load_lds_dwordx4 %[vs], %[sp]"]
        elif kind == "t":
            if i == 0:
                L += ["s_mov_b32 m0, %[la]", "s_nop 0"]
            L.append(f"global_load_lds_dwordx4 %[va{i}], %[ap]" + (f" offset:{i * 1024}" if i else ""))
        else:
            if i == 0:
                L += ["s_mov_b32 m0, %[lw]", "s_nop 0"]
            L.append(f"global_load_lds_dwordx4 %[vw{i}], %[wp]" + (f" offset:{i * 1024}" if i else ""))
        for _ in range(per):
            if rd:
                L.append(read_line(*rd.pop(0)))
    L += [read_line(*r) for r in rd]
    # a lane reads the one scale byte it feeds (its addresses point at byte lane / 16 of the row's scale dword): the
    # MFMA takes byte 0 of the register, and nothing stands between the LDS wait and the first MFMA
    for mt in range(p.mtw):
        L.append(f"ds_read_u8 v{p.sfa + mt}, %[sfa{mt}]")
    # the group's own token fragments and token scales (they live in its token slots) may still be out at the barrier
    L.append(f"s_waitcnt lgkmcnt({4 + p.mtw})")
    L.append(f"s_waitcnt vmcnt({p.ntc + 5}) ; explicit")
    L.append("s_barrier")
    L.append("s_waitcnt lgkmcnt(0)")
    return L


def mx_bookkeeping(p):
    """What changes from one K block to the next, advanced inside the statement: the lines sit behind the MFMAs of the
    matrix phase, where the wavefront has issue slots to spare, instead of between two statements, where they would
    delay the copies of the next memory phase (the critical path of a K block, the other group's MFMAs running beside
    it).  Every operand the memory phase uses is an in/out operand that holds the value for the coming K block:

        token slot (2-cycle)    %[td] = +-(bytes of a token slot): la -= td; al, sfa* += td; ah = al ^ 64; td = -td
        weight slot (3-cycle)   lw += S, back to %[lwbase] at %[lwend]; %[woff] in {0, S, 2S}: wl = wfrag + woff, wh = wl ^ 64,
                                sfwl = sfwrd + woff
        scale copy target       ls += %[lsinc], minus %[lswrap] at %[lsend] (the three roles differ in these constants only)
        copy sources            the lanes' byte offsets advance (the base pointers stay): by 128 (512 for the scale tiles)
                                while a later K block exists, counted down in %[rem] (K blocks after this one)

    Returns groups of lines; a group stays together (its s_cmp / s_cselect pair shares SCC with nothing else)."""
    S = 256 * 128 + 1024
    A = []
    A.append(["s_sub_u32 %[la], %[la], %[td]"])
    for mt in range(p.mtw):
        A.append([f"v_add_u32 %[sfa{mt}], %[td], %[sfa{mt}]"])
    A.append([f"s_add_u32 %[lw], %[lw], {S}", "s_cmp_lg_u32 %[lw], %[lwend]", "s_cselect_b32 %[lw], %[lw], %[lwbase]"])
    A.append([f"s_add_u32 %[woff], %[woff], {S}", f"s_cmp_lg_u32 %[woff], {3 * S}", "s_cselect_b32 %[woff], %[woff], 0"])
    A.append(["v_add_u32 %[wl], %[woff], %[wfrag]", "v_xor_b32 %[wh], 64, %[wl]", "v_add_u32 %[sfwl], %[woff], %[sfwrd]"])
    A.append(["s_add_u32 %[ls], %[ls], %[lsinc]", "s_cmp_ge_u32 %[ls], %[lsend]", "s_cselect_b32 vcc_lo, %[lswrap], 0",
              "s_sub_u32 %[ls], %[ls], vcc_lo"])
    A.append(["s_cmp_ge_u32 %[rem], 2", "s_cselect_b32 vcc_lo, 128, 0"] + [f"v_add_u32 %[va{i}], vcc_lo, %[va{i}]" for i in range(p.ntc)])
    A.append(["s_cmp_ge_u32 %[rem], 3", "s_cselect_b32 vcc_lo, 128, 0"] + [f"v_add_u32 %[vw{i}], vcc_lo, %[vw{i}]" for i in range(4)])
    A.append(["s_cmp_ge_u32 %[rem], %[sthr]", "s_cselect_b32 vcc_lo, 0x200, 0", "v_add_u32 %[vs], vcc_lo, %[vs]", "s_sub_u32 %[rem], %[rem], 1"])
    # after the last rolling token read (it still uses al, ah), and td's sign flips last
    late = [["v_add_u32 %[al], %[td], %[al]", "v_xor_b32 %[ah], 64, %[al]"], ["s_sub_u32 %[td], 0, %[td]"]]
    return A, late


def mx_matrix_phase(p):
    L = []
    atoms, late = mx_bookkeeping(p)
    total = p.mtw * NT
    last_roll = (p.mtw - 3) * NT      # MFMA behind which the last rolling token read issues
    for j in range(total):
        mt, nt = divmod(j, NT)
        if nt == 0 and mt >= 2:
            L.append("s_waitcnt lgkmcnt(2)" if mt + 1 < p.mtw else "s_waitcnt lgkmcnt(0)")
        L.append(f"v_mfma_scale_f32_16x16x128_f8f6f4 %[c{nt}_{mt}], {regs(p.w[nt], 8)}, {regs(p.a[mt % 3], 8)}, %[c{nt}_{mt}], "
                 f"v{p.sfw + nt}, v{p.sfa + mt} op_sel_hi:[0,0,0]")
        if nt == 0 and mt + 2 < p.mtw:
            b = p.a[(mt + 2) % 3]
            L.append(f"ds_read_b128 {regs(b, 4)}, %[al] offset:{(mt + 2) * 2048}")
            L.append(f"ds_read_b128 {regs(b + 4, 4)}, %[ah] offset:{(mt + 2) * 2048}")
        # one group of bookkeeping behind each of the first MFMAs; the token-slot group once al and ah are free
        if j >= 1 and atoms:
            L += atoms.pop(0)
        if j > last_roll and not atoms and late:
            L += late.pop(0)
    assert not atoms and not late, "more bookkeeping than MFMAs"
    L.append("s_waitcnt vmcnt(4) ; explicit")
    L.append("s_barrier")
    return L


def emit_mx(name, mtw, fuse=False):
    p = MxPlan(mtw, fuse)
    lines = mx_memory_phase(p) + with_prio(mx_matrix_phase(p), MATRIX_PRIO, "s_waitcnt vmcnt(4)")
    print_body(name, lines)
    outs = [f'[c{nt}_{mt}] "+v"(acc[{nt}][{mt}])' for mt in range(mtw) for nt in range(NT)]
    outs += [f'[va{i}] "+v"(va[{i}])' for i in range(p.ntc)] + [f'[vw{i}] "+v"(vw[{i}])' for i in range(4)]
    outs += ['[vs] "+v"(vs)', '[wl] "+v"(wl)', '[wh] "+v"(wh)', '[al] "+v"(al)', '[ah] "+v"(ah)', '[sfwl] "+v"(sfwl)']
    outs += [f'[sfa{mt}] "+v"(sfal[{mt}])' for mt in range(mtw)]
    outs += ['[la] "+s"(la)', '[lw] "+s"(lw)', '[ls] "+s"(ls)', '[td] "+s"(td)', '[woff] "+s"(woff)', '[rem] "+s"(rem)']
    print(f"#define {name}_OUTS " + ", ".join(outs))
    ins = ['[wfrag] "v"(wfrag)', '[sfwrd] "v"(sfw_rd)', '[ap] "s"(a_ptr)', '[wp] "s"(w_ptr)', '[sp] "s"(s_ptr)',
           '[lwbase] "s"(lwbase)', '[lwend] "s"(lwend)', '[lsinc] "s"(lsinc)', '[lsend] "s"(lsend)', '[lswrap] "s"(lswrap)',
           '[sthr] "s"(sthr)']
    print(f"#define {name}_INS " + ", ".join(ins))
    print(f"#define {name}_CLOBBERS " + ", ".join(p.clobbers()))
    print(f"#define {name}_LOWEST_FIXED_VGPR {p.lowest}")


def main():
    print("// Generated by gen_pp_phase.py; do not edit.")
    print("#pragma once")
    for mtw in (4, 6):
        emit(f"ESMOE_PP{mtw * 2}", mtw, False)
        emit(f"ESMOE_PP{mtw * 2}F", mtw, True)
        emit_mx(f"ESMOE_PPX{mtw * 2}", mtw)
        emit_mx(f"ESMOE_PPX{mtw * 2}F", mtw, True)


if __name__ == "__main__":
    main()
