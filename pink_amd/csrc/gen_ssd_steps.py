#!/usr/bin/env python3
"""Writes ssd_steps.inc: the chunk loop of the float32 distance kernel for small problems.

    python gen_ssd_steps.py > ssd_steps.inc
"""

# Registers of the lone-wave loop (all of them clobbers of its one asm statement).
BV = 32            # v[32:95]   the lane's 64 rotation values of the chunk being computed (from LDS)
DT = 96            # v[96:103]  eight differences in flight
ST = (104, 120)    # v[104:119], v[120:135]  rotation vectors of the chunks c + 1 and c + 2 on their way to LDS
NV = 136           # v[136:151] the neuron's chunks c .. c + 3, four registers each
S_RP, S_NP, S_CNT = 40, 42, 44      # s[40:41] rotation rows, s[42:43] neuron row, s44 chunks left
STAGE = 64 * 68 * 4                 # bytes of one LDS stage: 64 rows of 64 + 4 floats
ROWS16 = 16 * 68 * 4                # bytes between a thread's four staging vectors (16 rows)


def lone_wave_loop():
    """The whole chunk loop of the kernel for small problems (one neuron per wave, about one wave per SIMD) as
    ONE asm statement.  A lone wave issues an instruction of any kind about every eight clocks, so the loop is
    written down to the instruction: per 64-element chunk 64 DPP subtracts, 64 multiply-adds, 16 LDS reads,
    4 LDS writes, 5 global loads, 5 waits, a barrier and a compare-and-branch.  It is assembly as a whole
    because its loads run three and four chunks ahead with counted waits: the compiler neither keeps such
    loads where they are written nor knows, for loads issued by assembly, that a register is still being
    written -- inside one statement with fixed registers there is nothing for it to move, copy or reuse.

    Element e of a chunk of the neuron sits in register e % 4 of lane e / 4 of every row of 16 lanes (one
    16-byte load per lane) and reaches all lanes of the row as the DPP operand of the subtract; every
    (neuron, rotation) sum is one lane's multiply-add chain in element order.  No DPP source is written by
    the vector ALU (the loads write them), so no idle slots are needed before the subtracts.

    Loads issued per chunk c: four rotation vectors of chunk c + 3, then the neuron vector of chunk c + 4
    (the prologue issues the same sequence).  Behind the neuron vector of chunk c come 15 loads before chunk
    c needs it (11 in the prologue behind that of chunk 0; the first four of the 15 are rotation vectors that
    chunk c - 1 has already waited for, so the one wait for "at most 11 outstanding" serves both), behind the
    rotation vectors of chunk c + 1 come 6 before chunk c stores them to LDS.  The last chunk issues nothing;
    the loads of the three chunks before it read past the end of the rows."""
    A = []
    def vr(base, n=4):
        return "v[%d:%d]" % (base, base + n - 1)
    def gload(dst, voff, sbase, imm):
        A.append("global_load_dwordx4 %s, %s, s[%d:%d]%s" % (vr(dst), voff, sbase, sbase + 1, " offset:%d" % imm if imm else ""))
    A.append("s_mov_b64 s[%d:%d], %%[rp]" % (S_RP, S_RP + 1))
    A.append("s_mov_b64 s[%d:%d], %%[np]" % (S_NP, S_NP + 1))
    A.append("s_mov_b32 s%d, %%[cnt]" % S_CNT)
    for i in range(4):
        gload(BV + 4 * i, "%%[roff%d]" % i, S_RP, 0)              # chunk 0 of the rotations, through the chunk registers
    gload(NV + 0, "%[noff]", S_NP, 0)
    gload(NV + 4, "%[noff]", S_NP, 256)
    for i in range(4):
        gload(ST[0] + 4 * i, "%%[roff%d]" % i, S_RP, 256)
    gload(NV + 8, "%[noff]", S_NP, 512)
    for i in range(4):
        gload(ST[1] + 4 * i, "%%[roff%d]" % i, S_RP, 512)
    gload(NV + 12, "%[noff]", S_NP, 768)
    A.append("s_waitcnt vmcnt(12)")
    for i in range(4):
        A.append("ds_write_b128 %%[ldsw], %s%s" % (vr(BV + 4 * i), " offset:%d" % (i * ROWS16) if i else ""))
    A.append("s_waitcnt lgkmcnt(0)")
    A.append("s_barrier")
    A.append("0:")
    for u in range(4):
        rd, wr = (u & 1) * STAGE, ((u + 1) & 1) * STAGE
        for q in range(16):
            off = rd + 16 * q
            A.append("ds_read_b128 %s, %%[ldsr]%s" % (vr(BV + 4 * q), " offset:%d" % off if off else ""))
        nv = NV + 4 * u
        for sl in range(4):
            # (the neuron vector with the first slab; the rotation vectors that go to LDS behind the last slab with it)
            A.append("s_waitcnt %slgkmcnt(%d)" % ("vmcnt(11) " if sl == 0 else "vmcnt(6) " if sl == 3 else "", 12 - 4 * sl))
            def sub(e):
                return "v_sub_f32_dpp v%d, v%d, v%d row_newbcast:%d row_mask:0xf bank_mask:0xf" % (
                    DT + (e & 7), nv + (e & 3), BV + 16 * sl + e, 4 * sl + e // 4)
            def fma(e):
                return "v_fmac_f32_e32 %%[acc], v%d, v%d" % (DT + (e & 7), DT + (e & 7))
            A.extend(sub(e) for e in range(8))
            for e in range(8):
                A.extend([fma(e), sub(8 + e)])
            A.extend(fma(8 + e) for e in range(8))
        A.append("s_cmp_eq_u32 s%d, %d" % (S_CNT, u + 1))
        A.append("s_cbranch_scc1 1f")
        st = ST[u & 1]
        for i in range(4):
            A.append("ds_write_b128 %%[ldsw], %s offset:%d" % (vr(st + 4 * i), wr + i * ROWS16))
        for i in range(4):
            gload(st + 4 * i, "%%[roff%d]" % i, S_RP, (u + 3) * 256)
        gload(nv, "%[noff]", S_NP, (u + 4) * 256)
        A.append("s_waitcnt lgkmcnt(0)")
        A.append("s_barrier")
    A.append("s_sub_u32 s%d, s%d, 4" % (S_CNT, S_CNT))
    for sb in (S_RP, S_NP):
        A.append("s_add_u32 s%d, s%d, 0x400" % (sb, sb))
        A.append("s_addc_u32 s%d, s%d, 0" % (sb + 1, sb + 1))
    A.append("s_branch 0b")
    A.append("1:")
    A.append("s_waitcnt vmcnt(0)")
    lines = []
    lines.append("// The chunk loop of the kernel for small problems, one neuron per wave (see gen_ssd_steps.py).")
    lines.append("// roff: byte offsets of the thread's four staging vectors in a chunk of the block's 64 rotation rows; noff: byte")
    lines.append("// offset of the lane's neuron vector in a chunk; ldsw, ldsr: LDS byte addresses of the thread's first staging")
    lines.append("// vector and of the lane's row in stage 0; rp, np: chunk 0 of the rotation rows and of the neuron row; chunks >= 1.")
    lines.append("__device__ __forceinline__ void ssd_lone_wave_loop(float &acc, uint32_t roff0, uint32_t roff1, uint32_t roff2, uint32_t roff3,")
    lines.append("                                                   uint32_t noff, uint32_t ldsw, uint32_t ldsr, const float *rp, const float *np,")
    lines.append("                                                   uint32_t chunks)")
    lines.append("{")
    lines.append("    asm volatile(" + "\n        ".join('"%s\\n\\t"' % a for a in A))
    lines.append('        : [acc] "+v"(acc)')
    lines.append('        : [roff0] "v"(roff0), [roff1] "v"(roff1), [roff2] "v"(roff2), [roff3] "v"(roff3), [noff] "v"(noff), [ldsw] "v"(ldsw),')
    lines.append('          [ldsr] "v"(ldsr), [rp] "s"(rp), [np] "s"(np), [cnt] "s"(chunks)')
    clob = ['"v%d"' % r for r in range(BV, NV + 16)] + ['"s%d"' % r for r in range(S_RP, S_CNT + 1)] + ['"scc"', '"memory"']
    rows = [", ".join(clob[i:i + 16]) for i in range(0, len(clob), 16)]
    lines.append("        : " + ",\n          ".join(rows) + ");")
    lines.append("}")
    return "\n".join(lines)


print("// Generated by gen_ssd_steps.py -- do not edit.")
print()
print(lone_wave_loop())
