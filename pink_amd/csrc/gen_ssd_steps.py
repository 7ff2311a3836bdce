#!/usr/bin/env python3
"""Writes ssd_steps.inc: the chunk loop of the float32 distance kernel for small problems.

    python gen_ssd_steps.py > ssd_steps.inc
"""

# Registers of the lone-wave loop (all of them clobbers of its one asm statement).
BV = 32            # v[32:95]   the lane's 64 rotation values of the chunk being computed (from LDS)
DT = 96            # v[96:103]  eight differences in flight
ST = (104, 120)    # v[104:119], v[120:135]  rotation vectors of the chunks c + 1 and c + 2 on their way to LDS
NV = 136           # v[136:151] the neuron's chunks c .. c + 3, four registers each
WL = 152           # v[152:155] (updating form) the neuron's chunks c + 1 .. c + 4, one element per lane
XL = 156           # v[156:159] (updating form) the same elements of the variant that the neuron is pulled toward
S_RP, S_NP, S_CNT, S_F, S_XP, S_WP = 40, 42, 44, 45, 46, 48   # s[40:41] rotation rows, s[42:43] neuron row, s44 chunks left,
                                                              # s45 update factor, s[46:47] variant row, s[48:49] new neuron row
STAGE = 64 * 68 * 4                 # bytes of one LDS stage: 64 rows of 64 + 4 floats
ROWS16 = 16 * 68 * 4                # bytes between a thread's four staging vectors (16 rows)
PLAIN, UPDATE, COPY = 0, 1, 2
NAMES = {PLAIN: "ssd_lone_wave_loop", UPDATE: "ssd_lone_wave_loop_update", COPY: "ssd_lone_wave_loop_copy"}


def lone_wave_loop(mode, stage=True):
    """The whole chunk loop of the kernel for small problems (one neuron per wave, about one wave per SIMD) as
    ONE asm statement.  A lone wave issues an instruction of any kind about every eight clocks, so the loop is
    written down to the instruction: per 64-element chunk 64 DPP subtracts, 64 multiply-adds, 16 LDS reads,
    4 LDS writes, 5 global loads, 3 waits, a barrier and a compare-and-branch.  It is assembly as a whole
    because its loads run three and four chunks ahead with counted waits: the compiler neither keeps such
    loads where they are written nor knows, for loads issued by assembly, that a register is still being
    written -- inside one statement with fixed registers there is nothing for it to move, copy or reuse.

    Element e of a chunk of the neuron sits in register e % 4 of lane e / 4 of every row of 16 lanes (one
    16-byte load per lane) and reaches all lanes of the row as the DPP operand of the subtract; every
    (neuron, rotation) sum is one lane's multiply-add chain in element order.  A DPP operand must not be read within
    two instruction slots of a vector-ALU write of its register (nothing checks that inside assembly): in all three
    forms the registers that the subtracts read through DPP are written by memory or LDS loads only, behind counted
    waits, never by the vector ALU.

    Three forms.  PLAIN computes the distances.  UPDATE first pulls the neuron toward a variant x with factor
    f -- w = w - ((w - x) * f), three roundings -- stores the new row to a second buffer and computes the distances
    to the new values.  The update runs one chunk ahead and on one element per lane (lane l holds element l of
    the chunk: three vector-ALU instructions for the 64 elements, where the layout of the subtract's operand, four
    elements per lane repeated in every row of 16 lanes, would take twelve): the new chunk goes to memory as it
    is and through 256 bytes of LDS of the wave's own into the operand layout (one 4-byte write per lane, one
    16-byte read per lane at the start of the next chunk; LDS operations of a wave complete in order).  COPY
    stores the chunk unchanged (all lanes store: the four rows of 16 lanes write the same bytes to the same place).

    Memory operations issued per chunk c, in this order: the store of chunk c (COPY) or c + 1 (UPDATE), four
    rotation vectors of chunk c + 3, the neuron's chunk c + 4, the variant's chunk c + 4 (UPDATE); the prologue
    issues the loads of the chunks before in the same order.  Vector memory operations complete in the
    order of issue, so "at most n outstanding" waits for everything but the last n: the n of every wait is
    counted below over the prologue and three passes of the loop, the smallest count of a place is the one
    that holds in all of them (a smaller n waits for older operations too, which by then have long arrived).
    The last chunk issues no loads; the loads of the three chunks before it read past the end of the rows.

    stage=False: the same three forms for a fifth or sixth wave of a block, which computes its neuron against the
    rotation rows that the first four put into LDS and moves none of them itself (same barriers)."""
    upd, store = mode == UPDATE, mode != PLAIN
    def vr(base, n=4):
        return "v[%d:%d]" % (base, base + n - 1)
    def gload(dst, voff, sbase, imm, tag):
        return {"text": "global_load_dwordx4 %s, %s, s[%d:%d]%s" % (vr(dst), voff, sbase, sbase + 1, " offset:%d" % imm if imm else ""),
                "vm": tag}
    def plain(text):
        return {"text": text}
    def wait(tags, lgkm=None):
        return {"wait": tags, "lgkm": lgkm}

    pro = ([plain("s_mov_b64 s[%d:%d], %%[rp]" % (S_RP, S_RP + 1))] if stage else []) + [
           plain("s_mov_b64 s[%d:%d], %%[np]" % (S_NP, S_NP + 1)), plain("s_mov_b32 s%d, %%[cnt]" % S_CNT)]
    if upd:
        pro += [plain("s_mov_b64 s[%d:%d], %%[xp]" % (S_XP, S_XP + 1)), plain("s_mov_b32 s%d, %%[f]" % S_F)]
    if store:
        pro.append(plain("s_mov_b64 s[%d:%d], %%[wp]" % (S_WP, S_WP + 1)))
    def lane_load(dst, sbase, imm, tag):
        return {"text": "global_load_dword v%d, %%[loff], s[%d:%d]%s" % (dst, sbase, sbase + 1, " offset:%d" % imm if imm else ""), "vm": tag}
    def neuron_loads(u, imm, c):
        if upd:
            return [lane_load(WL + u, S_NP, imm, ("wl", c)), lane_load(XL + u, S_XP, imm, ("xl", c))]
        return [gload(NV + 4 * u, "%[noff]", S_NP, imm, ("nv", c))]
    def update(u, c, imm):       # chunk c (register set u): the new elements to memory and to the wave's LDS stage c % 2
        return [wait([("wl", c), ("xl", c)]),
                plain("v_sub_f32_e32 v%d, v%d, v%d" % (DT, WL + u, XL + u)),
                plain("v_mul_f32_e32 v%d, s%d, v%d" % (DT, S_F, DT)),
                plain("v_sub_f32_e32 v%d, v%d, v%d" % (WL + u, WL + u, DT)),
                {"text": "global_store_dword %%[loff], v%d, s[%d:%d]%s" % (WL + u, S_WP, S_WP + 1, " offset:%d" % imm if imm else ""), "vm": ("wr", c)},
                plain("ds_write_b32 %%[scw], v%d%s" % (WL + u, " offset:256" if c & 1 else ""))]
    if upd:
        # The caller has chunk 0 of the rotations in LDS already and brings chunk 0 of the neuron and of the variant in
        # registers (it requested them ahead of its search for the best match, whose result this form needs): what is
        # left of the prologue is the requests that run ahead and the update of chunk 0.
        pro += neuron_loads(1, 256, 1)
    else:
        for i in range(4 if stage else 0):
            pro.append(gload(BV + 4 * i, "%%[roff%d]" % i, S_RP, 0, ("st", 0)))   # chunk 0 of the rotations, through the chunk registers
        pro += neuron_loads(0, 0, 0) + neuron_loads(1, 256, 1)
    if stage:
        pro += [gload(ST[0] + 4 * i, "%%[roff%d]" % i, S_RP, 256, ("st", 1)) for i in range(4)]
    pro += neuron_loads(2, 512, 2)
    if stage:
        pro += [gload(ST[1] + 4 * i, "%%[roff%d]" % i, S_RP, 512, ("st", 2)) for i in range(4)]
    pro += neuron_loads(3, 768, 3)
    if upd:
        pro += [plain("v_sub_f32_e32 v%d, %%[w0], %%[x0]" % XL),               # (register set 0 is free until chunk 4 is requested)
                plain("v_mul_f32_e32 v%d, s%d, v%d" % (XL, S_F, XL)),
                plain("v_sub_f32_e32 v%d, %%[w0], v%d" % (WL, XL)),
                {"text": "global_store_dword %%[loff], v%d, s[%d:%d]" % (WL, S_WP, S_WP + 1), "vm": ("wr", 0)},
                plain("ds_write_b32 %%[scw], v%d" % WL)]
    elif stage:
        pro.append(wait([("st", 0)]))
        for i in range(4):
            pro.append(plain("ds_write_b128 %%[ldsw], %s%s" % (vr(BV + 4 * i), " offset:%d" % (i * ROWS16) if i else "")))
    pro += [plain("s_waitcnt lgkmcnt(0)"), plain("s_barrier"), plain("0:")]

    def chunk(u, c):        # chunk c = 4 * pass + u; tags are absolute so that the counting below can find them
        out = []
        rd, wr = (u & 1) * STAGE, ((u + 1) & 1) * STAGE
        nv = NV if upd else NV + 4 * u
        if upd:
            # the chunk's new values in the operand layout, then, unless this is the last chunk, the update of the next
            out.append(plain("ds_read_b128 %s, %%[scr]%s" % (vr(NV), " offset:256" if u & 1 else "")))
        for q in range(16):
            off = rd + 16 * q
            out.append(plain("ds_read_b128 %s, %%[ldsr]%s" % (vr(BV + 4 * q), " offset:%d" % off if off else "")))
        mine = [("nv", c)]
        if upd:
            out += [plain("s_cmp_eq_u32 s%d, %d" % (S_CNT, u + 1)), plain("s_cbranch_scc1 2f")]
            out += update((u + 1) & 3, c + 1, (u + 1) * 256)
            out.append(plain("2:"))
        elif store:
            out.append(wait(mine))
            out.append({"text": "global_store_dwordx4 %%[noff], %s, s[%d:%d]%s" % (vr(nv), S_WP, S_WP + 1, " offset:%d" % (u * 256) if u else ""),
                        "vm": ("wr", c)})
        for sl in range(4):
            # Two waits for the chunk's LDS reads: the first slab's before it (with the neuron vector where it comes from
            # memory), everything else before the second -- by then the first slab's 32 instructions have given the
            # other reads all the time they need, so a wait per slab would only cost its instruction slot; the rotation
            # vectors that go to LDS behind the last slab, requested two chunks ago, ride on the second wait.
            # (UPDATE: 17 or, with the write of the update, 18 LDS operations are in the queue, the neuron's values
            # first: the first count is that of 17.)
            if sl == 0:
                out.append(wait(mine if not store else [], 12))
            elif sl == 1:
                out.append(wait([("st", c + 1)] if stage else [], 0))
            def sub(e):
                return plain("v_sub_f32_dpp v%d, v%d, v%d row_newbcast:%d row_mask:0xf bank_mask:0xf" % (
                    DT + (e & 7), nv + (e & 3), BV + 16 * sl + e, 4 * sl + e // 4))
            def fma(e):
                return plain("v_fmac_f32_e32 %%[acc], v%d, v%d" % (DT + (e & 7), DT + (e & 7)))
            out += [sub(e) for e in range(8)]
            for e in range(8):
                out += [fma(e), sub(8 + e)]
            out += [fma(8 + e) for e in range(8)]
        if not upd:
            out.append(plain("s_cmp_eq_u32 s%d, %d" % (S_CNT, u + 1)))
        out.append(plain("s_cbranch_scc1 1f"))           # (UPDATE: the comparison above still stands)
        st = ST[u & 1]
        if stage:
            out += [plain("ds_write_b128 %%[ldsw], %s offset:%d" % (vr(st + 4 * i), wr + i * ROWS16)) for i in range(4)]
            out += [gload(st + 4 * i, "%%[roff%d]" % i, S_RP, (u + 3) * 256, ("st", c + 3)) for i in range(4)]
        out += neuron_loads(u, (u + 4) * 256, c + 4)
        out += [plain("s_waitcnt lgkmcnt(0)"), plain("s_barrier")]
        return out

    # the n of every wait: operations issued behind the last one it waits for, the fewest over the passes
    passes = 3
    stream = list(pro)
    sites = {}                               # (u, index in the chunk) -> counts seen
    for ps in range(passes):
        for u in range(4):
            for k, item in enumerate(chunk(u, 4 * ps + u)):
                item = dict(item)
                item["site"] = (u, k)
                stream.append(item)
    counts = {}
    for pos, item in enumerate(stream):
        if "wait" not in item or not item["wait"]:
            continue
        last = max(i for i in range(pos) if stream[i].get("vm") in item["wait"])
        assert all(any(stream[i].get("vm") == t for i in range(pos)) for t in item["wait"])
        behind = sum(1 for i in range(last + 1, pos) if "vm" in stream[i])
        key = item.get("site", ("pro", pos))
        counts[key] = min(counts.get(key, 1 << 30), behind)
    def wait_text(item, key):
        parts = []
        if item["wait"]:
            parts.append("vmcnt(%d)" % counts[key])
        if item.get("lgkm") is not None:
            parts.append("lgkmcnt(%d)" % item["lgkm"])
        return "s_waitcnt " + " ".join(parts)
    A = []
    for pos, item in enumerate(pro):
        A.append(wait_text(item, ("pro", pos)) if "wait" in item else item["text"])
    for u in range(4):
        for k, item in enumerate(chunk(u, u)):
            A.append(wait_text(item, (u, k)) if "wait" in item else item["text"])
    A.append("s_sub_u32 s%d, s%d, 4" % (S_CNT, S_CNT))
    for sb in ([S_RP] if stage else []) + [S_NP] + ([S_XP] if upd else []) + ([S_WP] if store else []):
        A.append("s_add_u32 s%d, s%d, 0x400" % (sb, sb))
        A.append("s_addc_u32 s%d, s%d, 0" % (sb + 1, sb + 1))
    A.append("s_branch 0b")
    A.append("1:")
    A.append("s_waitcnt vmcnt(0)")

    name = NAMES[mode] + ("" if stage else "_unstaged")
    extra_args = {PLAIN: "", UPDATE: ", const float *xp, float *wp, float f, uint32_t loff, uint32_t scw, uint32_t scr, float w0, float x0",
                  COPY: ", float *wp"}[mode]
    extra_ops = {PLAIN: "", UPDATE: ', [xp] "s"(xp), [wp] "s"(wp), [f] "s"(f), [loff] "v"(loff), [scw] "v"(scw), [scr] "v"(scr), [w0] "v"(w0), [x0] "v"(x0)',
                 COPY: ', [wp] "s"(wp)'}[mode]
    lines = []
    lines.append({PLAIN: "// The chunk loop of the kernel for small problems, one neuron per wave (see gen_ssd_steps.py).",
                  UPDATE: "// The same loop, the neuron pulled toward the variant row xp with factor f first and its new row stored to wp\n"
                          "// (loff: byte offset of the lane's element in a chunk; scw, scr: LDS byte addresses of the lane's element and of its\n"
                          "// 16-byte piece in 512 bytes of the wave's own; w0, x0: the lane's element of chunk 0 of the neuron and of the variant.\n"
                          "// The caller has stored chunk 0 of the rotation rows to LDS stage 0; the loop's first barrier publishes it.)",
                  COPY: "// The same loop, the neuron's row also stored to wp as it is."}[mode])
    if mode == PLAIN:
        lines.append("// roff: byte offsets of the thread's four staging vectors in a chunk of the block's 64 rotation rows; noff: byte")
        lines.append("// offset of the lane's neuron vector in a chunk; ldsw, ldsr: LDS byte addresses of the thread's first staging")
        lines.append("// vector and of the lane's row in stage 0; rp, np: chunk 0 of the rotation rows and of the neuron row; chunks >= 1.")
    if stage:
        lines.append("__device__ __forceinline__ void %s(float &acc, uint32_t roff0, uint32_t roff1, uint32_t roff2, uint32_t roff3," % name)
        lines.append("        uint32_t noff, uint32_t ldsw, uint32_t ldsr, const float *rp, const float *np, uint32_t chunks%s)" % extra_args)
    else:
        lines = ["// %s for a wave that stages no rotation rows (the block's first four do): the same operands but for" % NAMES[mode],
                 "// roff, ldsw and rp; UPDATE: the caller stores nothing to LDS."]
        lines.append("__device__ __forceinline__ void %s(float &acc, uint32_t noff, uint32_t ldsr, const float *np, uint32_t chunks%s)" % (name, extra_args))
    lines.append("{")
    lines.append("    asm volatile(" + "\n        ".join('"%s\\n\\t"' % a for a in A))
    lines.append('        : [acc] "+v"(acc)')
    if stage:
        lines.append('        : [roff0] "v"(roff0), [roff1] "v"(roff1), [roff2] "v"(roff2), [roff3] "v"(roff3), [noff] "v"(noff), [ldsw] "v"(ldsw),')
        lines.append('          [ldsr] "v"(ldsr), [rp] "s"(rp), [np] "s"(np), [cnt] "s"(chunks)%s' % extra_ops)
    else:
        lines.append('        : [noff] "v"(noff), [ldsr] "v"(ldsr), [np] "s"(np), [cnt] "s"(chunks)%s' % extra_ops)
    clob = ['"v%d"' % r for r in range(BV, XL + 4 if upd else NV + 16)] + ['"s%d"' % r for r in range(S_RP, S_WP + 2)] + ['"scc"', '"memory"']
    rows = [", ".join(clob[i:i + 16]) for i in range(0, len(clob), 16)]
    lines.append("        : " + ",\n          ".join(rows) + ");")
    lines.append("}")
    return "\n".join(lines)


print("// Generated by gen_ssd_steps.py -- do not edit.")
for stage in (True, False):
    for mode in (PLAIN, UPDATE, COPY):
        print()
        print(lone_wave_loop(mode, stage))
