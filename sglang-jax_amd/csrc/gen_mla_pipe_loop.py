#!/usr/bin/env python3
"""Generator of ``rpa_mla_pipe_loop.inc``: the steady-state tile loop of the absorbed-MLA kernels
(rpa_mla.hip) as hand-scheduled gfx950 assembly.

    python gen_mla_pipe_loop.py            # rewrites rpa_mla_pipe_loop.inc next to it

One wave of an eight-wave workgroup owns 16 heads of one row; a step covers one 32-token tile of
latent rows that sits in one slot of a four-slot LDS ring (rows of 1184 bytes):
    scores   S^T[32 tokens x 16 heads] = K . Q^T      36 MFMAs 16x16x32 (18 k-steps x 2 token blocks)
    softmax  p = 2^(s * scale2 - m), packed to bf16, row sums               (about 30 vector instructions)
    output   O^T[512 dims x 16 heads] += V^T . P^T    32 MFMAs, V^T read with the transposing LDS read
What the compiled loop cannot do for lack of registers it does not know how to spare -- 200 of the
wave's 256 registers are accumulators and Q^T -- this loop does with a ring of four 4-register
operand buffers shared by both products: every LDS operand is requested three matrix instructions
before the one that consumes it, so the matrix pipe no longer waits a full LDS round trip per
instruction.  The five global -> LDS copy instructions of the step (tile t + 3) are spread over the
first product; the page id of tile t + 4 is a scalar load issued at the top of the step.

The running maximum is a reference, not a maximum: probabilities are taken against the value
known before the tile, and a lane whose eight probabilities sum to more than 2^8 (a score beat
the reference by more than 5 in log2 units) sends the wave through the rare path, which raises
the reference of the heads concerned by 16, 32, 64, ... (accumulators, row sums rescaled by the
matching power of two) until the sum fits or eight rounds have passed.  No maximum is ever taken
across lanes.  Results do not depend on the reference: the normalisation divides it out, and the
merge of partial rows takes whatever (reference, sum) pair a piece leaves.

The loop is generated twice.  For bf16 caches as described.  For e4m3 caches (macros with F8 in their
names) a tile arrives as bytes in one of three staging areas (18 copy blocks, three copy instructions
per wave) and the ring has two bf16 slots: a step ends with a barrier (the bytes of tile t + 1 have
landed), the expansion of that tile -- every thread reads up to three 16-byte chunks, converts them with
v_cvt_scalef32_pk_bf16_fp8 and writes 32 bytes each into the ring slot the next step reads -- and a
second barrier; six unrolled steps cover the two-slot ring and the three staging areas.

Register use follows one table shared with the C++ side through the emitted constraint macros;
waits for LDS data and the issue distances the hardware does not interlock come from the
emitter of gen_prefill_pipe_loop.py.
"""

from __future__ import annotations

import os
import sys

sys.dont_write_bytecode = True  # no __pycache__ next to the sources
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from gen_prefill_pipe_loop import Emitter, Ins, rng, valu, vr  # noqa: E402

X = set(os.environ.get("RPA_MLA_PIPE_X", "").split(","))   # timing probes only (results are wrong)
AHEAD = int(os.environ.get("RPA_MLA_PIPE_AHEAD", 3))
NBUF = 4

ROW_B = 1184                 # bytes of a latent row in LDS
F8 = False                   # which of the two loops is being generated (set by emit_text)
BLOCKS = 37                  # 1 KiB copy blocks per tile (18 for a tile of bytes)
COPIES = 5                   # copy instructions per wave and tile (3)

# ---- vector registers
O = 0                        # 32 accumulators of 4
Q = 128                      # 18 Q^T operands of 4
S = [200, 204]               # scores of the two 16-token blocks
P = 208                      # packed probabilities (B operand of the second product)
E = 212                      # 8 exponent temporaries
RING = 220                   # NBUF operand buffers of 4
ML = 236                     # M, L, KBASE, VBASE (one operand of 4)
M, L, KBASE, VBASE = 236, 237, 238, 239
OFS = 240                    # one operand of 8: per-lane byte offsets of the wave's copies first, scratch behind
NEGM, PS, KADDR = 245, 246, 247
VADDR, D, A = 248, 249, 250
NUM_VGPR = 251
# e4m3 caches: three copy offsets, then what the expansion needs of every thread
F8_SRC = 243                 # byte offset of the thread's first chunk inside a staging area (16 * thread)
F8_DST = [244, 245, 246]     # byte offsets of its three chunks inside a ring slot
F8_TABLE = dict(NEGM=247, PS=248, KADDR=249, VADDR=250, D=251, A=252, NUM_VGPR=253)
BF_TABLE = dict(NEGM=245, PS=246, KADDR=247, VADDR=248, D=249, A=250, NUM_VGPR=251)

# ---- scalar registers used inside the block (all listed as clobbers)
SB = 60                      # s[60:61] global base of the tile being copied
ST = [62, 63, 64, 65]        # temporaries
PGN = 66                     # page id of tile t + 4
ONES, LIMIT, DELTA, PASS = 67, 68, 69, 70
PMASK, PSTR = 71, 72         # page_size - 1, bytes per page
SGPR_CLOBBERS = list(range(60, 73))


def mfma(dst, a, b, c):
    reads = list(rng(a, 4)) + list(rng(b, 4)) + (list(rng(c, 4)) if c is not None else [])
    if "nomfma" in X:
        return Ins("s_nop 0", "nop")
    ctext = vr(c, 4) if c is not None else "0"
    return Ins(f"v_mfma_f32_16x16x32_bf16 {vr(dst, 4)}, {vr(a, 4)}, {vr(b, 4)}, {ctext}", "mfma", reads, rng(dst, 4))


def ring(f):
    return RING + 4 * (f % NBUF)


def frag_read(f):
    """operand fragment f of the tile: 0..35 K of (k-step f >> 1, token block f & 1), 36..67 V^T of dim chunk f - 36"""
    dst = ring(f)
    if "nolds" in X or ("halflds" in X and f % 2 == 1):  # halflds: what fragments shared by 32 heads would read
        return []
    if f < 36:
        ks, b = f >> 1, f & 1
        off = b * 16 * ROW_B + ks * 64
        return [Ins(f"ds_read_b128 {vr(dst, 4)}, {vr(KADDR)} offset:{off}", "lds", [KADDR], rng(dst, 4), lds_tag=("k", f))]
    j = f - 36
    return [Ins(f"ds_read_b64_tr_b16 {vr(dst, 2)}, {vr(VADDR)} offset:{j * 32}", "lds", [VADDR], rng(dst, 2), lds_tag=("vlo", f)),
            Ins(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, {vr(VADDR)} offset:{j * 32 + 16 * ROW_B}", "lds", [VADDR],
                rng(dst + 2, 2), lds_tag=("vhi", f))]


def frag_mfma(f):
    if f < 36:
        ks, b = f >> 1, f & 1
        ins = mfma(S[b], ring(f), Q + 4 * ks, None if ks == 0 else S[b])
        ins.lds_need = None if "nolds" in X or ("halflds" in X and f % 2 == 1) else [("k", f)]
    else:
        j = f - 36
        ins = mfma(O + 4 * j, ring(f), P, O + 4 * j)
        ins.lds_need = None if "nolds" in X or ("halflds" in X and f % 2 == 1) else [("vlo", f), ("vhi", f)]
    return ins


def softmax(check=True):
    """x = s * scale2 - m, p = 2^x, packed pairs, the lane's sum of the eight; the scores stay in S"""
    out = [valu(f"v_mov_b32 {vr(PS)}, 0", [], [PS])]
    s_regs = [S[0] + r for r in range(4)] + [S[1] + r for r in range(4)]   # p[i]: token block i >> 2, register i & 3
    for i in range(8):
        out.append(valu(f"v_fma_f32 {vr(E + i)}, {vr(s_regs[i])}, %[scale2], {vr(NEGM)}", [s_regs[i], NEGM], [E + i]))
    for i in range(8):
        out.append(valu(f"v_exp_f32 {vr(E + i)}, {vr(E + i)}", [E + i], [E + i], "trans"))
    for j in range(4):
        out.append(valu(f"v_cvt_pk_bf16_f32 {vr(P + j)}, {vr(E + 2 * j)}, {vr(E + 2 * j + 1)}", [E + 2 * j, E + 2 * j + 1], [P + j]))
    for j in range(4):
        out.append(valu(f"v_dot2c_f32_bf16 {vr(PS)}, s{ONES}, {vr(P + j)}", [P + j, PS], [PS], "dot"))
    if check:
        out.append(valu(f"v_cmp_nle_f32 vcc, {vr(PS)}, s{LIMIT}", [PS], []))
    return out


def copy_group(n, fill_slot):
    """copy n of this wave: block 5 * wave + n of the slot (blocks past the 37th repeat block 0)"""
    a = f"s{ST[0]}"
    dst = f"%[stage{fill_slot}]" if F8 else f"%[slot{fill_slot}]"
    return [Ins(f"s_add_u32 {a}, %[wave_blk], {n * 1024}", "salu"),
            Ins(f"s_cmp_lt_u32 {a}, {BLOCKS * 1024}", "salu"),
            Ins(f"s_cselect_b32 {a}, {a}, 0", "salu"),
            Ins(f"s_add_u32 m0, {a}, {dst}", "salu"),
            Ins("s_nop 0", "nop"),
            Ins(f"global_load_lds_dwordx4 {vr(OFS + n)}, s[{SB}:{SB + 1}]", "vmem", [OFS + n], [])]


def tile_scalars(em):
    """s[SB:SB+1] = base of tile t + 3 (page %[pg]); page id of tile t + 4 requested into s[PGN]"""
    t0, t1, a, b = (f"s{x}" for x in ST)
    em.raw(f"s_lshl_b32 {t0}, %[t], 5")
    em.raw(f"s_add_u32 {t0}, {t0}, %[t_begin]")
    em.raw(f"s_add_u32 {t0}, {t0}, 96")                        # first token of tile t + 3
    em.raw(f"s_add_u32 {t1}, {t0}, 32")                        # ... of tile t + 4
    em.raw(f"s_min_i32 {t0}, {t0}, %[last_tile_tok]")          # past the end: the last tile again
    em.raw(f"s_min_i32 {t1}, {t1}, %[last_tile_tok]")
    em.raw(f"s_and_b32 {a}, {t0}, s{PMASK}")
    em.raw(f"s_mul_i32 {a}, {a}, %[row_bytes]")                # bytes inside the page (< 2^32)
    em.raw(f"s_mul_hi_u32 {b}, %[pg], s{PSTR}")
    em.raw(f"s_mul_i32 s{SB}, %[pg], s{PSTR}")
    em.raw(f"s_add_u32 s{SB}, s{SB}, {a}")
    em.raw(f"s_addc_u32 {b}, {b}, 0")
    em.raw(f"s_add_u32 s{SB}, s{SB}, %[cache_lo]")
    em.raw(f"s_addc_u32 s{SB + 1}, {b}, %[cache_hi]")
    em.raw(f"s_lshr_b32 {t1}, {t1}, %[pshift]")
    em.raw(f"s_lshl_b32 {t1}, {t1}, 2")
    em.raw(f"s_load_dword s{PGN}, %[pages], {t1}")


def expansion(em, stage, slot):
    """e4m3 caches: the staged bytes of the next tile become bf16 rows of ring slot `slot`.  Thread i owns chunks
    i, i + 512 and (waves 0 and 1 only) i + 1024 of the tile's 1152 chunks of 16 elements."""
    # registers that are idle between two steps: (bytes read, bf16 out) twice over, used alternately so that no
    # conversion writes what an LDS write issued just before still reads
    sets = [(RING, RING + 4), (RING + 12, E)]
    em.emit(valu(f"v_add_u32 {vr(KADDR)}, %[stage{stage}], {vr(F8_SRC)}", [F8_SRC], [KADDR]))

    def read(i):
        src = sets[i & 1][0]
        em.emit(Ins(f"ds_read_b128 {vr(src, 4)}, {vr(KADDR)} offset:{8192 * i}", "lds", [KADDR], rng(src, 4), lds_tag=("x", i)))

    def convert_and_write(i):
        src, tmp = sets[i & 1]
        em.emit(valu(f"v_add_u32 {vr(VADDR)}, %[slot{slot}], {vr(F8_DST[i])}", [F8_DST[i]], [VADDR]))
        for d in range(4):
            lo = valu(f"v_cvt_scalef32_pk_bf16_fp8 {vr(tmp + 2 * d)}, {vr(src + d)}, 1.0", [src + d], [tmp + 2 * d])
            lo.lds_need = [("x", i)]
            em.emit(lo)
            em.emit(valu(f"v_cvt_scalef32_pk_bf16_fp8 {vr(tmp + 2 * d + 1)}, {vr(src + d)}, 1.0 op_sel:[1,0,0]", [src + d],
                         [tmp + 2 * d + 1]))
        em.emit(Ins(f"ds_write_b128 {vr(VADDR)}, {vr(tmp, 4)}", "lds", [VADDR] + list(rng(tmp, 4)), []))
        em.emit(Ins(f"ds_write_b128 {vr(VADDR)}, {vr(tmp + 4, 4)} offset:16", "lds", [VADDR] + list(rng(tmp + 4, 4)), []))
        em.raw("s_nop 1", "nop")       # the address register is rewritten next: let the writes pick it up

    read(0)
    read(1)
    convert_and_write(0)
    convert_and_write(1)
    em.raw(f"s_cmp_lt_u32 %[wave_blk], {2 * COPIES * 1024}")   # waves 0 and 1
    em.raw(f"s_cbranch_scc0 L_expanded_{stage}_{slot}_%=")
    read(2)
    convert_and_write(2)
    em.label(f"L_expanded_{stage}_{slot}_%=")
    em.raw("s_waitcnt lgkmcnt(0)", "wait")
    em.lds_queue = []
    em.raw("s_barrier")


def step(em, k):
    """bf16: tile t in slot k, tile t + 3 goes to slot (k + 3) & 3.  e4m3: tile t in ring slot k & 1, the bytes of
    tile t + 3 go to staging area k % 3, tile t + 1 (staging area (k + 1) % 3) is expanded into the other slot."""
    fill = (k % 3) if F8 else ((k + 3) & 3)
    cur = (k & 1) if F8 else k
    tile_scalars(em)
    em.emit(valu(f"v_add_u32 {vr(KADDR)}, %[slot{cur}], {vr(KBASE)}", [KBASE], [KADDR]))
    em.emit(valu(f"v_add_u32 {vr(VADDR)}, %[slot{cur}], {vr(VBASE)}", [VBASE], [VADDR]))
    for f in range(AHEAD):
        for x in frag_read(f):
            em.emit(x)
    copies = [] if "nocopy" in X else [copy_group(n, fill) for n in range(COPIES)]
    copy_at = {4 + (30 // COPIES) * n: n for n in range(COPIES)}   # behind these matrix instructions of the first product
    if "copypv" in X:
        copy_at = {38 + 6 * n: n for n in range(COPIES)}
    if "copyend" in X:
        copy_at = {67: -1}
    if "copyfirst" in X:
        copy_at = {}
        for grp in copies:
            for x in grp:
                em.emit(x)
    sm = softmax()
    for f in range(36):
        em.emit(frag_mfma(f))
        if f + AHEAD < 68:
            for x in frag_read(f + AHEAD):
                em.emit(x)
        if f in copy_at and copies:
            for x in copies[copy_at[f]]:
                em.emit(x)
    if "novalu" not in X:
        for x in sm:
            em.emit(x)
        if "norare" not in X:
            em.raw(f"s_cbranch_vccnz L_rare_{k}_%=")
    em.label(f"L_back_{k}_%=")
    if "novalu" not in X:
        em.emit(valu(f"v_add_f32 {vr(L)}, {vr(L)}, {vr(PS)}", [L, PS], [L]))
    for f in range(36, 68):
        em.emit(frag_mfma(f))
        if f + AHEAD < 68:
            for x in frag_read(f + AHEAD):
                em.emit(x)
        if f in copy_at and copies:
            for grp in (copies if copy_at[f] < 0 else [copies[copy_at[f]]]):
                for x in grp:
                    em.emit(x)
    assert not em.lds_queue
    # end of step: tile t + 1 has landed once only the ten newest copies (tiles t + 2, t + 3) are outstanding;
    # every LDS read of tile t has returned, so its slot may be refilled after the barrier
    em.raw("s_waitcnt lgkmcnt(0)" if "novmwait" in X else f"s_waitcnt vmcnt({2 * COPIES}) lgkmcnt(0)", "wait")
    em.raw(f"s_mov_b32 %[pg], s{PGN}")
    if "nobarrier" not in X:
        em.raw("s_barrier")
    if F8:
        expansion(em, (k + 1) % 3, (k + 1) & 1)
    em.raw("s_add_u32 %[t], %[t], 1")
    em.raw("s_cmp_lt_i32 %[t], %[t_end]")


def rare_block(em, k):
    """some lane's sum blew up: raise the reference of its head (all four lanes of the head alike) and redo the
    tile's probabilities; twice the raise on every further round"""
    a, b = f"s{ST[0]}", f"s{ST[1]}"
    em.label(f"L_rare_{k}_%=")
    em.raw(f"s_mov_b32 s{DELTA}, 0x41800000")                   # 16.0
    em.raw(f"s_mov_b32 s{PASS}, 0")
    em.label(f"L_rare_again_{k}_%=")
    # a head's four lanes are c, c + 16, c + 32, c + 48: fold the mask onto 16 bits and spread it again
    em.raw(f"s_or_b32 {a}, vcc_lo, vcc_hi")
    em.raw(f"s_lshr_b32 {b}, {a}, 16")
    em.raw(f"s_or_b32 {a}, {a}, {b}")
    em.raw(f"s_and_b32 {a}, {a}, 0xffff")
    em.raw(f"s_lshl_b32 {b}, {a}, 16")
    em.raw(f"s_or_b32 {a}, {a}, {b}")
    em.raw(f"s_mov_b32 vcc_lo, {a}")
    em.raw(f"s_mov_b32 vcc_hi, {a}")
    em.emit(valu(f"v_mov_b32 {vr(A)}, s{DELTA}", [], [A]))
    em.raw("s_nop 1", "nop")                                    # scalar write of vcc -> vector read as a mask
    em.emit(valu(f"v_cndmask_b32 {vr(D)}, 0, {vr(A)}, vcc", [A], [D]))
    em.emit(valu(f"v_sub_f32 {vr(NEGM)}, {vr(NEGM)}, {vr(D)}", [NEGM, D], [NEGM]))
    em.emit(valu(f"v_add_f32 {vr(M)}, {vr(M)}, {vr(D)}", [M, D], [M]))
    em.emit(valu(f"v_exp_f32 {vr(A)}, -{vr(D)}", [D], [A], "trans"))
    em.emit(valu(f"v_mul_f32 {vr(L)}, {vr(L)}, {vr(A)}", [L, A], [L]))
    for r in range(128):
        em.emit(valu(f"v_mul_f32 {vr(O + r)}, {vr(O + r)}, {vr(A)}", [O + r, A], [O + r]))
    for x in softmax():
        em.emit(x)
    em.raw(f"s_add_u32 s{PASS}, s{PASS}, 1")
    em.raw(f"s_add_u32 s{DELTA}, s{DELTA}, 0x00800000")         # twice the raise next time: exponent + 1
    em.raw(f"s_cmp_ge_u32 s{PASS}, 8")
    em.raw(f"s_cbranch_scc1 L_rare_done_{k}_%=")
    em.raw(f"s_cbranch_vccnz L_rare_again_{k}_%=")
    em.label(f"L_rare_done_{k}_%=")
    em.raw("s_nop 3", "nop")                                    # P and O were written by the vector pipe
    em.raw(f"s_branch L_back_{k}_%=")


def generate():
    em = Emitter()
    em.raw("s_waitcnt lgkmcnt(0)", "wait")
    em.raw("s_nop 11", "nop")                                   # the caller's matrix instructions have finished
    em.raw(f"s_mov_b32 s{ONES}, 0x3f803f80")
    em.raw(f"s_mov_b32 s{LIMIT}, 0x43800000")                   # 256.0
    em.raw(f"s_lshl_b32 s{PMASK}, 1, %[pshift]")
    em.raw(f"s_sub_u32 s{PMASK}, s{PMASK}, 1")
    em.raw(f"s_lshl_b32 s{PSTR}, %[row_bytes], %[pshift]")
    em.emit(valu(f"v_mul_f32 {vr(NEGM)}, -1.0, {vr(M)}", [M], [NEGM]))
    # the unrolled copies of the step differ in their LDS constants only: tile t takes copy t & 3 (bf16: four
    # ring slots) or t % 6 (e4m3: two ring slots, three staging areas)
    a, b = f"s{ST[0]}", f"s{ST[1]}"
    n_steps = 6 if F8 else 4
    if F8:
        em.raw(f"s_mul_hi_u32 {a}, %[t], 0xaaaaaaab")
        em.raw(f"s_lshr_b32 {a}, {a}, 2")                       # t / 6
        em.raw(f"s_mul_i32 {a}, {a}, 6")
        em.raw(f"s_sub_u32 {a}, %[t], {a}")
    else:
        em.raw(f"s_and_b32 {a}, %[t], 3")
    for k in range(1, n_steps):
        em.raw(f"s_cmp_eq_u32 {a}, {k}")
        em.raw(f"s_cbranch_scc1 L_step_{k}_%=")
    for k in range(n_steps):
        em.label(f"L_step_{k}_%=")
        step(em, k)
        if k < n_steps - 1:
            em.raw("s_cbranch_scc0 L_exit_%=")
        else:
            em.raw("s_cbranch_scc1 L_step_0_%=")
            em.raw("s_branch L_exit_%=")
    for k in range(n_steps):
        rare_block(em, k)
    em.label("L_exit_%=")
    em.raw("s_nop 11", "nop")
    return em


def emit_text(f8):
    global F8, BLOCKS, COPIES, NEGM, PS, KADDR, VADDR, D, A, NUM_VGPR
    F8 = f8
    BLOCKS, COPIES = (18, 3) if f8 else (37, 5)
    tab = F8_TABLE if f8 else BF_TABLE
    NEGM, PS, KADDR, VADDR, D, A, NUM_VGPR = (tab[k] for k in ("NEGM", "PS", "KADDR", "VADDR", "D", "A", "NUM_VGPR"))
    em = generate()
    n_mfma = sum(1 for i in em.out if i.kind == "mfma")
    n_valu = sum(1 for i in em.out if i.kind in ("valu", "trans", "swap", "dot"))
    pre = "RPA_MLA_PIPE_F8" if f8 else "RPA_MLA_PIPE"
    text = (f"// {'e4m3' if f8 else 'bf16'} caches: {len(em.out)} lines, {n_mfma} matrix and {n_valu} vector instructions "
            f"({6 if f8 else 4} unrolled steps and their rare paths), {em.nops} padding wait states; {NUM_VGPR} vector registers\n")
    if not f8:
        binds = {f"O{i}": (O + 16 * i, 16) for i in range(8)}
        binds.update({"Q0": (Q, 32), "Q1": (Q + 32, 32), "Q2": (Q + 64, 8), "ML": (ML, 4), "OFS": (OFS, 8)})
        for name, (lo, n) in binds.items():
            text += f'#define RPA_MLA_PIPE_C_{name} "{{{vr(lo, n)}}}"\n'
    lines = ['    "%s\\n"' % ins.text for ins in em.out]
    text += f"#define {pre}_ASM \\\n" + " \\\n".join(lines) + "\n"
    clob = ['"v%d"' % r for r in list(range(S[0], ML)) + list(range(OFS + 8, NUM_VGPR))]
    clob += ['"s%d"' % r for r in SGPR_CLOBBERS]
    text += f"#define {pre}_CLOBBERS " + ", ".join(clob) + ', "vcc", "scc", "m0", "memory"\n'
    print(f"MLA {'e4m3' if f8 else 'bf16'}: {len(em.out)} lines, {n_mfma} MFMAs, {n_valu} vector, {em.nops} padding wait states, "
          f"{NUM_VGPR} VGPRs")
    return text


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    text = ("// GENERATED by gen_mla_pipe_loop.py -- do not edit; edit the generator and run it.\n"
            "// Steady-state tile loop of the absorbed-MLA kernels: tiles t .. t_end-1 of one wave (16 heads).  The\n"
            "// RPA_MLA_PIPE_C_* macros are the register constraints that bind the kernel's variables to the\n"
            "// registers the assembly uses.\n")
    text += emit_text(False)
    text += emit_text(True)
    with open(os.path.join(here, "rpa_mla_pipe_loop.inc"), "w") as f:
        f.write(text)


if __name__ == "__main__":
    sys.exit(main())
