#!/usr/bin/env python3
"""Generator of ``rpa_mla_wide_loop.inc``: the tile loop of the wide absorbed-MLA kernels (rpa_mla.hip,
four waves of 32 heads per workgroup) as hand-scheduled gfx950 assembly.

    python gen_mla_wide_loop.py            # rewrites rpa_mla_wide_loop.inc next to it

One wave owns TWO blocks of 16 heads of one row, so that every operand fragment read from LDS feeds two
matrix instructions: LDS reads, not the matrix pipe, are what the eight-wave workgroups of
gen_mla_pipe_loop.py wait for.  A step covers one 32-token tile of latent rows in one slot of a four-slot
LDS ring (rows of 1184 bytes), per block of heads:
    scores   S^T[32 tokens x 16 heads] = K . Q^T      36 MFMAs 16x16x32
    softmax  p = 2^(s * scale2 - m), packed to bf16, row sums
    output   O^T[512 dims x 16 heads] += V^T . P^T    32 MFMAs, V^T read with the transposing LDS read
The 256 accumulators live in the accumulation registers and are touched by nothing but the matrix
instructions (and the rare path); Q^T takes 144 vector registers; one wave per SIMD.

A step runs scores, softmax, second product of one tile in that order, LDS operands requested six fragments
(twelve matrix instructions) ahead into a ring of eight buffers.  `RPA_MLA_WIDE_X=pipe` generates a loop that
is software-pipelined across tiles instead (step t issues the scores of tile t + 1 into a second set of score
registers, interleaved one for one with the softmax of tile t; four operand buffers): measured 4 % slower --
what bounds a lone wave is the number of instructions it has to issue, not the softmax's place in the step.

The loop runs EVERY tile of a segment, so no compiled code ever holds the accumulators:
  * the reference the probabilities are taken against comes in from the caller (the maximum of the first
    tile's scores, worked out before any accumulator exists) and only ever rises (rare path, as in
    gen_mla_pipe_loop.py: +16, +32, +64 ... for the heads whose row sum passed 2^8);
  * the first tile and the row's last tile take a masking detour after their scores: tokens before the
    window's edge or past the row's end get -1e30 (per-lane limits come in with the caller's operands).  Token
    groups (a wave's two blocks of heads belong to neighbouring query tokens of a chunk, whose rows end up to
    seven tokens before the group's last) also take it on the tile before the last (%[mask_early] = 1), and the
    second block's row ends %[hi_step] tokens after the first's;
  * from the moment the tile being copied (three ahead) is the row's last, the copies use a second set of
    per-lane offsets whose rows are clamped to the last valid token, so no bytes from beyond the row ever
    reach LDS.

Register use follows one table shared with the C++ side through the emitted constraint macros; waits for
LDS data and the issue distances the hardware does not interlock come from the emitter of
gen_prefill_pipe_loop.py.
"""

from __future__ import annotations

import os
import sys

sys.dont_write_bytecode = True  # no __pycache__ next to the sources
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from gen_prefill_pipe_loop import ACC, Emitter, Ins, rng, valu, vr  # noqa: E402

X = set(os.environ.get("RPA_MLA_WIDE_X", "").split(","))   # timing probes (nocopy, nolds, novalu, norare: wrong results)
PIPELINED = "pipe" in X      # scores of tile t + 1 under the softmax of tile t (measured slower: off)
NBUF = 4 if PIPELINED else 8  # operand fragment buffers (the second set of score registers of the pipelined loop pays for four)
AHEAD = int(os.environ.get("RPA_MLA_WIDE_AHEAD", 3 if PIPELINED else 6))
assert AHEAD < NBUF
WAITGROUP = int(os.environ.get("RPA_MLA_WIDE_WAITGROUP", 4))  # fragments whose data one wait instruction covers
assert 1 <= WAITGROUP <= AHEAD

ROW_B = 1184                 # bytes of a latent row in LDS
SLOT_B = 37 * 1024           # one ring slot
BLOCKS = 37                  # 1 KiB copy blocks per tile
COPIES = 10                  # copy instructions per wave and tile

# ---- accumulation registers: O[hb] = 32 accumulators of 4
O = [ACC, ACC + 128]
# ---- vector registers
Q = [0, 72]                  # 18 Q^T operands of 4 per block of heads
SC = [[144, 148], [152, 156]]            # scores [hb][token block]
if PIPELINED:
    SC2 = [[160, 164], [168, 172]]       # the other set (sets alternate per step)
    P = [176, 180]           # packed probabilities per block of heads
    E = 184                  # 8 exponent temporaries
    RING = 192               # NBUF operand buffers of 4
else:
    SC2 = SC
    P = [160, 164]
    E = 168
    RING = 176
ML = 208                     # one operand of 8: M0, L0, M1, L1, KBASE, VBASE, LO, HI
M = [208, 210]
L = [209, 211]
KBASE, VBASE, LO, HI = 212, 213, 214, 215
OFS = 216                    # one operand of 16: 10 per-lane copy offsets, scratch behind
NEGM = [226, 227]
PS, KADDR, VADDR, D = 228, 229, 230, 231
OFSL = 232                   # one operand of 16: the 10 offsets with rows clamped to the row's last token, scratch behind
A, T0, T1, KADDR2 = 242, 243, 244, 245
TR = [246, 247]              # temporaries of the accumulator rescale
NUM_VGPR = 248

# ---- scalar registers used inside the block (all listed as clobbers)
SB = 60                      # s[60:61] global base of the tile being copied
ST = [62, 63, 64, 65]        # temporaries
PGN = 66                     # page id of tile t + 4
ONES, LIMIT, DELTA, PASS = 67, 68, 69, 70
PMASK, PSTR = 71, 72         # page_size - 1, bytes per page
LASTK = 73                   # first tile, counted from the segment's first, of the masked tail (the row's last, or the one before)
CPB = 74                     # LDS address of this wave's first copy block in slot 0 (see copy_group)
SGPR_CLOBBERS = list(range(60, 75))

NEG_BIG = "0xf149f2ca"       # -1e30


def mfma(dst, a, b, c):
    reads = list(rng(a, 4)) + list(rng(b, 4)) + (list(rng(c, 4)) if c is not None else [])
    if "nomfma" in X:
        return Ins("s_nop 0", "nop")
    ctext = vr(c, 4) if c is not None else "0"
    return Ins(f"v_mfma_f32_16x16x32_bf16 {vr(dst, 4)}, {vr(a, 4)}, {vr(b, 4)}, {ctext}", "mfma", reads, rng(dst, 4))


def ring(f):
    return RING + 4 * (f % NBUF)


def frag_read(f, kaddr=None):
    """operand fragment f of a tile: 0..35 K of (k-step f >> 1, token block f & 1), 36..67 V^T of dim chunk f - 36"""
    dst = ring(f)
    if "nolds" in X:
        return []
    if f < 36:
        ks, b = f >> 1, f & 1
        off = b * 16 * ROW_B + ks * 64
        ka = KADDR if kaddr is None else kaddr
        return [Ins(f"ds_read_b128 {vr(dst, 4)}, {vr(ka)} offset:{off}", "lds", [ka], rng(dst, 4), lds_tag=("k", f))]
    j = f - 36
    return [Ins(f"ds_read_b64_tr_b16 {vr(dst, 2)}, {vr(VADDR)} offset:{j * 32}", "lds", [VADDR], rng(dst, 2), lds_tag=("vlo", f)),
            Ins(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, {vr(VADDR)} offset:{j * 32 + 16 * ROW_B}", "lds", [VADDR],
                rng(dst + 2, 2), lds_tag=("vhi", f))]


def frag_tags(f):
    return [("k", f)] if f < 36 else [("vlo", f), ("vhi", f)]


def frag_mfmas(f, sc):
    """the two matrix instructions (one per block of heads) that consume fragment f; scores go to `sc`.  The first
    instruction of every WAITGROUP-th fragment also waits for the fragments behind it in its group (requested long
    before): one wait instruction per group -- a lone wave pays for every instruction it issues."""
    out = []
    for hb in range(2):
        if f < 36:
            ks, b = f >> 1, f & 1
            ins = mfma(sc[hb][b], ring(f), Q[hb] + 4 * ks, None if ks == 0 else sc[hb][b])
        else:
            j = f - 36
            ins = mfma(O[hb] + 4 * j, ring(f), P[hb], O[hb] + 4 * j)
        ins.lds_need = None if "nolds" in X else list(frag_tags(f))
        if hb == 0 and f % WAITGROUP == 0 and ins.lds_need is not None:
            for g in range(f + 1, min(f + WAITGROUP, 68)):
                ins.lds_need += frag_tags(g)
        out.append(ins)
    return out


def softmax(hb, sc, check=True):
    """x = s * scale2 - m, p = 2^x, packed pairs, the lane's sum of the eight; the scores stay where they are"""
    out = [valu(f"v_mov_b32 {vr(PS)}, 0", [], [PS])]
    s_regs = [sc[hb][0] + r for r in range(4)] + [sc[hb][1] + r for r in range(4)]   # p[i]: token block i >> 2, register i & 3
    for i in range(8):
        out.append(valu(f"v_fma_f32 {vr(E + i)}, {vr(s_regs[i])}, %[scale2], {vr(NEGM[hb])}", [s_regs[i], NEGM[hb]], [E + i]))
    for i in range(8):
        out.append(valu(f"v_exp_f32 {vr(E + i)}, {vr(E + i)}", [E + i], [E + i], "trans"))
    for j in range(4):
        out.append(valu(f"v_cvt_pk_bf16_f32 {vr(P[hb] + j)}, {vr(E + 2 * j)}, {vr(E + 2 * j + 1)}", [E + 2 * j, E + 2 * j + 1], [P[hb] + j]))
    for j in range(4):
        out.append(valu(f"v_dot2c_f32_bf16 {vr(PS)}, s{ONES}, {vr(P[hb] + j)}", [P[hb] + j, PS], [PS], "dot"))
    if check:
        out.append(valu(f"v_cmp_nle_f32 vcc, {vr(PS)}, s{LIMIT}", [PS], []))
    return out


def copy_dest(n, fill_slot):
    """m0 = LDS address of copy n of this wave: block wave + 4 n of the slot for n < 9 (36 blocks), the 37th block for
    every wave's last copy (the same bytes four times).  s[CPB] = slot 0 + 1024 * wave."""
    if n < COPIES - 1:
        return Ins(f"s_add_u32 m0, s{CPB}, {fill_slot * SLOT_B + n * 4096}", "salu")
    return Ins(f"s_add_u32 m0, %[slot0], {fill_slot * SLOT_B + (BLOCKS - 1) * 1024}", "salu")


def copy_load(n):
    return Ins(f"global_load_lds_dwordx4 {vr(OFS + n)}, s[{SB}:{SB + 1}]", "vmem", [OFS + n], [])


def copy_group(n, fill_slot):
    """one copy as a self-contained group (a wait state between the write of m0 and its use)"""
    return [copy_dest(n, fill_slot), Ins("s_nop 0", "nop"), copy_load(n)]


def copy_bases(em):
    """once per loop"""
    em.raw(f"s_add_u32 s{CPB}, %[slot0], %[wave_blk]")


def tile_scalars(em, k):
    """s[SB:SB+1] = base of tile t + 3 (page %[pg]); page id of tile t + 4 requested into s[PGN]; once tile t + 3 is
    the row's last tile the copy offsets become the clamped ones"""
    t0, t1, a, b = (f"s{x}" for x in ST)
    em.raw(f"s_lshl_b32 {t0}, %[t], 5")
    em.raw(f"s_add_u32 {t0}, {t0}, %[t_begin]")
    em.raw(f"s_add_u32 {t0}, {t0}, 96")                        # first token of tile t + 3
    em.raw(f"s_cmp_ge_i32 {t0}, %[last_tile_tok]")
    em.raw(f"s_cbranch_scc1 L_lastofs_{k}_%=")
    em.label(f"L_ofs_back_{k}_%=")
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


def lastofs_block(em, k):
    em.label(f"L_lastofs_{k}_%=")
    for n in range(COPIES):
        em.emit(valu(f"v_mov_b32 {vr(OFS + n)}, {vr(OFSL + n)}", [OFSL + n], [OFS + n]))
    em.raw(f"s_branch L_ofs_back_{k}_%=")


def mask_block(em, k, sc, tag):
    """tile t is the segment's first tile or the row's last: scores of tokens before the window's edge or past
    the row's end become -1e30.  Token of score i = 4b + r of lane group g: 32 t + 16 b + 4 g + r (from t_begin);
    LO / HI hold (edge - t_begin - 4 g) and (row end - t_begin - 4 g) per lane."""
    em.label(f"L_mask_{tag}_%=")
    em.raw("s_nop 15", "nop")                                   # the scores come straight from the matrix pipe
    em.raw("s_nop 3", "nop")
    a = f"s{ST[0]}"
    em.raw(f"s_lshl_b32 {a}, %[t], 5")
    em.emit(valu(f"v_subrev_u32 {vr(T0)}, {a}, {vr(LO)}", [LO], [T0]))       # LO - 32 t
    em.emit(valu(f"v_subrev_u32 {vr(T1)}, {a}, {vr(HI)}", [HI], [T1]))       # HI - 32 t
    em.emit(valu(f"v_mov_b32 {vr(A)}, {NEG_BIG}", [], [A]))
    for hb in range(2):
        if hb == 1:
            em.emit(valu(f"v_add_u32 {vr(T1)}, %[hi_step], {vr(T1)}", [T1], [T1]))   # the second block's own row end
        for b in range(2):
            for r in range(4):
                reg = sc[hb][b] + r
                cst = 16 * b + r
                em.emit(valu(f"v_cmp_ge_i32 vcc, {cst}, {vr(T0)}", [T0], []))
                em.emit(valu(f"v_cndmask_b32 {vr(reg)}, {vr(A)}, {vr(reg)}, vcc", [reg, A], [reg]))
                em.emit(valu(f"v_cmp_lt_i32 vcc, {cst}, {vr(T1)}", [T1], []))
                em.emit(valu(f"v_cndmask_b32 {vr(reg)}, {vr(A)}, {vr(reg)}, vcc", [reg, A], [reg]))
    em.raw(f"s_branch L_mask_back_{tag}_%=")


def mask_check(em, tag):
    """detour for the segment's first tile (t == 0) and the masked tail (t >= LASTK)"""
    em.raw("s_cmp_eq_u32 %[t], 0")
    em.raw(f"s_cbranch_scc1 L_mask_{tag}_%=")
    em.raw(f"s_cmp_ge_i32 %[t], s{LASTK}")
    em.raw(f"s_cbranch_scc1 L_mask_{tag}_%=")
    em.label(f"L_mask_back_{tag}_%=")


def rare_block(em, tag, hb, sc):
    """some lane's sum blew up: raise the reference of its head (all four lanes of the head alike) and redo the
    tile's probabilities; twice the raise on every further round"""
    a, b = f"s{ST[0]}", f"s{ST[1]}"
    em.label(f"L_rare_{tag}_%=")
    em.raw(f"s_mov_b32 s{DELTA}, 0x41800000")                   # 16.0
    em.raw(f"s_mov_b32 s{PASS}, 0")
    em.label(f"L_rare_again_{tag}_%=")
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
    em.emit(valu(f"v_sub_f32 {vr(NEGM[hb])}, {vr(NEGM[hb])}, {vr(D)}", [NEGM[hb], D], [NEGM[hb]]))
    em.emit(valu(f"v_add_f32 {vr(M[hb])}, {vr(M[hb])}, {vr(D)}", [M[hb], D], [M[hb]]))
    em.emit(valu(f"v_exp_f32 {vr(A)}, -{vr(D)}", [D], [A], "trans"))
    em.emit(valu(f"v_mul_f32 {vr(L[hb])}, {vr(L[hb])}, {vr(A)}", [L[hb], A], [L[hb]]))
    em.raw("s_nop 15", "nop")                                   # matrix instructions still writing the accumulators
    em.raw("s_nop 15", "nop")
    for r in range(128):
        t = TR[r & 1]
        acc = O[hb] + r
        em.raw(f"v_accvgpr_read_b32 {vr(t)}, {vr(acc)}", "valu")
        em.raw("s_nop 0", "nop")
        em.raw(f"v_mul_f32 {vr(t)}, {vr(t)}, {vr(A)}", "valu")
        em.raw("s_nop 0", "nop")
        em.raw(f"v_accvgpr_write_b32 {vr(acc)}, {vr(t)}", "valu")
    for x in softmax(hb, sc):
        em.emit(x)
    em.raw(f"s_add_u32 s{PASS}, s{PASS}, 1")
    em.raw(f"s_add_u32 s{DELTA}, s{DELTA}, 0x00800000")         # twice the raise next time: exponent + 1
    em.raw(f"s_cmp_ge_u32 s{PASS}, 8")
    em.raw(f"s_cbranch_scc1 L_rare_done_{tag}_%=")
    em.raw(f"s_cbranch_vccnz L_rare_again_{tag}_%=")
    em.label(f"L_rare_done_{tag}_%=")
    em.raw("s_nop 7", "nop")                                    # P and O were written by the vector pipe
    em.raw(f"s_branch L_back_{tag}_%=")


def emit_all(em, items):
    for x in items:
        em.emit(x)


def softmax_and_check(em, k, hb, sc):
    """softmax of one block of heads followed by its rare-path check and the row sum update"""
    if "novalu" not in X:
        emit_all(em, softmax(hb, sc))
        if "norare" not in X:
            em.raw(f"s_cbranch_vccnz L_rare_{k}_{hb}_%=")
    em.label(f"L_back_{k}_{hb}_%=")
    if "novalu" not in X:
        em.emit(valu(f"v_add_f32 {vr(L[hb])}, {vr(L[hb])}, {vr(PS)}", [L[hb], PS], [L[hb]]))


def qk_phase(em, sc, kaddr, copies, extra=None, into_pv=False):
    """the 72 matrix instructions of a tile's scores; copy groups and (pipelined loop) vector work in between.
    `into_pv`: the operand requests run on into the second product's first fragments, which then travel under the
    softmax"""
    extra = list(extra or [])
    copy_at = {2 + 3 * n: n for n in range(COPIES)}
    for f in range(AHEAD):
        emit_all(em, frag_read(f, kaddr))
    for f in range(36):
        cp = copies[copy_at[f]] if (f in copy_at and copies) else None
        if cp:
            em.emit(cp[0])       # m0; the matrix instructions behind it are the wait state its use needs
        for ins in frag_mfmas(f, sc):
            em.emit(ins)
            if extra:
                em.emit(extra.pop(0))
        if f + AHEAD < (68 if into_pv else 36):
            emit_all(em, frag_read(f + AHEAD, kaddr))
        if cp:
            em.emit(cp[1])
    emit_all(em, extra)


def pv_phase(em, prefetched=False):
    if not prefetched:
        for f in range(36, 36 + AHEAD):
            emit_all(em, frag_read(f))
    for f in range(36, 68):
        emit_all(em, frag_mfmas(f, None))
        if f + AHEAD < 68:
            emit_all(em, frag_read(f + AHEAD))


def end_of_step(em):
    # The next step reads tile t + 1 and (pipelined loop) the K rows of tile t + 2: they have landed once only the
    # newest copies -- tile t + 3's ten, plus tile t + 2's in the plain loop -- are outstanding.  Every LDS read of
    # tile t has returned, so its slot may be refilled after the barrier.
    assert not em.lds_queue
    ahead = COPIES if PIPELINED else 2 * COPIES
    em.raw("s_waitcnt lgkmcnt(0)" if "novmwait" in X else f"s_waitcnt vmcnt({ahead}) lgkmcnt(0)", "wait")
    em.raw(f"s_mov_b32 %[pg], s{PGN}")
    if "nobarrier" not in X:
        em.raw("s_barrier")
    em.raw("s_add_u32 %[t], %[t], 1")
    em.raw("s_cmp_lt_i32 %[t], %[t_end]")


def step_plain(em, k):
    """tile t in slot k: scores, softmax, second product; tile t + 3 goes to slot (k + 3) & 3"""
    fill = (k + 3) & 3
    tile_scalars(em, k)
    em.emit(valu(f"v_add_u32 {vr(KADDR)}, {k * SLOT_B}, {vr(KBASE)}", [KBASE], [KADDR]))
    em.emit(valu(f"v_add_u32 {vr(VADDR)}, {k * SLOT_B}, {vr(VBASE)}", [VBASE], [VADDR]))
    copies = [] if "nocopy" in X else [(copy_dest(n, fill), copy_load(n)) for n in range(COPIES)]
    qk_phase(em, SC, KADDR, copies, into_pv=True)
    mask_check(em, f"{k}")
    for hb in range(2):
        softmax_and_check(em, k, hb, SC)
    pv_phase(em, prefetched=True)
    end_of_step(em)


def step_pipelined(em, k):
    """tile t in slot k (scores in set k & 1): scores of tile t + 1 (slot (k + 1) & 3) into the other set,
    interleaved with the softmax of tile t; then the second product of tile t"""
    fill = (k + 3) & 3
    cur, nxt = (SC, SC2) if k % 2 == 0 else (SC2, SC)
    tile_scalars(em, k)
    em.emit(valu(f"v_add_u32 {vr(KADDR2)}, {((k + 1) & 3) * SLOT_B}, {vr(KBASE)}", [KBASE], [KADDR2]))
    em.emit(valu(f"v_add_u32 {vr(VADDR)}, {k * SLOT_B}, {vr(VBASE)}", [VBASE], [VADDR]))
    copies = [] if "nocopy" in X else [copy_group(n, fill) for n in range(COPIES)]
    mask_check(em, f"{k}")
    # the softmax of block 0, its check and the softmax of block 1 ride on the matrix instructions of the next
    # tile's scores; a rare path taken in between leaves and re-enters the instruction stream at its label
    sm0 = [] if "novalu" in X else softmax(0, cur)
    qk_first = 40   # matrix instructions the first softmax is spread over
    copy_at = {2 + 3 * n: n for n in range(COPIES)}
    for f in range(AHEAD):
        emit_all(em, frag_read(f, KADDR2))
    issued = 0
    pending = list(sm0)
    stage = 0
    sm1 = None
    for f in range(36):
        for ins in frag_mfmas(f, nxt):
            em.emit(ins)
            issued += 1
            if pending:
                em.emit(pending.pop(0))
            if stage == 0 and not pending and issued >= len(sm0):
                # the first block's probabilities are complete: check, row sum, then the second block's softmax
                if "novalu" not in X and "norare" not in X:
                    em.raw(f"s_cbranch_vccnz L_rare_{k}_0_%=")
                em.label(f"L_back_{k}_0_%=")
                if "novalu" not in X:
                    em.emit(valu(f"v_add_f32 {vr(L[0])}, {vr(L[0])}, {vr(PS)}", [L[0], PS], [L[0]]))
                    pending = softmax(1, cur)
                stage = 1
        if f + AHEAD < 36:
            emit_all(em, frag_read(f + AHEAD, KADDR2))
        if f in copy_at and copies:
            emit_all(em, copies[copy_at[f]])
    emit_all(em, pending)
    assert stage == 1
    if "novalu" not in X and "norare" not in X:
        em.raw(f"s_cbranch_vccnz L_rare_{k}_1_%=")
    em.label(f"L_back_{k}_1_%=")
    if "novalu" not in X:
        em.emit(valu(f"v_add_f32 {vr(L[1])}, {vr(L[1])}, {vr(PS)}", [L[1], PS], [L[1]]))
    pv_phase(em)
    end_of_step(em)


def generate():
    em = Emitter()
    a = f"s{ST[0]}"
    em.raw("s_waitcnt lgkmcnt(0)", "wait")
    em.raw("s_nop 11", "nop")                                   # the caller's matrix instructions have finished
    em.raw(f"s_mov_b32 s{ONES}, 0x3f803f80")
    em.raw(f"s_mov_b32 s{LIMIT}, 0x43800000")                   # 256.0
    em.raw(f"s_lshl_b32 s{PMASK}, 1, %[pshift]")
    em.raw(f"s_sub_u32 s{PMASK}, s{PMASK}, 1")
    em.raw(f"s_lshl_b32 s{PSTR}, %[row_bytes], %[pshift]")
    em.raw(f"s_sub_u32 s{LASTK}, %[last_tile_tok], %[t_begin]")
    em.raw(f"s_ashr_i32 s{LASTK}, s{LASTK}, 5")                 # the row's last tile, counted from the segment's first
    em.raw(f"s_sub_u32 s{LASTK}, s{LASTK}, %[mask_early]")
    copy_bases(em)
    for hb in range(2):
        em.emit(valu(f"v_mul_f32 {vr(NEGM[hb])}, -1.0, {vr(M[hb])}", [M[hb]], [NEGM[hb]]))
    if PIPELINED:
        # scores of the first tile (slot t & 3) into the set step t reads
        for k in range(4):
            em.raw(f"s_and_b32 {a}, %[t], 3")
            em.raw(f"s_cmp_eq_u32 {a}, {k}")
            em.raw(f"s_cbranch_scc0 L_pre_skip_{k}_%=")
            em.emit(valu(f"v_add_u32 {vr(KADDR2)}, {k * SLOT_B}, {vr(KBASE)}", [KBASE], [KADDR2]))
            qk_phase(em, SC if k % 2 == 0 else SC2, KADDR2, None)
            em.raw("s_waitcnt lgkmcnt(0)", "wait")
            em.lds_queue = []
            em.label(f"L_pre_skip_{k}_%=")
    em.raw(f"s_and_b32 {a}, %[t], 3")
    for k in range(1, 4):
        em.raw(f"s_cmp_eq_u32 {a}, {k}")
        em.raw(f"s_cbranch_scc1 L_step_{k}_%=")
    for k in range(4):
        em.label(f"L_step_{k}_%=")
        (step_pipelined if PIPELINED else step_plain)(em, k)
        if k < 3:
            em.raw("s_cbranch_scc0 L_exit_%=")
        else:
            em.raw("s_cbranch_scc1 L_step_0_%=")
            em.raw("s_branch L_exit_%=")
    for k in range(4):
        cur = SC if (k % 2 == 0 or not PIPELINED) else SC2
        for hb in range(2):
            rare_block(em, f"{k}_{hb}", hb, cur)
        mask_block(em, k, cur, f"{k}")
        lastofs_block(em, k)
    em.label("L_exit_%=")
    em.raw("s_nop 15", "nop")
    em.raw("s_nop 3", "nop")
    return em


def emit_text():
    em = generate()
    n_mfma = sum(1 for i in em.out if i.kind == "mfma")
    n_valu = sum(1 for i in em.out if i.kind in ("valu", "trans", "swap", "dot"))
    pre = "RPA_MLA_WIDE"
    text = (f"// {len(em.out)} lines, {n_mfma} matrix and {n_valu} vector instructions (four unrolled steps, their rare paths "
            f"and masking detours), {em.nops} padding wait states; {NUM_VGPR} vector + 256 accumulation registers\n")
    binds = {f"O{i}": (ACC + 32 * i, 32) for i in range(8)}
    binds.update({"Q0": (0, 32), "Q1": (32, 32), "Q2": (64, 32), "Q3": (96, 32), "Q4": (128, 16),
                  "ML": (ML, 8), "OFS": (OFS, 16), "OFSL": (OFSL, 16)})
    for name, (lo, n) in binds.items():
        text += f'#define {pre}_C_{name} "{{{vr(lo, n)}}}"\n'
    text += (f"#define {pre}_COPIES_AHEAD {COPIES if PIPELINED else 2 * COPIES}"
             "  // copies that may be outstanding when a step starts\n")
    lines = ['    "%s\\n"' % ins.text for ins in em.out]
    text += f"#define {pre}_ASM \\\n" + " \\\n".join(lines) + "\n"
    clob = ['"v%d"' % r for r in list(range(SC[0][0], ML)) + list(range(OFSL + 16, NUM_VGPR))]
    clob += ['"s%d"' % r for r in SGPR_CLOBBERS]
    text += f"#define {pre}_CLOBBERS " + ", ".join(clob) + ', "vcc", "scc", "m0", "memory"\n'
    print(f"MLA wide: {len(em.out)} lines, {n_mfma} MFMAs, {n_valu} vector, {em.nops} padding wait states, {NUM_VGPR} VGPRs")
    return text


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    text = ("// GENERATED by gen_mla_wide_loop.py -- do not edit; edit the generator and run it.\n"
            "// Tile loop of the wide absorbed-MLA kernels: tiles t .. t_end-1 of one wave (two blocks of 16 heads).\n"
            "// The RPA_MLA_WIDE_C_* macros are the register constraints that bind the kernel's variables to the\n"
            "// registers the assembly uses.\n")
    text += emit_text()
    with open(os.path.join(here, "rpa_mla_wide_loop.inc"), "w") as f:
        f.write(text)


if __name__ == "__main__":
    sys.exit(main())
