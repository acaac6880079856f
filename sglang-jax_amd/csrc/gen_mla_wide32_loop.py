#!/usr/bin/env python3
"""Generator of ``rpa_mla_wide32_loop.inc``: the tile loop of the wide absorbed-MLA kernels with 32x32x16
matrix instructions -- the same workgroup (four waves of 32 heads), ring, copies, masks and reference scheme as
gen_mla_wide_loop.py, half the matrix instructions per tile:

    python gen_mla_wide32_loop.py          # rewrites rpa_mla_wide32_loop.inc next to it

A lone wave per SIMD is bound by the number of instructions it issues.  With v_mfma_f32_32x32x16_bf16 a
tile is 36 + 32 matrix instructions instead of 72 + 64, and one lane owns one head:
    scores   S^T[32 tokens x 32 heads] = K . Q^T      36 MFMAs, two interleaved accumulation chains
                                                      (even / odd k-steps: a dependent MFMA would wait)
    softmax  16 scores per lane: s = s_a + s_b, p = 2^(s * scale2 - m), packed pairs, row sum
    output   O^T[512 dims x 32 heads] += V^T . P^T    32 MFMAs (16 blocks of 32 dims x 2 k-steps of 16 tokens)
The S^T result layout (lane = head, registers = tokens 8 (i / 4) + 4 h + i % 4, h = lane / 32) is the B operand
layout of the second product when the 16 tokens of a k-step are taken in that order; the V^T operand is read in
the same order with two transposing LDS reads.  256 accumulators in the accumulation registers, 144 vector
registers of Q^T.
"""

from __future__ import annotations

import os
import sys

sys.dont_write_bytecode = True
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import gen_mla_wide_loop as W  # noqa: E402
from gen_mla_wide_loop import (ACC, COPIES, LIMIT, ONES, DELTA, PASS, LASTK, ML, OFS, OFSL, PMASK, PSTR, ROW_B, SLOT_B, ST,  # noqa: E402
                               SGPR_CLOBBERS, Emitter, Ins, copy_bases, copy_group, emit_all, lastofs_block, rng,
                               tile_scalars, valu, vr)

X = set(os.environ.get("RPA_MLA_WIDE32_X", "").split(","))
NBUF = 6
AHEAD = int(os.environ.get("RPA_MLA_WIDE32_AHEAD", 5))
assert AHEAD < NBUF

O = ACC                      # 16 blocks of 16 accumulators
Q = 0                        # 36 Q^T operands of 4
SA, SB_ = 144, 160           # the two score chains; after the softmax SA holds the scores, SB_ the exponentials
P = 176                      # packed probabilities: k-step kk at P + 4 kk
RING = 184                   # NBUF operand buffers of 4
M, L, KBASE, VBASE, LO, HI = 208, 209, 210, 211, 212, 213
NEGM, PS, KADDR, VADDR, D, A = 226, 227, 228, 229, 230, 231
T0, T1, TR = 242, 243, [244, 245]
NUM_VGPR = 248
NEG_BIG = "0xf149f2ca"       # -1e30


def mfma(dst, a, b, c):
    reads = list(rng(a, 4)) + list(rng(b, 4)) + (list(rng(c, 16)) if c is not None else [])
    if "nomfma" in X:
        return Ins("s_nop 0", "nop")
    ctext = vr(c, 16) if c is not None else "0"
    return Ins(f"v_mfma_f32_32x32x16_bf16 {vr(dst, 16)}, {vr(a, 4)}, {vr(b, 4)}, {ctext}", "mfma", reads, rng(dst, 16))


def ring(f):
    return RING + 4 * (f % NBUF)


def frag_read(f):
    """fragment f: 0..35 K of k-step f (32 tokens x 16 dims); 36..67 V^T of (dim block d, k-step kk), 36 + 2 d + kk"""
    dst = ring(f)
    if "nolds" in X:
        return []
    if f < 36:
        return [Ins(f"ds_read_b128 {vr(dst, 4)}, {vr(KADDR)} offset:{32 * f}", "lds", [KADDR], rng(dst, 4), lds_tag=("k", f))]
    d, kk = (f - 36) >> 1, (f - 36) & 1
    off = 64 * d + 16 * kk * ROW_B
    return [Ins(f"ds_read_b64_tr_b16 {vr(dst, 2)}, {vr(VADDR)} offset:{off}", "lds", [VADDR], rng(dst, 2), lds_tag=("vlo", f)),
            Ins(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, {vr(VADDR)} offset:{off + 8 * ROW_B}", "lds", [VADDR], rng(dst + 2, 2),
                lds_tag=("vhi", f))]


def frag_mfma(f):
    if f < 36:
        chain = SA if f % 2 == 0 else SB_
        ins = mfma(chain, ring(f), Q + 4 * f, None if f < 2 else chain)
        ins.lds_need = None if "nolds" in X else [("k", f)]
    else:
        d, kk = (f - 36) >> 1, (f - 36) & 1
        ins = mfma(O + 16 * d, ring(f), P + 4 * kk, O + 16 * d)
        ins.lds_need = None if "nolds" in X else [("vlo", f), ("vhi", f)]
    return ins


def combine():
    """s = s_a + s_b (kept in SA: the rare path starts from it)"""
    return [valu(f"v_add_f32 {vr(SA + i)}, {vr(SA + i)}, {vr(SB_ + i)}", [SA + i, SB_ + i], [SA + i]) for i in range(16)]


def softmax(check=True):
    """x = s * scale2 - m into SB_, p = 2^x, packed pairs, the lane's sum of the sixteen"""
    out = [valu(f"v_mov_b32 {vr(PS)}, 0", [], [PS])]
    for i in range(16):
        out.append(valu(f"v_fma_f32 {vr(SB_ + i)}, {vr(SA + i)}, %[scale2], {vr(NEGM)}", [SA + i, NEGM], [SB_ + i]))
    for i in range(16):
        out.append(valu(f"v_exp_f32 {vr(SB_ + i)}, {vr(SB_ + i)}", [SB_ + i], [SB_ + i], "trans"))
    for j in range(8):
        out.append(valu(f"v_cvt_pk_bf16_f32 {vr(P + j)}, {vr(SB_ + 2 * j)}, {vr(SB_ + 2 * j + 1)}", [SB_ + 2 * j, SB_ + 2 * j + 1], [P + j]))
    for j in range(8):
        out.append(valu(f"v_dot2c_f32_bf16 {vr(PS)}, s{ONES}, {vr(P + j)}", [P + j, PS], [PS], "dot"))
    if check:
        out.append(valu(f"v_cmp_nle_f32 vcc, {vr(PS)}, s{LIMIT}", [PS], []))
    return out


def mask_block(em, k):
    """first tile of the segment / last tile of the row: token of score i of lane group h is 32 t + 8 (i / 4) + 4 h +
    i % 4 (from t_begin); LO / HI hold (edge - t_begin - 4 h) and (row end - t_begin - 4 h) per lane"""
    em.label(f"L_mask_{k}_%=")
    em.raw("s_nop 15", "nop")
    em.raw("s_nop 7", "nop")
    a = f"s{ST[0]}"
    em.raw(f"s_lshl_b32 {a}, %[t], 5")
    em.emit(valu(f"v_subrev_u32 {vr(T0)}, {a}, {vr(LO)}", [LO], [T0]))
    em.emit(valu(f"v_subrev_u32 {vr(T1)}, {a}, {vr(HI)}", [HI], [T1]))
    em.emit(valu(f"v_mov_b32 {vr(A)}, {NEG_BIG}", [], [A]))
    for i in range(16):
        reg, cst = SA + i, 8 * (i >> 2) + (i & 3)
        em.emit(valu(f"v_cmp_ge_i32 vcc, {cst}, {vr(T0)}", [T0], []))
        em.emit(valu(f"v_cndmask_b32 {vr(reg)}, {vr(A)}, {vr(reg)}, vcc", [reg, A], [reg]))
        em.emit(valu(f"v_cmp_lt_i32 vcc, {cst}, {vr(T1)}", [T1], []))
        em.emit(valu(f"v_cndmask_b32 {vr(reg)}, {vr(A)}, {vr(reg)}, vcc", [reg, A], [reg]))
    em.raw(f"s_branch L_mask_back_{k}_%=")


def rare_block(em, k):
    """some lane's sum blew up: raise the reference of its head (both lanes of the head alike), rescale what has been
    accumulated, redo the tile's probabilities; twice the raise on every further round"""
    a = f"s{ST[0]}"
    em.label(f"L_rare_{k}_%=")
    em.raw(f"s_mov_b32 s{DELTA}, 0x41800000")                   # 16.0
    em.raw(f"s_mov_b32 s{PASS}, 0")
    em.label(f"L_rare_again_{k}_%=")
    em.raw(f"s_or_b32 {a}, vcc_lo, vcc_hi")                     # a head's two lanes are c and c + 32
    em.raw(f"s_mov_b32 vcc_lo, {a}")
    em.raw(f"s_mov_b32 vcc_hi, {a}")
    em.emit(valu(f"v_mov_b32 {vr(A)}, s{DELTA}", [], [A]))
    em.raw("s_nop 1", "nop")
    em.emit(valu(f"v_cndmask_b32 {vr(D)}, 0, {vr(A)}, vcc", [A], [D]))
    em.emit(valu(f"v_sub_f32 {vr(NEGM)}, {vr(NEGM)}, {vr(D)}", [NEGM, D], [NEGM]))
    em.emit(valu(f"v_add_f32 {vr(M)}, {vr(M)}, {vr(D)}", [M, D], [M]))
    em.emit(valu(f"v_exp_f32 {vr(A)}, -{vr(D)}", [D], [A], "trans"))
    em.emit(valu(f"v_mul_f32 {vr(L)}, {vr(L)}, {vr(A)}", [L, A], [L]))
    em.raw("s_nop 15", "nop")                                   # matrix instructions still writing the accumulators
    em.raw("s_nop 15", "nop")
    em.raw("s_nop 15", "nop")
    for r in range(256):
        t = TR[r & 1]
        em.raw(f"v_accvgpr_read_b32 {vr(t)}, {vr(O + r)}", "valu")
        em.raw("s_nop 0", "nop")
        em.raw(f"v_mul_f32 {vr(t)}, {vr(t)}, {vr(A)}", "valu")
        em.raw("s_nop 0", "nop")
        em.raw(f"v_accvgpr_write_b32 {vr(O + r)}, {vr(t)}", "valu")
    emit_all(em, softmax())
    em.raw(f"s_add_u32 s{PASS}, s{PASS}, 1")
    em.raw(f"s_add_u32 s{DELTA}, s{DELTA}, 0x00800000")
    em.raw(f"s_cmp_ge_u32 s{PASS}, 8")
    em.raw(f"s_cbranch_scc1 L_rare_done_{k}_%=")
    em.raw(f"s_cbranch_vccnz L_rare_again_{k}_%=")
    em.label(f"L_rare_done_{k}_%=")
    em.raw("s_nop 7", "nop")
    em.raw(f"s_branch L_back_{k}_%=")


def step(em, k):
    """tile t in slot k: scores, softmax, second product; tile t + 3 goes to slot (k + 3) & 3"""
    fill = (k + 3) & 3
    tile_scalars(em, k)
    em.emit(valu(f"v_add_u32 {vr(KADDR)}, {k * SLOT_B}, {vr(KBASE)}", [KBASE], [KADDR]))
    em.emit(valu(f"v_add_u32 {vr(VADDR)}, {k * SLOT_B}, {vr(VBASE)}", [VBASE], [VADDR]))
    copies = [] if "nocopy" in X else [copy_group(n, fill) for n in range(COPIES)]
    copy_at = {2 + 3 * n: n for n in range(COPIES)}
    for f in range(AHEAD):
        emit_all(em, frag_read(f))
    for f in range(36):
        em.emit(frag_mfma(f))
        if f + AHEAD < 68:
            emit_all(em, frag_read(f + AHEAD))      # the first V^T fragments travel under the last score MFMAs and the softmax
        if f in copy_at and copies:
            emit_all(em, copies[copy_at[f]])
    if "novalu" not in X:
        emit_all(em, combine())
    em.raw("s_cmp_eq_u32 %[t], 0")
    em.raw(f"s_cbranch_scc1 L_mask_{k}_%=")
    em.raw(f"s_cmp_eq_u32 %[t], s{LASTK}")
    em.raw(f"s_cbranch_scc1 L_mask_{k}_%=")
    em.label(f"L_mask_back_{k}_%=")
    if "novalu" not in X:
        emit_all(em, softmax())
        if "norare" not in X:
            em.raw(f"s_cbranch_vccnz L_rare_{k}_%=")
    em.label(f"L_back_{k}_%=")
    if "novalu" not in X:
        em.emit(valu(f"v_add_f32 {vr(L)}, {vr(L)}, {vr(PS)}", [L, PS], [L]))
    for f in range(36, 68):
        em.emit(frag_mfma(f))
        if f + AHEAD < 68:
            emit_all(em, frag_read(f + AHEAD))
    assert not em.lds_queue
    em.raw("s_waitcnt lgkmcnt(0)" if "novmwait" in X else f"s_waitcnt vmcnt({2 * COPIES}) lgkmcnt(0)", "wait")
    em.raw(f"s_mov_b32 %[pg], s{W.PGN}")
    em.raw("s_barrier")
    em.raw("s_add_u32 %[t], %[t], 1")
    em.raw("s_cmp_lt_i32 %[t], %[t_end]")


def generate():
    em = Emitter()
    a = f"s{ST[0]}"
    em.raw("s_waitcnt lgkmcnt(0)", "wait")
    em.raw("s_nop 15", "nop")
    em.raw(f"s_mov_b32 s{ONES}, 0x3f803f80")
    em.raw(f"s_mov_b32 s{LIMIT}, 0x43800000")                   # 256.0
    em.raw(f"s_lshl_b32 s{PMASK}, 1, %[pshift]")
    em.raw(f"s_sub_u32 s{PMASK}, s{PMASK}, 1")
    em.raw(f"s_lshl_b32 s{PSTR}, %[row_bytes], %[pshift]")
    em.raw(f"s_sub_u32 s{LASTK}, %[last_tile_tok], %[t_begin]")
    em.raw(f"s_ashr_i32 s{LASTK}, s{LASTK}, 5")
    copy_bases(em)
    em.emit(valu(f"v_mul_f32 {vr(NEGM)}, -1.0, {vr(M)}", [M], [NEGM]))
    em.raw(f"s_and_b32 {a}, %[t], 3")
    for k in range(1, 4):
        em.raw(f"s_cmp_eq_u32 {a}, {k}")
        em.raw(f"s_cbranch_scc1 L_step_{k}_%=")
    for k in range(4):
        em.label(f"L_step_{k}_%=")
        step(em, k)
        if k < 3:
            em.raw("s_cbranch_scc0 L_exit_%=")
        else:
            em.raw("s_cbranch_scc1 L_step_0_%=")
            em.raw("s_branch L_exit_%=")
    for k in range(4):
        rare_block(em, k)
        mask_block(em, k)
        lastofs_block(em, k)
    em.label("L_exit_%=")
    em.raw("s_nop 15", "nop")
    em.raw("s_nop 15", "nop")
    return em


def emit_text():
    em = generate()
    n_mfma = sum(1 for i in em.out if i.kind == "mfma")
    n_valu = sum(1 for i in em.out if i.kind in ("valu", "trans", "swap", "dot"))
    pre = "RPA_MLA_WIDE32"
    text = (f"// {len(em.out)} lines, {n_mfma} matrix and {n_valu} vector instructions (four unrolled steps, their rare paths "
            f"and masking detours), {em.nops} padding wait states; {NUM_VGPR} vector + 256 accumulation registers\n")
    binds = {f"O{i}": (ACC + 32 * i, 32) for i in range(8)}
    binds.update({"Q0": (0, 32), "Q1": (32, 32), "Q2": (64, 32), "Q3": (96, 32), "Q4": (128, 16),
                  "ML": (ML, 8), "OFS": (OFS, 16), "OFSL": (OFSL, 16)})
    for name, (lo, n) in binds.items():
        text += f'#define {pre}_C_{name} "{{{vr(lo, n)}}}"\n'
    text += f"#define {pre}_COPIES_AHEAD {2 * COPIES}  // copies that may be outstanding when a step starts\n"
    lines = ['    "%s\\n"' % ins.text for ins in em.out]
    text += f"#define {pre}_ASM \\\n" + " \\\n".join(lines) + "\n"
    clob = ['"v%d"' % r for r in list(range(SA, ML)) + list(range(OFSL + 16, NUM_VGPR))]
    clob += ['"s%d"' % r for r in SGPR_CLOBBERS]
    text += f"#define {pre}_CLOBBERS " + ", ".join(clob) + ', "vcc", "scc", "m0", "memory"\n'
    print(f"MLA wide32: {len(em.out)} lines, {n_mfma} MFMAs, {n_valu} vector, {em.nops} padding wait states, {NUM_VGPR} VGPRs")
    return text


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    text = ("// GENERATED by gen_mla_wide32_loop.py -- do not edit; edit the generator and run it.\n"
            "// Tile loop of the wide absorbed-MLA kernels with 32x32x16 matrix instructions: tiles t .. t_end-1 of one\n"
            "// wave (32 heads, one per lane and half).  The RPA_MLA_WIDE32_C_* macros bind the kernel's variables to the\n"
            "// registers the assembly uses.\n")
    text += emit_text()
    with open(os.path.join(here, "rpa_mla_wide32_loop.inc"), "w") as f:
        f.write(text)


if __name__ == "__main__":
    sys.exit(main())
