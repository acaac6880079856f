#!/usr/bin/env python3
"""Generator of ``rpa_prefill_pipe_loop.inc``: the steady-state loop of the pipelined prefill
kernel (rpa_prefill_pipe.hip) as one hand-scheduled gfx950 assembly block.

    python gen_prefill_pipe_loop.py            # rewrites rpa_prefill_pipe_loop.inc next to it

The loop runs "fast steps" of one wave: step t = iterations (2t-1, 2t) over 32-token halves,
    iteration i:  S(i+1) = K(i+1).Q^T   (8 MFMAs)      O += V(i-1)^T.P(i-1)^T   (8 MFMAs)
                  P(i) = bf16(2^(S(i) c - m c)), row sum, row maximum            (vector pipe)
with the matrix and vector instructions interleaved one by one, LDS operands fetched a fixed
number of matrix instructions ahead, the eight global->LDS copy instructions of the step spread
over its first iteration, and one barrier at the end of the step.

The generator keeps three promises the assembler cannot check:
  * every `s_waitcnt lgkmcnt(n)` is computed from the issue order of the LDS reads;
  * the issue distances the hardware does not interlock are verified (and padded with s_nop):
    MFMA result -> vector read/write (11), vector write -> MFMA operand (2), transcendental
    result -> vector read (1), vector write -> v_permlane32_swap (2);
  * register use follows one table (REG) shared with the C++ side through the emitted macros.
"""

from __future__ import annotations

import os
import sys

# ------------------------------------------------------------------ register table (VGPRs)
O = [16 * d for d in range(4)]            # O[d] = v[16d : 16d+15]
S = [64, 80]                              # S0, S1
P = [96, 104]                             # P0, P1 (8 registers each: two B operands)
Q = 112                                   # Q^T operands, 8 x 4 registers
KOFF = 144                                # 8 LDS byte offsets of the K operand reads
VOFF = 152                                # 4 LDS byte offsets of the V^T operand reads
OFSK = 156                                # 4 per-lane global byte offsets of this wave's K copies
OFSV = 160                                # 4 ... V copies
M, L, NEGM, MX, T0, T1, PS0, PS1 = 164, 165, 166, 167, 168, 169, 170, 171
E = 172                                   # 8 temporaries of the exponentials
KF = 180                                  # 4 K fragments x 4 registers
VF = 196                                  # 4 V^T fragments x 4 registers
NUM_VGPR = 212

K_SLOT = [0, 16384]
V_SLOT = [32768, 49152]
HALF = 8192

MFMA_TO_VALU = 11
VALU_TO_MFMA = 2
TRANS_TO_VALU = 1
VALU_TO_SWAP = 2


def vr(lo, n=1):
    return f"v{lo}" if n == 1 else f"v[{lo}:{lo + n - 1}]"


class Ins:
    def __init__(self, text, kind, reads=(), writes=(), lds_tag=None, lds_need=None):
        self.text, self.kind = text, kind
        self.reads, self.writes = set(reads), set(writes)
        self.lds_tag = lds_tag      # this instruction is an LDS read with this tag
        self.lds_need = lds_need    # tags of LDS reads whose data this instruction consumes


def rng(lo, n):
    return range(lo, lo + n)


def mfma(dst, a, b, c):
    """dst/c: base of 16 registers (c None => zero), a/b: base of 4 registers"""
    ctext = "0" if c is None else vr(c, 16)
    reads = list(rng(a, 4)) + list(rng(b, 4)) + ([] if c is None else list(rng(c, 16)))
    return Ins(f"v_mfma_f32_32x32x16_bf16 {vr(dst, 16)}, {vr(a, 4)}, {vr(b, 4)}, {ctext}", "mfma", reads, rng(dst, 16))


def valu(text, reads, writes, kind="valu"):
    return Ins(text, kind, reads, writes)


class Emitter:
    """Collects instructions, inserts LDS waits and hazard padding."""

    def __init__(self):
        self.out = []           # final list of Ins
        self.lds_queue = []     # tags of LDS reads in flight, oldest first
        self.nops = 0

    def _wait_states_since(self, pred):
        """instructions issued since the last instruction satisfying pred (None if never)"""
        n = 0
        for ins in reversed(self.out):
            if pred(ins):
                return n
            n += ins_wait_states(ins)
        return None

    def _pad(self, need, pred, why):
        have = self._wait_states_since(pred)
        if have is not None and have < need:
            k = need - have
            self.out.append(Ins(f"s_nop {k - 1}", "nop"))
            self.nops += k

    def emit(self, ins):
        if ins.kind == "label":
            self.out.append(ins)
            return
        # LDS data dependencies
        if ins.lds_need:
            pos = max(self.lds_queue.index(t) for t in ins.lds_need)
            behind = len(self.lds_queue) - 1 - pos
            assert behind <= 15
            self.out.append(Ins(f"s_waitcnt lgkmcnt({behind})", "wait"))
            self.lds_queue = self.lds_queue[pos + 1:]
        r, w = ins.reads, ins.writes
        if ins.kind in ("valu", "trans", "swap"):
            self._pad(MFMA_TO_VALU, lambda p: p.kind == "mfma" and (p.writes & (r | w)), "mfma->valu")
            self._pad(TRANS_TO_VALU, lambda p: p.kind == "trans" and (p.writes & r), "trans->valu")
            if ins.kind == "swap":
                self._pad(VALU_TO_SWAP, lambda p: p.kind in ("valu", "trans") and (p.writes & r), "valu->swap")
        if ins.kind == "mfma":
            self._pad(VALU_TO_MFMA, lambda p: p.kind in ("valu", "trans", "swap") and (p.writes & r), "valu->mfma")
        if ins.kind in ("lds", "vmem"):
            self._pad(MFMA_TO_VALU, lambda p: p.kind == "mfma" and (p.writes & r), "mfma->mem")
        if ins.lds_tag is not None:
            self.lds_queue.append(ins.lds_tag)
            assert len(self.lds_queue) <= 15, "too many LDS reads in flight"
        self.out.append(ins)

    def drain_lds(self):
        if self.lds_queue:
            self.out.append(Ins("s_waitcnt lgkmcnt(0)", "wait"))
            self.lds_queue = []

    def raw(self, text, kind="salu"):
        self.out.append(Ins(text, kind))

    def label(self, name):
        self.out.append(Ins(f"{name}:", "label"))


def ins_wait_states(ins):
    if ins.kind == "nop":
        return int(ins.text.split()[1]) + 1
    if ins.kind in ("label",):
        return 0
    return 1


# ------------------------------------------------------------------ instruction streams of one iteration
def lds_k(k, slot, half):
    """K fragment of k-step k -> KF[k % 4]"""
    dst = KF + 4 * (k % 4)
    off = K_SLOT[slot] + half * HALF
    return Ins(f"ds_read_b128 {vr(dst, 4)}, {vr(KOFF + k)} offset:{off}", "lds", [KOFF + k], rng(dst, 4), lds_tag=("k", k))


def lds_v(k, slot, half):
    """two transposing reads: V^T fragment of (k-step k >> 2, dim tile k & 3) -> VF[k % 4]"""
    dst = VF + 4 * (k % 4)
    d, kk = k & 3, k >> 2
    off = V_SLOT[slot] + half * HALF + kk * 4096
    return [Ins(f"ds_read_b64_tr_b16 {vr(dst, 2)}, {vr(VOFF + d)} offset:{off}", "lds", [VOFF + d], rng(dst, 2), lds_tag=("vlo", k)),
            Ins(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, {vr(VOFF + d)} offset:{off + 2048}", "lds", [VOFF + d], rng(dst + 2, 2),
                lds_tag=("vhi", k))]


def mfma_qk(k, sn):
    ins = mfma(S[sn], KF + 4 * (k % 4), Q + 4 * k, None if k == 0 else S[sn])
    ins.lds_need = [("k", k)]
    return ins


def mfma_pv(k, pp):
    d, kk = k & 3, k >> 2
    ins = mfma(O[d], VF + 4 * (k % 4), P[pp] + 4 * kk, O[d])
    ins.lds_need = [("vlo", k), ("vhi", k)]
    return ins


def softmax_pair(j, sc, pc, with_max=True):
    """vector work of score pair j of S[sc]: two exponentials, packed into register j of P[pc]"""
    s0, s1 = S[sc] + 2 * j, S[sc] + 2 * j + 1
    e0, e1 = E + 2 * (j % 4), E + 2 * (j % 4) + 1
    w = P[pc] + j
    ps = PS0 + (j & 1)
    out = [
        valu(f"v_fma_f32 {vr(e0)}, {vr(s0)}, %[sc2], {vr(NEGM)}", [s0, NEGM], [e0]),
        valu(f"v_fma_f32 {vr(e1)}, {vr(s1)}, %[sc2], {vr(NEGM)}", [s1, NEGM], [e1]),
        valu(f"v_exp_f32 {vr(e0)}, {vr(e0)}", [e0], [e0], "trans"),
        valu(f"v_exp_f32 {vr(e1)}, {vr(e1)}", [e1], [e1], "trans"),
    ]
    if with_max:
        if j == 0:
            out.append(valu(f"v_max_f32 {vr(MX)}, {vr(s0)}, {vr(s1)}", [s0, s1], [MX]))
        else:
            out.append(valu(f"v_max3_f32 {vr(MX)}, {vr(MX)}, {vr(s0)}, {vr(s1)}", [MX, s0, s1], [MX]))
    out += [
        valu(f"v_cvt_pk_bf16_f32 {vr(w)}, {vr(e0)}, {vr(e1)}", [e0, e1], [w]),
        valu(f"v_dot2c_f32_bf16 {vr(ps)}, {vr(w)}, %[ones]", [w, ps], [ps]),
    ]
    return out


def softmax_tail():
    """row maximum across the two lane halves and the test against the running maximum"""
    return [
        valu(f"v_mov_b32 {vr(T0)}, {vr(MX)}", [MX], [T0]),
        valu(f"v_mov_b32 {vr(T1)}, 0", [], [T1]),  # filler between the write of T0 and the swap
        Ins(f"v_permlane32_swap_b32 {vr(MX)}, {vr(T0)}", "swap", [MX, T0], [MX, T0]),
        valu(f"v_max_f32 {vr(MX)}, {vr(MX)}, {vr(T0)}", [MX, T0], [MX]),
        valu(f"v_sub_f32 {vr(T0)}, {vr(MX)}, {vr(M)}", [MX, M], [T0]),
        valu(f"v_mul_f32 {vr(T0)}, %[sc2], {vr(T0)}", [T0], [T0]),
        valu(f"v_cmp_lt_f32 vcc, %[slack], {vr(T0)}", [T0], []),
    ]


def copy_ins(n, is_v, fill_slot):
    """global -> LDS copy n (0..3) of this wave: 1 KiB block 4*wave + n of the slot"""
    base = (V_SLOT if is_v else K_SLOT)[fill_slot] + n * 1024
    ofs = (OFSV if is_v else OFSK) + n
    sbase = "%[vb_lo]" if is_v else "%[kb_lo]"
    return [Ins(f"s_add_u32 m0, %[lds_wave], {base}", "salu"),
            Ins("s_nop 0", "nop"),
            Ins(f"global_load_lds_dwordx4 {vr(ofs)}, {'%[vb]' if is_v else '%[kb]'}", "vmem", [ofs], [])]


def iteration(em, sc, slot_k, slot_v, half, copies, tag, prefetched):
    """One fast iteration.  S[sc] holds the scores to soften, S[1-sc] receives the next ones,
    P[sc] receives the probabilities, P[1-sc] feeds the second product.
    copies: list of copy instruction groups to spread over the iteration.
    prefetched: number of (K, V) fragment pairs already requested by the caller."""
    sn, pc, pp = 1 - sc, sc, 1 - sc
    AHEAD = 2
    vec = []
    vec.append([valu(f"v_mov_b32 {vr(PS0)}, 0", [], [PS0]), valu(f"v_mov_b32 {vr(PS1)}, 0", [], [PS1])])
    pairs = [softmax_pair(j, sc, pc) for j in range(8)]
    tail = softmax_tail()
    # vector instructions as one list, dealt out behind the matrix instructions
    stream = vec[0] + [x for p_ in pairs for x in p_] + tail
    per_slot = [4] * 16
    extra = len(stream) - sum(per_slot)
    i = 0
    while extra > 0:
        per_slot[i % 16] += 1
        extra -= 1
        i += 2
    pos = 0

    def deal(n):
        nonlocal pos
        for _ in range(n):
            if pos < len(stream):
                em.emit(stream[pos])
                pos += 1

    for k in range(prefetched, AHEAD):
        em.emit(lds_k(k, slot_k, half))
        for x in lds_v(k, slot_v, half):
            em.emit(x)
    for k in range(8):
        if k + AHEAD < 8:
            em.emit(lds_k(k + AHEAD, slot_k, half))
        em.emit(mfma_qk(k, sn))
        deal(per_slot[2 * k])
        if copies:
            for x in copies.pop(0):
                em.emit(x)
        if k + AHEAD < 8:
            for x in lds_v(k + AHEAD, slot_v, half):
                em.emit(x)
        em.emit(mfma_pv(k, pp))
        deal(per_slot[2 * k + 1])
    deal(len(stream))
    assert pos == len(stream)


def rare_block(em, sc, name, back):
    """the row maximum outgrew the stale one: raise it, rescale what is accumulated, redo P(i)"""
    pc = sc
    em.label(name)
    em.raw("s_nop 15", "nop")  # the second product of this iteration is still writing O
    em.emit(valu(f"v_max_f32 {vr(T1)}, {vr(M)}, {vr(MX)}", [M, MX], [T1]))
    em.emit(valu(f"v_sub_f32 {vr(T0)}, {vr(M)}, {vr(T1)}", [M, T1], [T0]))
    em.emit(valu(f"v_mul_f32 {vr(T0)}, %[sc2], {vr(T0)}", [T0], [T0]))
    em.emit(valu(f"v_exp_f32 {vr(T0)}, {vr(T0)}", [T0], [T0], "trans"))
    em.emit(valu(f"v_mov_b32 {vr(M)}, {vr(T1)}", [T1], [M]))
    em.emit(valu(f"v_mul_f32 {vr(NEGM)}, %[nsc2], {vr(T1)}", [T1], [NEGM]))
    em.emit(valu(f"v_mul_f32 {vr(L)}, {vr(L)}, {vr(T0)}", [L, T0], [L]))
    for r in range(64):
        em.emit(valu(f"v_mul_f32 {vr(r)}, {vr(r)}, {vr(T0)}", [r, T0], [r]))
    em.emit(valu(f"v_mov_b32 {vr(PS0)}, 0", [], [PS0]))
    em.emit(valu(f"v_mov_b32 {vr(PS1)}, 0", [], [PS1]))
    for j in range(8):
        for x in softmax_pair(j, sc, pc, with_max=False):
            em.emit(x)
    em.raw("s_nop 1", "nop")  # P(i) was written by the vector pipe; a matrix instruction may follow at once
    em.raw(f"s_branch {back}")


def step(em, par, uid):
    """Fast step with K tile t in K slot `par` and V tile t-1 in V slot 1-par."""
    ks, vs = par, 1 - par
    # ---- copy bases: K tile t+1 uses page pg_b, V tile t page pg_a ----
    em.raw("; ---- step, slot parity %d" % par, "label")
    # tb = t_lo + 64 t; in-page byte offset = (tb & pmask) * tok_stride
    em.raw("s_lshl_b32 %[s0], %[t], 6")
    em.raw("s_add_u32 %[s0], %[s0], %[t_lo]")                 # tb(t)
    em.raw("s_add_u32 %[s1], %[s0], 64")                      # tb(t+1)
    em.raw("s_and_b32 %[s2], %[s0], %[pmask]")
    em.raw("s_mul_i32 %[s2], %[s2], %[tok_stride]")           # in-page bytes of tile t
    em.raw("s_and_b32 %[s3], %[s1], %[pmask]")
    em.raw("s_mul_i32 %[s3], %[s3], %[tok_stride]")           # in-page bytes of tile t+1
    # V base = vh + pg_a * page_stride + s2
    em.raw("s_mul_hi_u32 %[s4], %[pg_a], %[pstr_lo]")
    em.raw("s_mul_i32 %[s5], %[pg_a], %[pstr_hi]")
    em.raw("s_add_u32 %[s4], %[s4], %[s5]")
    em.raw("s_mul_i32 %[s5], %[pg_a], %[pstr_lo]")
    em.raw("s_add_u32 %[s5], %[s5], %[s2]")
    em.raw("s_addc_u32 %[s4], %[s4], 0")
    em.raw("s_add_u32 %[vb_lo], %[vh_lo], %[s5]")
    em.raw("s_addc_u32 %[vb_hi], %[vh_hi], %[s4]")
    # K base = kh + pg_b * page_stride + s3
    em.raw("s_mul_hi_u32 %[s4], %[pg_b], %[pstr_lo]")
    em.raw("s_mul_i32 %[s5], %[pg_b], %[pstr_hi]")
    em.raw("s_add_u32 %[s4], %[s4], %[s5]")
    em.raw("s_mul_i32 %[s5], %[pg_b], %[pstr_lo]")
    em.raw("s_add_u32 %[s5], %[s5], %[s3]")
    em.raw("s_addc_u32 %[s4], %[s4], 0")
    em.raw("s_add_u32 %[kb_lo], %[kh_lo], %[s5]")
    em.raw("s_addc_u32 %[kb_hi], %[kh_hi], %[s4]")
    # page id of tile t+2 (clamped to the last tile of the sequence), consumed at the end of the step
    em.raw("s_add_u32 %[s1], %[s1], 64")
    em.raw("s_min_i32 %[s1], %[s1], %[last_tile_tok]")
    em.raw("s_lshr_b32 %[s1], %[s1], %[pshift]")
    em.raw("s_lshl_b32 %[s1], %[s1], 2")
    em.raw("s_load_dword %[pg_c], %[pages], %[s1]")
    copies = [copy_ins(n, False, 1 - ks) for n in range(4)] + [copy_ins(n, True, 1 - vs) for n in range(4)]
    # ---- iteration 2t-1: softmax of S1, scores into S0, second product with P0 ----
    iteration(em, 1, ks, vs, 0, copies, f"{uid}a", 0)
    assert not copies
    em.raw(f"s_cbranch_vccnz L_rare_{uid}a_%=")
    em.label(f"L_back_{uid}a_%=")
    em.emit(valu(f"v_add_f32 {vr(PS0)}, {vr(PS0)}, {vr(PS1)}", [PS0, PS1], [PS0]))
    em.emit(valu(f"v_add_f32 {vr(L)}, {vr(L)}, {vr(PS0)}", [L, PS0], [L]))
    # ---- iteration 2t: softmax of S0, scores into S1, second product with P1 ----
    iteration(em, 0, ks, vs, 1, [], f"{uid}b", 0)
    em.raw(f"s_cbranch_vccnz L_rare_{uid}b_%=")
    em.label(f"L_back_{uid}b_%=")
    em.emit(valu(f"v_add_f32 {vr(PS0)}, {vr(PS0)}, {vr(PS1)}", [PS0, PS1], [PS0]))
    em.emit(valu(f"v_add_f32 {vr(L)}, {vr(L)}, {vr(PS0)}", [L, PS0], [L]))
    # ---- end of step ----
    em.drain_lds()
    em.raw("s_waitcnt vmcnt(0) lgkmcnt(0)", "wait")
    em.raw("s_mov_b32 %[pg_a], %[pg_b]")
    em.raw("s_mov_b32 %[pg_b], %[pg_c]")
    em.raw("s_barrier")
    em.raw("s_add_u32 %[t], %[t], 1")
    em.raw("s_cmp_lt_i32 %[t], %[t_end]")


def generate():
    em = Emitter()
    em.raw("s_nop 15", "nop")   # matrix instructions issued by the code in front of this block have finished
    em.raw("s_nop 15", "nop")
    em.raw("s_bitcmp1_b32 %[t], 0")
    em.raw("s_cbranch_scc1 L_odd_%=")
    em.label("L_even_%=")
    step(em, 0, "e")
    em.raw("s_cbranch_scc0 L_exit_%=")
    em.label("L_odd_%=")
    step(em, 1, "o")
    em.raw("s_cbranch_scc1 L_even_%=")
    em.raw("s_branch L_exit_%=")
    for uid in ("e", "o"):
        rare_block(em, 1, f"L_rare_{uid}a_%=", f"L_back_{uid}a_%=")
        rare_block(em, 0, f"L_rare_{uid}b_%=", f"L_back_{uid}b_%=")
    em.label("L_exit_%=")
    em.raw("s_nop 15", "nop")   # results of the last matrix instructions are visible to what follows
    em.raw("s_nop 15", "nop")
    return em


def main():
    em = generate()
    here = os.path.dirname(os.path.abspath(__file__))
    lines = []
    for ins in em.out:
        t = ins.text
        lines.append('    "%s\\n"' % t)
    body = "\n".join(lines)
    n_mfma = sum(1 for i in em.out if i.kind == "mfma")
    head = (
        "// GENERATED by gen_prefill_pipe_loop.py -- do not edit; edit the generator and run it.\n"
        "// Steady-state loop of rpa_prefill_pipe_kernel: fast steps t .. t_end-1 of one wave.\n"
        f"// {len(em.out)} lines, {n_mfma} matrix instructions, {em.nops} padding wait states.\n"
        "// Register table (physical VGPRs, shared with rpa_prefill_pipe.hip):\n"
        f"//   O v[0:63]  S0 v[{S[0]}:{S[0]+15}]  S1 v[{S[1]}:{S[1]+15}]  P0 v[{P[0]}:{P[0]+7}]  P1 v[{P[1]}:{P[1]+7}]\n"
        f"//   Q v[{Q}:{Q+31}]  koff v[{KOFF}:{KOFF+7}]  voff v[{VOFF}:{VOFF+3}]  ofs_k v[{OFSK}:{OFSK+3}]  ofs_v v[{OFSV}:{OFSV+3}]\n"
        f"//   m v{M}  l v{L}  -m*c v{NEGM}  scratch v[{MX}:{NUM_VGPR-1}]\n"
    )
    clobbers = ", ".join('"v%d"' % r for r in range(MX, NUM_VGPR))
    text = head + "#define RPA_PIPE_LOOP_ASM \\\n" + "\n".join(l + " \\" for l in lines)[:-2] + "\n"
    text += "#define RPA_PIPE_LOOP_CLOBBERS " + clobbers + ', "vcc", "scc", "m0", "memory"\n'
    with open(os.path.join(here, "rpa_prefill_pipe_loop.inc"), "w") as f:
        f.write(text)
    print(f"wrote rpa_prefill_pipe_loop.inc: {len(em.out)} lines, {n_mfma} MFMAs, {em.nops} padding wait states")


if __name__ == "__main__":
    sys.exit(main())
