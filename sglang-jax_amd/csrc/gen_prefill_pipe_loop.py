#!/usr/bin/env python3
"""Generator of ``rpa_prefill_pipe_loop.inc``: the steady-state loop of the pipelined prefill
kernel (rpa_prefill_pipe.hip) as hand-scheduled gfx950 assembly, for NQ = 1 and NQ = 2 blocks of
32 query rows per wave.

    python gen_prefill_pipe_loop.py            # rewrites rpa_prefill_pipe_loop.inc next to it

The loop runs steps t .. t_end-1 of one wave.  A step covers one 64-token K/V tile as two
iterations over 32-token halves; per block of 32 query rows:
    iteration i:  S(i+1) = K(i+1).Q^T - m   (8 MFMAs)   O += V(i-1)^T.P(i-1)^T   (8 MFMAs)
                  P(i) = bf16(2^S(i)), row sum                                    (vector pipe)
The queries are pre-multiplied by sm_scale * log2(e), and the first MFMA of a score chain takes
the negated running maximum as its C operand (a 16-register splat), so a score leaves the matrix
pipe ready for v_exp_f32: the vector pipe spends one instruction per score plus one per pair
(packing) and one per pair (row sum).  With two blocks of rows per wave every K and V^T fragment
read from LDS feeds two MFMAs.  The matrix and vector instructions are interleaved one by one, LDS
operands are fetched a fixed number of fragments ahead, the eight global -> LDS copy instructions of
the step (K tile t+1, V tile t) are spread over its first iteration, one barrier ends the step.

The running maximum is checked after the fact: a half's probabilities are taken against the
maximum known before it; if some row sum of the half exceeds 2^8 (a score beat the stale maximum
by more than 4) the wave takes the rare path: the true maximum is taken, accumulators, row sums,
the splat and the scores in flight are moved to it and the half's probabilities redone.

A second variant of the loop (masked = True, one block of rows per wave only) applies the causal mask to every
half before its exponentials: one compare of the register's token offset against a per-lane threshold
(query position - first token of the half - 4 * lane half) and one select of -1e30 per score.  It runs the
steps that touch the causal diagonal, which would otherwise fall back to the compiled general step.

The whole loop is one block because the register allocator will not keep hundreds of registers in
place around a block that is only a loop body: here they are moved in and out once per loop.

The generator keeps three promises the assembler cannot check:
  * every `s_waitcnt lgkmcnt(n)` is computed from the issue order of the LDS reads (the one scalar
    load in flight only makes the counted waits longer, never shorter);
  * the issue distances the hardware does not interlock are verified (and padded with s_nop):
    MFMA result -> vector read/write (12), vector write -> MFMA operand (2), transcendental
    result -> vector read (1), vector write -> v_permlane32_swap (2), dot-product result -> any other
    vector instruction (3), scalar write of m0 -> copy (1);
  * register use follows one table shared with the C++ side through the emitted macros.
"""

from __future__ import annotations

import os
import sys

ACC = 1000                                # register ids >= ACC name accumulation registers a[id - ACC]
# Experiment switches (timing probes only: results are wrong with any of them set)
X = set(os.environ.get("RPA_PIPE_X", "").split(","))
AHEAD = int(os.environ.get("RPA_PIPE_AHEAD", 3))   # fragments requested ahead of the MFMAs that use them
STAGGER = int(os.environ.get("RPA_PIPE_STAGGER", 4))  # matrix slots a wave spreads its copies over (with X = stagger)
NBUF = 4                                  # operand fragment buffers per matrix

# scalar registers used inside the block (all listed as clobbers)
KB, VB = 60, 62                           # s[60:61], s[62:63]: global base of the K / V tile being copied
ST = [64, 65, 66, 67]                     # temporaries
PGC = 68                                  # page id of tile t + 2
WV = 69                                   # this wave's index in its workgroup (staggered copies)
MASK_SGPR = [70, 72, 74, 76]              # s[70:71] .. s[76:77]: lane masks of the masked variant
SGPR_BASE = 5000                          # register ids >= SGPR_BASE name scalar registers in the hazard bookkeeping
SGPR_CLOBBERS = list(range(60, 70 if "stagger" in X else 69))

K_SLOT = [0, 16384]                       # byte offsets of the ring slots from the LDS array's start
V_SLOT = [32768, 49152]
V_READ = [0, 16384]                       # ... of the V slots from the addresses in VOFF (which point into V slot 0)
HALF = 8192

MFMA_TO_VALU = 12
VALU_TO_MFMA = 2
TRANS_TO_VALU = 1
VALU_TO_SWAP = 2
DOT_TO_VALU = 3
VALU_SGPR_TO_VALU = 2                     # a vector instruction's scalar result read by a vector instruction


class Table:
    """Register table of one NQ variant."""

    def __init__(self, nq, masked=False):
        self.nq = nq
        self.masked = masked
        self._v, self._a = 0, ACC

        def v(n):
            lo = self._v
            self._v += n
            return lo

        def a(n):
            # one block of rows fits the 256 vector registers of a wave at two waves per SIMD (and leaves the
            # compiler all of them outside the loop); two blocks need the accumulation registers as well
            if nq == 1:
                return v(n)
            lo = self._a
            self._a += n
            return lo

        self.O = [[a(16) for d in range(4)] for q in range(nq)]    # accumulators: only matrix instructions touch them
        self.Q = [a(32) for q in range(nq)]                        # Q^T operands, 8 x 4 registers
        self.KF = a(4 * NBUF)                                      # K fragments, 4 registers each
        self.VF = a(4 * NBUF)                                      # V^T fragments
        self.S = [[v(16), v(16)] for q in range(nq)]               # scores of the even / odd half in flight
        self.P = [[v(8), v(8)] for q in range(nq)]                 # probabilities of the even / odd half
        self.NM = [v(16) for q in range(nq)]                       # minus the running maximum, 16 times
        self.M = [v(1) for q in range(nq)]                         # running maximum (log2 units)
        self.L = [v(1) for q in range(nq)]                         # running sum
        self.KOFF = v(8)                                           # LDS byte addresses of the K operand reads
        self.VOFF = v(4)                                           # ... of the V^T operand reads
        self.OFSK = v(4)                                           # per-lane global byte offsets of this wave's K copies
        self.OFSV = v(4)
        if masked:
            self.THR = v(1)                                        # query position - first token of the half - 4 * lane half
            self.NINF = v(1)                                       # -1e30
        self.first_scratch = self._v
        self.PS = [[v(1), v(1)] for q in range(nq)]                # row-sum accumulators of the half
        self.MX, self.T0, self.T1 = v(1), v(1), v(1)
        self.E = [v(8) for q in range(nq)]                         # temporaries of the exponentials
        self.num_vgpr = self._v
        self.num_agpr = self._a - ACC


def vr(lo, n=1):
    f, lo = ("a", lo - ACC) if lo >= ACC else ("v", lo)
    return f"{f}{lo}" if n == 1 else f"{f}[{lo}:{lo + n - 1}]"


def rng(lo, n):
    return range(lo, lo + n)


class Ins:
    def __init__(self, text, kind, reads=(), writes=(), lds_tag=None, lds_need=None):
        self.text, self.kind = text, kind
        self.reads, self.writes = set(reads), set(writes)
        self.lds_tag = lds_tag      # this instruction is an LDS read with this tag
        self.lds_need = lds_need    # tags of LDS reads whose data this instruction consumes


def wait_states(ins):
    if ins.kind == "nop":
        return int(ins.text.split()[1]) + 1
    if ins.kind in ("label", "skip"):  # "skip": inside a branch some waves jump over: counts for nothing
        return 0
    return 1


class Emitter:
    """Collects instructions, inserts LDS waits and hazard padding."""

    def __init__(self):
        self.out = []
        self.lds_queue = []     # tags of LDS reads in flight, oldest first
        self.nops = 0

    def _since(self, pred):
        n = 0
        for ins in reversed(self.out):
            if pred(ins):
                return n
            n += wait_states(ins)
        return None

    def _pad(self, need, pred):
        have = self._since(pred)
        if have is not None and have < need:
            k = need - have
            self.out.append(Ins(f"s_nop {k - 1}", "nop"))
            self.nops += k

    def emit(self, ins):
        need = [t for t in (ins.lds_need or []) if t in self.lds_queue]
        if need:
            pos = max(self.lds_queue.index(t) for t in need)
            behind = len(self.lds_queue) - 1 - pos
            assert behind <= 15
            self.out.append(Ins(f"s_waitcnt lgkmcnt({behind})", "wait"))
            self.lds_queue = self.lds_queue[pos + 1:]
        r, w = ins.reads, ins.writes
        if ins.kind in ("valu", "trans", "swap", "dot"):
            sr = {x for x in r if x >= SGPR_BASE}
            if sr:
                self._pad(VALU_SGPR_TO_VALU, lambda p: p.kind in ("valu", "trans", "swap", "dot") and (p.writes & sr))
            self._pad(MFMA_TO_VALU, lambda p: p.kind == "mfma" and (p.writes & (r | w)))
            self._pad(TRANS_TO_VALU, lambda p: p.kind == "trans" and (p.writes & r))
            if ins.kind == "swap":
                self._pad(VALU_TO_SWAP, lambda p: p.kind in ("valu", "trans", "dot") and (p.writes & r))
            if ins.kind != "dot":  # a dot instruction accumulates into the previous one's result at once; nothing else may touch it yet
                self._pad(DOT_TO_VALU, lambda p: p.kind == "dot" and (p.writes & (r | w)))
        if ins.kind == "mfma":
            self._pad(VALU_TO_MFMA, lambda p: p.kind in ("valu", "trans", "swap", "dot") and (p.writes & r))
        if ins.kind in ("lds", "vmem"):
            self._pad(MFMA_TO_VALU, lambda p: p.kind == "mfma" and (p.writes & r))
        if ins.lds_tag is not None:
            self.lds_queue.append(ins.lds_tag)
            assert len(self.lds_queue) <= 15, "too many LDS reads in flight"
        self.out.append(ins)

    def raw(self, text, kind="salu"):
        self.out.append(Ins(text, kind))

    def label(self, name):
        self.out.append(Ins(f"{name}:", "label"))


def valu(text, reads, writes, kind="valu"):
    return Ins(text, kind, reads, writes)


class Gen:
    def __init__(self, nq, masked=False):
        assert not (masked and nq != 1)
        self.nq = nq
        self.masked = masked
        self.t = Table(nq, masked)

    # ---------------------------------------------------------------- instruction builders
    def mfma(self, dst, a, b, c):
        reads = list(rng(a, 4)) + list(rng(b, 4)) + list(rng(c, 16))
        if "nomfma" in X:
            return Ins("s_nop 0", "nop")
        return Ins(f"v_mfma_f32_32x32x16_bf16 {vr(dst, 16)}, {vr(a, 4)}, {vr(b, 4)}, {vr(c, 16)}", "mfma", reads, rng(dst, 16))

    def lds_k(self, f, slot):
        """K fragment f (0..15: half f // 8, k-step f % 8) -> KF[f % NBUF]"""
        t = self.t
        k, half = f % 8, f // 8
        dst = t.KF + 4 * (f % NBUF)
        off = K_SLOT[slot] + half * HALF
        return [Ins(f"ds_read_b128 {vr(dst, 4)}, {vr(t.KOFF + k)} offset:{off}", "lds", [t.KOFF + k], rng(dst, 4), lds_tag=("k", f))]

    def lds_v(self, f, slot):
        """two transposing reads: V^T fragment f (half f // 8, k-step (f % 8) >> 2, dim tile f & 3) -> VF[f % NBUF]"""
        t = self.t
        k, half = f % 8, f // 8
        dst = t.VF + 4 * (f % NBUF)
        d, kk = k & 3, k >> 2
        off = V_READ[slot] + half * HALF + kk * 4096
        return [Ins(f"ds_read_b64_tr_b16 {vr(dst, 2)}, {vr(t.VOFF + d)} offset:{off}", "lds", [t.VOFF + d], rng(dst, 2), lds_tag=("vlo", f)),
                Ins(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, {vr(t.VOFF + d)} offset:{off + 2048}", "lds", [t.VOFF + d],
                    rng(dst + 2, 2), lds_tag=("vhi", f))]

    def mfma_qk(self, f, q, sn):
        t = self.t
        k = f % 8
        ins = self.mfma(t.S[q][sn], t.KF + 4 * (f % NBUF), t.Q[q] + 4 * k, t.NM[q] if k == 0 else t.S[q][sn])
        ins.lds_need = None if "nolds" in X else [("k", f)]
        return ins

    def mfma_pv(self, f, q, pp):
        t = self.t
        k = f % 8
        d, kk = k & 3, k >> 2
        ins = self.mfma(t.O[q][d], t.VF + 4 * (f % NBUF), t.P[q][pp] + 4 * kk, t.O[q][d])
        ins.lds_need = None if "nolds" in X else [("vlo", f), ("vhi", f)]
        return ins

    def softmax_ops(self, q, sc):
        """The vector work of the 16 scores of S[q][sc] as three stages per score pair j: the two
        exponentials, the packing into register j of P[q][sc], the row-sum update."""
        t = self.t

        def exps(j):
            s0, s1 = t.S[q][sc] + 2 * j, t.S[q][sc] + 2 * j + 1
            e0, e1 = t.E[q] + 2 * (j % 4), t.E[q] + 2 * (j % 4) + 1
            return [valu(f"v_exp_f32 {vr(e0)}, {vr(s0)}", [s0], [e0], "trans"),
                    valu(f"v_exp_f32 {vr(e1)}, {vr(s1)}", [s1], [e1], "trans")]

        def cvt(j):
            e0, e1 = t.E[q] + 2 * (j % 4), t.E[q] + 2 * (j % 4) + 1
            return [valu(f"v_cvt_pk_bf16_f32 {vr(t.P[q][sc] + j)}, {vr(e0)}, {vr(e1)}", [e0, e1], [t.P[q][sc] + j])]

        def dot(j):
            w, ps = t.P[q][sc] + j, t.PS[q][j & 1]
            return [valu(f"v_dot2c_f32_bf16 {vr(ps)}, %[ones], {vr(w)}", [w, ps], [ps], "dot")]

        return exps, cvt, dot

    def mask_ops(self, q, sc):
        """Causal mask of the 16 scores of S[q][sc], per score pair j: the two compares (token offset of the
        register inside the half against the lane's threshold) into a pair of scalar registers each, and the two
        selects.  The compares of a pair are issued one pair ahead of its selects."""
        t = self.t

        def cmps(j):
            out = []
            for e in (0, 1):
                v = 2 * j + e
                k = 8 * (v >> 2) + (v & 3)
                sg = MASK_SGPR[2 * (j & 1) + e]
                out.append(valu(f"v_cmp_gt_i32_e64 s[{sg}:{sg + 1}], {k}, {vr(t.THR)}", [t.THR], [SGPR_BASE + sg]))
            return out

        def sels(j):
            out = []
            for e in (0, 1):
                v = 2 * j + e
                sg = MASK_SGPR[2 * (j & 1) + e]
                r = t.S[q][sc] + v
                out.append(valu(f"v_cndmask_b32_e64 {vr(r)}, {vr(r)}, {vr(t.NINF)}, s[{sg}:{sg + 1}]",
                                [r, t.NINF, SGPR_BASE + sg], [r]))
            return out

        return cmps, sels

    def softmax_stream(self, sc, check=True, masked=False):
        """All row blocks' softmax work in issue order.  The stages of a pair are spread out (packing
        `lag` pairs behind the exponentials, the row sum one pair behind the packing) and the row blocks
        are interleaved, so no instruction needs the result of the few in front of it: a wave issues in
        order, and a vector instruction that waits holds up the matrix instructions behind it."""
        t, nq = self.t, self.nq
        lag = 2 if nq == 1 else 1
        out = []
        ops = [self.softmax_ops(q, sc) for q in range(nq)]
        for q in range(nq):
            out += [valu(f"v_mov_b32 {vr(t.PS[q][0])}, 0", [], [t.PS[q][0]]), valu(f"v_mov_b32 {vr(t.PS[q][1])}, 0", [], [t.PS[q][1]])]
        if masked:
            cmps, sels = self.mask_ops(0, sc)
            out = cmps(0) + out
        for step in range(8 + lag + 1):
            if masked and step < 8:
                if step + 1 < 8:
                    out += cmps(step + 1)
                else:  # the last compares of the half are out: the threshold moves on to the next half
                    out.append(valu(f"v_subrev_u32_e32 {vr(t.THR)}, 32, {vr(t.THR)}", [t.THR], [t.THR]))
                out += sels(step)
            for q in range(nq):
                if step < 8:
                    out += ops[q][0](step)
            for q in range(nq):
                if 0 <= step - lag < 8:
                    out += ops[q][1](step - lag)
            for q in range(nq):
                if 0 <= step - lag - 1 < 8:
                    out += ops[q][2](step - lag - 1)
        for q in range(nq):
            out.append(valu(f"v_add_f32 {vr(t.PS[q][0])}, {vr(t.PS[q][0])}, {vr(t.PS[q][1])}", t.PS[q], [t.PS[q][0]]))
        if not check:
            return out
        # any row sum of the half above the limit (or not a number)?
        if nq == 2:
            out.append(valu(f"v_max_f32 {vr(t.T0)}, {vr(t.PS[0][0])}, {vr(t.PS[1][0])}", [t.PS[0][0], t.PS[1][0]], [t.T0]))
            out.append(valu(f"v_cmp_nle_f32 vcc, {vr(t.T0)}, %[limit]", [t.T0], []))
        else:
            out.append(valu(f"v_cmp_nle_f32 vcc, {vr(t.PS[0][0])}, %[limit]", [t.PS[0][0]], []))
        return out

    def copy_ins(self, n, is_v, fill_slot):
        """global -> LDS copy n (0..3) of this wave: 1 KiB block 4*wave + n of the slot"""
        t = self.t
        base = (V_SLOT if is_v else K_SLOT)[fill_slot] + n * 1024
        ofs = (t.OFSV if is_v else t.OFSK) + n
        sb = VB if is_v else KB
        if "copyexec0" in X:  # probe: the instruction is issued, no lane moves data
            return [Ins(f"s_add_u32 m0, %[lds_wave], {base}", "salu"),
                    Ins("s_mov_b64 exec, 0", "salu"),
                    Ins(f"global_load_lds_dwordx4 {vr(ofs)}, s[{sb}:{sb + 1}]", "vmem", [ofs], []),
                    Ins("s_mov_b64 exec, -1", "salu")]
        return [Ins(f"s_add_u32 m0, %[lds_wave], {base}", "salu"),
                Ins("s_nop 0", "nop"),
                Ins(f"global_load_lds_dwordx4 {vr(ofs)}, s[{sb}:{sb + 1}]", "vmem", [ofs], [])]

    # ---------------------------------------------------------------- one iteration
    def iteration(self, em, it, ks, vs, copies, uid=""):
        """Iteration `it` (0 / 1) of a step.  it = 0: softmax of the odd-half scores into the odd-half
        probabilities, scores of the tile's first half into the even buffers, second product with the
        even-half probabilities; it = 1: the mirror image on the tile's second half."""
        nq = self.nq
        sc = 1 - it
        sn, pp = 1 - sc, 1 - sc
        stream = self.softmax_stream(sc, masked=self.masked)
        pos = 0

        def deal(n):
            nonlocal pos
            for _ in range(n):
                if pos < len(stream):
                    if "novalu" not in X:
                        em.emit(stream[pos])
                    pos += 1

        def frag_reads(which, f):
            if f >= 16 or "nolds" in X:
                return
            for x in (self.lds_k(f, ks) if which == "k" else self.lds_v(f, vs)):
                em.emit(x)

        # the first iteration's scores were finished in the previous step: a first chunk of vector work
        # runs while the step's first fragments travel; the rest is dealt out behind the matrix instructions
        lead = (12 if self.masked else 6) if it == 0 else 0
        deal(lead)
        slots = 16 * nq
        rest = len(stream) - lead
        per = [rest // slots] * slots
        rem = rest - sum(per)
        for i in range(rem):
            per[(i * slots) // rem] += 1
        s = 0
        for k in range(8):
            f = 8 * it + k
            for q in range(nq):
                em.emit(self.mfma_qk(f, q, sn))
                if q == nq - 1:
                    frag_reads("k", f + AHEAD)
                deal(per[s])
                s += 1
            for q in range(nq):
                em.emit(self.mfma_pv(f, q, pp))
                if q == nq - 1:
                    frag_reads("v", f + AHEAD)
                    if copies and "stagger" in X:
                        # wave w of the workgroup issues its eight copies at matrix slots 4w .. 4w+3 of the
                        # step (two per slot): the four waves never queue for the texture path together
                        j = 8 * it + k
                        if j < 4 * STAGGER:
                            per_slot = 8 // STAGGER
                            em.raw(f"s_cmp_eq_u32 s{WV}, {j // STAGGER}", "skip")
                            em.raw(f"s_cbranch_scc0 L_nc_{uid}{j}_%=", "skip")
                            for g in range(per_slot * (j % STAGGER), per_slot * (j % STAGGER + 1)):
                                for x in copies[g]:
                                    em.raw(x.text, "skip")
                            em.label(f"L_nc_{uid}{j}_%=")
                    elif copies:
                        for x in copies.pop(0):
                            em.emit(x)
                deal(per[s])
                s += 1
        deal(len(stream))
        assert pos == len(stream)

    def rare_block(self, em, it, name, back):
        """some row sum blew up: take the true maxima, move everything to them, redo the half's probabilities"""
        t = self.t
        sc, sn = 1 - it, it
        em.label(name)
        em.raw("s_nop 15", "nop")  # the matrix instructions of this iteration are still writing O and the new scores
        for q in range(self.nq):
            S = t.S[q][sc]
            em.emit(valu(f"v_max3_f32 {vr(t.MX)}, {vr(S)}, {vr(S + 1)}, {vr(S + 2)}", [S, S + 1, S + 2], [t.MX]))
            for v in range(3, 15, 2):
                em.emit(valu(f"v_max3_f32 {vr(t.MX)}, {vr(t.MX)}, {vr(S + v)}, {vr(S + v + 1)}", [t.MX, S + v, S + v + 1], [t.MX]))
            em.emit(valu(f"v_max_f32 {vr(t.MX)}, {vr(t.MX)}, {vr(S + 15)}", [t.MX, S + 15], [t.MX]))
            em.emit(valu(f"v_mov_b32 {vr(t.T0)}, {vr(t.MX)}", [t.MX], [t.T0]))
            em.emit(valu(f"v_mov_b32 {vr(t.T1)}, 0", [], [t.T1]))
            em.emit(Ins(f"v_permlane32_swap_b32 {vr(t.MX)}, {vr(t.T0)}", "swap", [t.MX, t.T0], [t.MX, t.T0]))
            em.emit(valu(f"v_max3_f32 {vr(t.MX)}, {vr(t.MX)}, {vr(t.T0)}, 0", [t.MX, t.T0], [t.MX]))   # d >= 0: the maximum only rises
            em.emit(valu(f"v_add_f32 {vr(t.M[q])}, {vr(t.M[q])}, {vr(t.MX)}", [t.M[q], t.MX], [t.M[q]]))
            em.emit(valu(f"v_exp_f32 {vr(t.T0)}, -{vr(t.MX)}", [t.MX], [t.T0], "trans"))                 # 2^-d
            em.emit(valu(f"v_mul_f32 {vr(t.L[q])}, {vr(t.L[q])}, {vr(t.T0)}", [t.L[q], t.T0], [t.L[q]]))
            for r in [o + v for o in t.O[q] for v in range(16)]:
                if r >= ACC:
                    em.emit(valu(f"v_accvgpr_read_b32 {vr(t.T1)}, {vr(r)}", [r], [t.T1]))
                    em.emit(valu(f"v_mul_f32 {vr(t.T1)}, {vr(t.T1)}, {vr(t.T0)}", [t.T1, t.T0], [t.T1]))
                    em.emit(valu(f"v_accvgpr_write_b32 {vr(r)}, {vr(t.T1)}", [t.T1], [r]))
                else:
                    em.emit(valu(f"v_mul_f32 {vr(r)}, {vr(r)}, {vr(t.T0)}", [r, t.T0], [r]))
            for base in (t.NM[q], t.S[q][sc], t.S[q][sn]):
                for v in range(16):
                    em.emit(valu(f"v_sub_f32 {vr(base + v)}, {vr(base + v)}, {vr(t.MX)}", [base + v, t.MX], [base + v]))
        for x in self.softmax_stream(sc, check=False):
            em.emit(x)
        em.raw("s_nop 3", "nop")  # P, NM and O were written by the vector pipe; a matrix instruction may follow at once
        em.raw(f"s_branch {back}")

    def tile_base(self, em, dst, pg, tb_reg, head_lo, head_hi):
        """s[dst:dst+1] = head + pg * page_stride + (tb & (page_size - 1)) * tok_stride"""
        a, b = f"s{ST[2]}", f"s{ST[3]}"
        em.raw(f"s_and_b32 {a}, {tb_reg}, %[pmask]")
        em.raw(f"s_mul_i32 {a}, {a}, %[tok_stride]")              # bytes inside the page (< 2^32)
        em.raw(f"s_mul_hi_u32 {b}, {pg}, %[pstr]")
        em.raw(f"s_mul_i32 s{dst}, {pg}, %[pstr]")
        em.raw(f"s_add_u32 s{dst}, s{dst}, {a}")
        em.raw(f"s_addc_u32 {b}, {b}, 0")
        em.raw(f"s_add_u32 s{dst}, s{dst}, {head_lo}")
        em.raw(f"s_addc_u32 s{dst + 1}, {b}, {head_hi}")

    def step(self, em, par, uid):
        """Step with K tile t in K slot `par` and V tile t-1 in V slot 1-par; fills K slot 1-par with
        tile t+1 (page pg_b) and V slot par with tile t (page pg_a)."""
        t = self.t
        ks, vs = par, 1 - par
        t0, t1 = f"s{ST[0]}", f"s{ST[1]}"
        em.raw(f"s_lshl_b32 {t0}, %[t], 6")
        em.raw(f"s_add_u32 {t0}, {t0}, %[t_lo]")                   # first token of tile t
        em.raw(f"s_add_u32 {t1}, {t0}, 64")                        # ... of tile t + 1
        self.tile_base(em, VB, "%[pg_a]", t0, "%[vh_lo]", "%[vh_hi]")
        self.tile_base(em, KB, "%[pg_b]", t1, "%[kh_lo]", "%[kh_hi]")
        # page id of tile t + 2 (clamped to the sequence's last tile), consumed at the end of the step
        em.raw(f"s_add_u32 {t1}, {t1}, 64")
        em.raw(f"s_min_i32 {t1}, {t1}, %[last_tile_tok]")
        em.raw(f"s_lshr_b32 {t1}, {t1}, %[pshift]")
        em.raw(f"s_lshl_b32 {t1}, {t1}, 2")
        em.raw(f"s_load_dword s{PGC}, %[pages], {t1}")
        if "nolds" not in X:
            for f in range(AHEAD):
                for x in self.lds_k(f, ks) + self.lds_v(f, vs):
                    em.emit(x)
        copies = [self.copy_ins(n, False, 1 - ks) for n in range(4)] + [self.copy_ins(n, True, 1 - vs) for n in range(4)]
        if "nocopy" in X:
            copies = []
        if "halfcopy" in X:  # probe: half of the tile bytes (what a tile shared by 256 rows would move per wave)
            copies = [c if i % 2 == 0 else [] for i, c in enumerate(copies)]
        if "copyfirst" in X:
            for grp in copies:
                for x in grp:
                    em.emit(x)
            copies = []
        if "stagger" in X:
            em.raw(f"s_bfe_u32 s{WV}, %[lds_wave], 0x2000c")      # (lds_wave >> 12) & 3
        for it in (0, 1):
            self.iteration(em, it, ks, vs, copies, uid)
            tag = uid + "ab"[it]
            if "norare" not in X:
                em.raw(f"s_cbranch_vccnz L_rare_{tag}_%=")
            em.label(f"L_back_{tag}_%=")
            for q in range(self.nq):
                em.emit(valu(f"v_add_f32 {vr(t.L[q])}, {vr(t.L[q])}, {vr(t.PS[q][0])}", [t.L[q], t.PS[q][0]], [t.L[q]]))
        assert ("stagger" in X or not copies) and not em.lds_queue
        # ---- end of step: the copies have landed, everybody has finished reading the slots they overwrite next
        em.raw("s_waitcnt lgkmcnt(0)" if "novmwait" in X else "s_waitcnt vmcnt(0) lgkmcnt(0)", "wait")
        if "copysame" not in X:  # probe: every step copies the same pages (cache hits)
            em.raw("s_mov_b32 %[pg_a], %[pg_b]")
            em.raw(f"s_mov_b32 %[pg_b], s{PGC}")
        if "nobarrier" not in X:
            em.raw("s_barrier")
        em.raw("s_add_u32 %[t], %[t], 1")
        em.raw("s_cmp_lt_i32 %[t], %[t_end]")

    def generate(self):
        em = Emitter()
        # Nothing of the caller's is in flight on the LDS / scalar-memory counter.  Matrix instructions the
        # caller issued before this block have finished: a barrier and this block's entry moves lie in between.
        em.raw("s_waitcnt lgkmcnt(0)", "wait")
        em.raw("s_nop 11", "nop")
        em.raw("s_bitcmp1_b32 %[t], 0")
        em.raw("s_cbranch_scc1 L_odd_%=")
        em.label("L_even_%=")
        self.step(em, 0, "e")
        em.raw("s_cbranch_scc0 L_exit_%=")
        em.label("L_odd_%=")
        self.step(em, 1, "o")
        em.raw("s_cbranch_scc1 L_even_%=")
        em.raw("s_branch L_exit_%=")
        for uid in ("e", "o"):
            self.rare_block(em, 0, f"L_rare_{uid}a_%=", f"L_back_{uid}a_%=")
            self.rare_block(em, 1, f"L_rare_{uid}b_%=", f"L_back_{uid}b_%=")
        em.label("L_exit_%=")
        em.raw("s_nop 11", "nop")                # results of the last matrix instructions are visible to what follows
        return em

    def emit_text(self):
        t, nq = self.t, self.nq
        em = self.generate()
        n_mfma = sum(1 for i in em.out if i.kind == "mfma")
        n_valu = sum(1 for i in em.out if i.kind in ("valu", "trans", "swap", "dot"))
        sfx = f"_NQ{nq}" + ("M" if self.masked else "")
        text = (
            f"// ---- NQ = {nq}{' with the causal mask' if self.masked else ''}: {len(em.out)} lines, {n_mfma} matrix and {n_valu} vector instructions (rare paths "
            f"included), {em.nops} padding wait states; {t.num_vgpr} vector + {t.num_agpr} accumulation registers\n"
        )
        binds = {}
        for q in range(nq):
            for d in range(4):
                binds[f"O{q}{d}"] = (t.O[q][d], 16)
            binds[f"Q{q}"] = (t.Q[q], 32)
            binds[f"S{q}0"], binds[f"S{q}1"] = (t.S[q][0], 16), (t.S[q][1], 16)
            binds[f"P{q}0"], binds[f"P{q}1"] = (t.P[q][0], 8), (t.P[q][1], 8)
            binds[f"NM{q}"] = (t.NM[q], 16)
            binds[f"M{q}"], binds[f"L{q}"] = (t.M[q], 1), (t.L[q], 1)
        binds.update({"KOFF": (t.KOFF, 8), "VOFF": (t.VOFF, 4), "OFSK": (t.OFSK, 4), "OFSV": (t.OFSV, 4)})
        if self.masked:
            binds.update({"THR": (t.THR, 1), "NINF": (t.NINF, 1)})
        for name, (lo, n) in binds.items():
            text += f'#define RPA_PIPE{sfx}_C_{name} "{{{vr(lo, n)}}}"\n'
        lines = ['    "%s\\n"' % ins.text for ins in em.out]
        text += f"#define RPA_PIPE{sfx}_ASM \\\n" + " \\\n".join(lines) + "\n"
        clob = ['"v%d"' % r for r in range(t.first_scratch, t.num_vgpr)]
        clob += ['"%s"' % vr(r) for r in list(rng(t.KF, 4 * NBUF)) + list(rng(t.VF, 4 * NBUF))]
        clob += ['"s%d"' % r for r in SGPR_CLOBBERS]
        if self.masked:
            clob += ['"s%d"' % r for sg in MASK_SGPR for r in (sg, sg + 1)]
        text += f"#define RPA_PIPE{sfx}_CLOBBERS " + ", ".join(clob) + ', "vcc", "scc", "m0", "memory"\n'
        print(f"NQ={nq}{'M' if self.masked else ''}: {len(em.out)} lines, {n_mfma} MFMAs, {n_valu} vector, {em.nops} padding wait states, "
              f"{t.num_vgpr} VGPRs + {t.num_agpr} AGPRs")
        return text


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    text = ("// GENERATED by gen_prefill_pipe_loop.py -- do not edit; edit the generator and run it.\n"
            "// Steady-state loop of rpa_prefill_pipe_kernel: steps t .. t_end-1 of one wave, for one and two\n"
            "// blocks of 32 query rows per wave.  The RPA_PIPE_NQn_C_* macros are the register constraints\n"
            "// that bind the kernel's variables to the registers the assembly uses.\n")
    for nq in (1, 2):
        text += Gen(nq).emit_text()
    text += Gen(1, masked=True).emit_text()
    with open(os.path.join(here, "rpa_prefill_pipe_loop.inc"), "w") as f:
        f.write(text)


if __name__ == "__main__":
    sys.exit(main())
