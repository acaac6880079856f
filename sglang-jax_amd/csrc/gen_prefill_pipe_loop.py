#!/usr/bin/env python3
"""Generator of ``rpa_prefill_pipe_loop.inc``: the steady-state loop of the pipelined prefill
kernel (rpa_prefill_pipe.hip) as one hand-scheduled gfx950 assembly block.

    python gen_prefill_pipe_loop.py            # rewrites rpa_prefill_pipe_loop.inc next to it

The loop runs steps t .. t_end-1 of one wave.  A step covers one 64-token K/V tile as two
iterations over 32-token halves:
    iteration i:  S(i+1) = K(i+1).Q^T   (8 MFMAs)      O += V(i-1)^T.P(i-1)^T   (8 MFMAs)
                  P(i) = bf16(2^(S(i) c - m c)), row sum, row maximum            (vector pipe)
with the matrix and vector instructions interleaved one by one, the LDS operands fetched a fixed
number of matrix instructions ahead, the eight global -> LDS copy instructions of the step (K tile
t+1, V tile t) spread over its first iteration, and one barrier at the end of the step.  The whole
loop is one block because the register allocator will not keep two hundred registers in place
around a block that is only a loop body: here they are moved in and out once per loop.

The generator keeps three promises the assembler cannot check:
  * every `s_waitcnt lgkmcnt(n)` is computed from the issue order of the LDS reads (the one scalar
    load in flight only makes the counted waits longer, never shorter);
  * the issue distances the hardware does not interlock are verified (and padded with s_nop):
    MFMA result -> vector read/write (12), vector write -> MFMA operand (2), transcendental
    result -> vector read (1), vector write -> v_permlane32_swap (2), scalar write of m0 -> copy (1);
  * register use follows one table shared with the C++ side through the emitted macros.
"""

from __future__ import annotations

import os
import sys

# ------------------------------------------------------------------ register table
# Experiment switches (timing probes only: results are wrong with any of them set, except "oacc")
X = set(os.environ.get("RPA_PIPE_X", "").split(","))
ACC = 1000                                # register ids >= ACC name accumulation registers a[id - ACC]
O_IN_ACC = "ovgpr" not in X               # the output accumulators live in a[0:63]: only matrix instructions touch them

_next = 0
_next_acc = ACC + (64 if O_IN_ACC else 0)


def _alloc(n, acc=False):
    """n consecutive vector registers, or accumulation registers when the whole table goes that way"""
    global _next, _next_acc
    if acc and O_IN_ACC:
        lo = _next_acc
        _next_acc += n
        return lo
    lo = _next
    _next += n
    return lo


O = [ACC + 16 * d for d in range(4)] if O_IN_ACC else [_alloc(16) for d in range(4)]
S = [_alloc(16), _alloc(16)]              # S0, S1
P = [_alloc(8), _alloc(8)]                # P0, P1 (8 registers each: two B operands)
Q = _alloc(32, acc=True)                          # Q^T operands, 8 x 4 registers
KOFF = _alloc(8)                          # 8 LDS byte addresses of the K operand reads
VOFF = _alloc(4)                          # 4 LDS byte addresses of the V^T operand reads
M, L = _alloc(1), _alloc(1)
OFSK = _alloc(4)                          # 4 per-lane global byte offsets of this wave's K copies
OFSV = _alloc(4)                          # 4 ... V copies
FIRST_SCRATCH = _next
NEGM, MX, T0, T1, PS0, PS1 = (_alloc(1) for _ in range(6))
E = _alloc(8)                             # 8 temporaries of the exponentials
NBUF = 4                                  # operand fragment buffers per matrix
KF = _alloc(4 * NBUF, acc=True)                   # K fragments, 4 registers each
VF = _alloc(4 * NBUF, acc=True)                   # V^T fragments, 4 registers each
NUM_VGPR = _next

# scalar registers used inside the block (all listed as clobbers)
KB, VB = 60, 62                           # s[60:61], s[62:63]: global base of the K / V tile being copied
ST = [64, 65, 66, 67]                     # temporaries
PGC = 68                                  # page id of tile t + 2
SGPR_CLOBBERS = list(range(60, 69))

K_SLOT = [0, 16384]                       # byte offsets of the ring slots from the LDS array's start
V_SLOT = [32768, 49152]
V_READ = [0, 16384]                       # ... of the V slots from the addresses in VOFF (which point into V slot 0)
HALF = 8192
AHEAD = 3                                 # fragments requested ahead of the MFMA that uses them

AHEAD = int(os.environ.get("RPA_PIPE_AHEAD", AHEAD))

MFMA_TO_VALU = 12
VALU_TO_MFMA = 2
TRANS_TO_VALU = 1
VALU_TO_SWAP = 2


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
    if ins.kind == "label":
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
        if ins.lds_need:
            pos = max(self.lds_queue.index(t) for t in ins.lds_need)
            behind = len(self.lds_queue) - 1 - pos
            assert behind <= 15
            self.out.append(Ins(f"s_waitcnt lgkmcnt({behind})", "wait"))
            self.lds_queue = self.lds_queue[pos + 1:]
        r, w = ins.reads, ins.writes
        if ins.kind in ("valu", "trans", "swap"):
            self._pad(MFMA_TO_VALU, lambda p: p.kind == "mfma" and (p.writes & (r | w)))
            self._pad(TRANS_TO_VALU, lambda p: p.kind == "trans" and (p.writes & r))
            if ins.kind == "swap":
                self._pad(VALU_TO_SWAP, lambda p: p.kind in ("valu", "trans") and (p.writes & r))
        if ins.kind == "mfma":
            self._pad(VALU_TO_MFMA, lambda p: p.kind in ("valu", "trans", "swap") and (p.writes & r))
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


# ------------------------------------------------------------------ instruction builders
def mfma(dst, a, b, c):
    """dst/c: base of 16 registers (c None => zero), a/b: base of 4 registers"""
    ctext = "0" if c is None else vr(c, 16)
    reads = list(rng(a, 4)) + list(rng(b, 4)) + ([] if c is None else list(rng(c, 16)))
    return Ins(f"v_mfma_f32_32x32x16_bf16 {vr(dst, 16)}, {vr(a, 4)}, {vr(b, 4)}, {ctext}", "mfma", reads, rng(dst, 16))


def valu(text, reads, writes, kind="valu"):
    return Ins(text, kind, reads, writes)


def lds_k(f, slot):
    """K fragment f (0..15: half f // 8, k-step f % 8) -> KF[f % NBUF]"""
    k, half = f % 8, f // 8
    dst = KF + 4 * (f % NBUF)
    off = K_SLOT[slot] + half * HALF
    return [Ins(f"ds_read_b128 {vr(dst, 4)}, {vr(KOFF + k)} offset:{off}", "lds", [KOFF + k], rng(dst, 4), lds_tag=("k", f))]


def lds_v(f, slot):
    """two transposing reads: V^T fragment f (half f // 8, k-step (f % 8) >> 2, dim tile f & 3) -> VF[f % NBUF]"""
    k, half = f % 8, f // 8
    dst = VF + 4 * (f % NBUF)
    d, kk = k & 3, k >> 2
    off = V_READ[slot] + half * HALF + kk * 4096
    return [Ins(f"ds_read_b64_tr_b16 {vr(dst, 2)}, {vr(VOFF + d)} offset:{off}", "lds", [VOFF + d], rng(dst, 2), lds_tag=("vlo", f)),
            Ins(f"ds_read_b64_tr_b16 {vr(dst + 2, 2)}, {vr(VOFF + d)} offset:{off + 2048}", "lds", [VOFF + d], rng(dst + 2, 2),
                lds_tag=("vhi", f))]


def mfma_qk(f, sn):
    k = f % 8
    ins = mfma(S[sn], KF + 4 * (f % NBUF), Q + 4 * k, None if k == 0 else S[sn])
    ins.lds_need = None if "nolds" in X else [("k", f)]
    if "nomfma" in X:
        return Ins("s_nop 0", "nop")
    return ins


def mfma_pv(f, pp):
    k = f % 8
    d, kk = k & 3, k >> 2
    ins = mfma(O[d], VF + 4 * (f % NBUF), P[pp] + 4 * kk, O[d])
    ins.lds_need = None if "nolds" in X else [("vlo", f), ("vhi", f)]
    if "nomfma" in X:
        return Ins("s_nop 0", "nop")
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
        valu(f"v_dot2c_f32_bf16 {vr(ps)}, %[ones], {vr(w)}", [w, ps], [ps]),
    ]
    return out


def softmax_head():
    return [valu(f"v_mul_f32 {vr(NEGM)}, %[nsc2], {vr(M)}", [M], [NEGM]),
            valu(f"v_mov_b32 {vr(PS0)}, 0", [], [PS0]),
            valu(f"v_mov_b32 {vr(PS1)}, 0", [], [PS1])]


def softmax_tail():
    """row maximum across the two lane halves and the test against the running maximum"""
    return [
        valu(f"v_mov_b32 {vr(T0)}, {vr(MX)}", [MX], [T0]),
        valu(f"v_mov_b32 {vr(T1)}, 0", [], [T1]),  # filler between the write of T0 and the swap
        Ins(f"v_permlane32_swap_b32 {vr(MX)}, {vr(T0)}", "swap", [MX, T0], [MX, T0]),
        valu(f"v_max_f32 {vr(MX)}, {vr(MX)}, {vr(T0)}", [MX, T0], [MX]),
        valu(f"v_sub_f32 {vr(T0)}, {vr(MX)}, {vr(M)}", [MX, M], [T0]),
        valu(f"v_mul_f32 {vr(T0)}, %[sc2], {vr(T0)}", [T0], [T0]),
        valu(f"v_cmp_lt_f32 vcc, 8.0, {vr(T0)}", [T0], []),   # kMaxSlack
    ]


def copy_ins(n, is_v, fill_slot):
    """global -> LDS copy n (0..3) of this wave: 1 KiB block 4*wave + n of the slot"""
    base = (V_SLOT if is_v else K_SLOT)[fill_slot] + n * 1024
    ofs = (OFSV if is_v else OFSK) + n
    sb = VB if is_v else KB
    return [Ins(f"s_add_u32 m0, %[lds_wave], {base}", "salu"),
            Ins("s_nop 0", "nop"),
            Ins(f"global_load_lds_dwordx4 {vr(ofs)}, s[{sb}:{sb + 1}]", "vmem", [ofs], [])]


def iteration(em, it, ks, vs, frag_reads, copies):
    """Iteration `it` (0 / 1) of a step.  it = 0: softmax of S1 into P1, scores of the tile's first
    half into S0, second product with P0; it = 1: the mirror image on the second half.
    frag_reads(f): emits the LDS reads of fragment pair f (no-op past the step's last fragment).
    copies: copy instruction groups, one dealt out behind each second-product MFMA."""
    sc = 1 - it
    sn, pc, pp = 1 - sc, sc, 1 - sc
    stream = softmax_head() + [x for j in range(8) for x in softmax_pair(j, sc, pc)] + softmax_tail()
    # the first iteration's scores were finished in the previous step: a first chunk of vector work
    # runs while the step's first fragments travel; the rest is dealt out behind the matrix instructions
    lead = 8 if it == 0 else 0
    pos = 0

    def deal(n):
        nonlocal pos
        for _ in range(n):
            if pos < len(stream):
                if "novalu" not in X:
                    em.emit(stream[pos])
                pos += 1

    deal(lead)
    rest = len(stream) - lead
    per = [rest // 16] * 16
    rem = rest - sum(per)
    for i in range(rem):
        per[(i * 16) // rem] += 1
    for k in range(8):
        f = 8 * it + k
        em.emit(mfma_qk(f, sn))
        frag_reads("k", f + AHEAD)
        deal(per[2 * k])
        em.emit(mfma_pv(f, pp))
        frag_reads("v", f + AHEAD)
        if copies:
            for x in copies.pop(0):
                em.emit(x)
        deal(per[2 * k + 1])
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
    for r in [o + v for o in O for v in range(16)]:
        if O_IN_ACC:
            em.emit(valu(f"v_accvgpr_read_b32 {vr(T1)}, {vr(r)}", [r], [T1]))
            em.emit(valu(f"v_mul_f32 {vr(T1)}, {vr(T1)}, {vr(T0)}", [T1, T0], [T1]))
            em.emit(valu(f"v_accvgpr_write_b32 {vr(r)}, {vr(T1)}", [T1], [r]))
        else:
            em.emit(valu(f"v_mul_f32 {vr(r)}, {vr(r)}, {vr(T0)}", [r, T0], [r]))
    em.emit(valu(f"v_mov_b32 {vr(PS0)}, 0", [], [PS0]))
    em.emit(valu(f"v_mov_b32 {vr(PS1)}, 0", [], [PS1]))
    for j in range(8):
        for x in softmax_pair(j, sc, pc, with_max=False):
            em.emit(x)
    em.raw("s_nop 3", "nop")  # P(i) and O were written by the vector pipe; a matrix instruction may follow at once
    em.raw(f"s_branch {back}")


def tile_base(em, dst, pg, tb_reg, head_lo, head_hi):
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


def step(em, par, uid):
    """Step with K tile t in K slot `par` and V tile t-1 in V slot 1-par; fills K slot 1-par with
    tile t+1 (page pg_b) and V slot par with tile t (page pg_a)."""
    ks, vs = par, 1 - par
    t0, t1 = f"s{ST[0]}", f"s{ST[1]}"
    em.raw(f"s_lshl_b32 {t0}, %[t], 6")
    em.raw(f"s_add_u32 {t0}, {t0}, %[t_lo]")                   # first token of tile t
    em.raw(f"s_add_u32 {t1}, {t0}, 64")                        # ... of tile t + 1
    tile_base(em, VB, "%[pg_a]", t0, "%[vh_lo]", "%[vh_hi]")
    tile_base(em, KB, "%[pg_b]", t1, "%[kh_lo]", "%[kh_hi]")
    # page id of tile t + 2 (clamped to the sequence's last tile), consumed at the end of the step
    em.raw(f"s_add_u32 {t1}, {t1}, 64")
    em.raw(f"s_min_i32 {t1}, {t1}, %[last_tile_tok]")
    em.raw(f"s_lshr_b32 {t1}, {t1}, %[pshift]")
    em.raw(f"s_lshl_b32 {t1}, {t1}, 2")
    em.raw(f"s_load_dword s{PGC}, %[pages], {t1}")

    def frag_reads(which, f):
        if f >= 16 or "nolds" in X:
            return
        for x in (lds_k(f, ks) if which == "k" else lds_v(f, vs)):
            em.emit(x)

    for f in range(AHEAD):
        frag_reads("k", f)
        frag_reads("v", f)
    copies = [copy_ins(n, False, 1 - ks) for n in range(4)] + [copy_ins(n, True, 1 - vs) for n in range(4)]
    if "nocopy" in X:
        copies = []
    for it in (0, 1):
        iteration(em, it, ks, vs, frag_reads, copies)
        tag = uid + "ab"[it]
        if "norare" not in X:
            em.raw(f"s_cbranch_vccnz L_rare_{tag}_%=")
        em.label(f"L_back_{tag}_%=")
        em.emit(valu(f"v_add_f32 {vr(PS0)}, {vr(PS0)}, {vr(PS1)}", [PS0, PS1], [PS0]))
        em.emit(valu(f"v_add_f32 {vr(L)}, {vr(L)}, {vr(PS0)}", [L, PS0], [L]))
    assert not copies and not em.lds_queue
    # ---- end of step: the copies have landed, everybody has finished reading the slots they overwrite next
    em.raw("s_waitcnt vmcnt(0) lgkmcnt(0)", "wait")
    em.raw("s_mov_b32 %[pg_a], %[pg_b]")
    em.raw(f"s_mov_b32 %[pg_b], s{PGC}")
    if "nobarrier" not in X:
        em.raw("s_barrier")
    em.raw("s_add_u32 %[t], %[t], 1")
    em.raw("s_cmp_lt_i32 %[t], %[t_end]")


def generate():
    em = Emitter()
    # Nothing of the caller's is in flight on the LDS / scalar-memory counter.  Matrix instructions the
    # caller issued before this block have finished: a barrier and this block's entry moves lie in between.
    em.raw("s_waitcnt lgkmcnt(0)", "wait")
    em.raw("s_nop 11", "nop")
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
    em.raw("s_nop 11", "nop")                # results of the last matrix instructions are visible to what follows
    return em


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    em = generate()
    n_mfma = sum(1 for i in em.out if i.kind == "mfma")
    n_valu = sum(1 for i in em.out if i.kind in ("valu", "trans", "swap"))
    text = (
        "// GENERATED by gen_prefill_pipe_loop.py -- do not edit; edit the generator and run it.\n"
        "// Steady-state loop of rpa_prefill_pipe_kernel: steps t .. t_end-1 of one wave.\n"
        f"// {len(em.out)} lines, {n_mfma} matrix and {n_valu} vector instructions (rare paths included), "
        f"{em.nops} padding wait states.\n"
        "// Register table (shared with rpa_prefill_pipe.hip through the RPA_PIPE_C_* constraint macros):\n"
        f"//   O {vr(O[0], 64)}  S0 {vr(S[0], 16)}  S1 {vr(S[1], 16)}  P0 {vr(P[0], 8)}  P1 {vr(P[1], 8)}\n"
        f"//   Q {vr(Q, 32)}  koff {vr(KOFF, 8)}  voff {vr(VOFF, 4)}  m {vr(M)}  l {vr(L)}\n"
        f"//   ofs_k {vr(OFSK, 4)}  ofs_v {vr(OFSV, 4)}  scratch {vr(FIRST_SCRATCH, NUM_VGPR - FIRST_SCRATCH)}\n"
    )
    binds = {"O0": (O[0], 16), "O1": (O[1], 16), "O2": (O[2], 16), "O3": (O[3], 16), "S0": (S[0], 16), "S1": (S[1], 16),
             "P00": (P[0], 4), "P01": (P[0] + 4, 4), "P10": (P[1], 4), "P11": (P[1] + 4, 4), "QA": (Q, 16), "QB": (Q + 16, 16),
             "KOFF": (KOFF, 8), "VOFF": (VOFF, 4), "M": (M, 1), "L": (L, 1), "OFSK": (OFSK, 4), "OFSV": (OFSV, 4)}
    for name, (lo, n) in binds.items():
        text += f'#define RPA_PIPE_C_{name} "{{{vr(lo, n)}}}"\n'
    lines = ['    "%s\\n"' % ins.text for ins in em.out]
    text += "#define RPA_PIPE_LOOP_ASM \\\n" + " \\\n".join(lines) + "\n"
    clobbers = ", ".join('"v%d"' % r for r in range(FIRST_SCRATCH, NUM_VGPR))
    if O_IN_ACC:
        clobbers += ", " + ", ".join('"a%d"' % (r - ACC) for r in list(range(KF, KF + 4 * NBUF)) + list(range(VF, VF + 4 * NBUF)))
    clobbers += ", " + ", ".join('"s%d"' % r for r in SGPR_CLOBBERS)
    text += "#define RPA_PIPE_LOOP_CLOBBERS " + clobbers + ', "vcc", "scc", "m0", "memory"\n'
    with open(os.path.join(here, "rpa_prefill_pipe_loop.inc"), "w") as f:
        f.write(text)
    print(f"wrote rpa_prefill_pipe_loop.inc: {len(em.out)} lines, {n_mfma} MFMAs, {n_valu} vector, {em.nops} padding wait states")


if __name__ == "__main__":
    sys.exit(main())
