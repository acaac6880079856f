// Software-pipelined flash kernel for the common prefill case on gfx950: bf16 cache, 128-wide
// heads, power-of-two pages of at least 64 tokens, causal mask (optionally with a sliding window),
// no score options.
//
// LDS layout and copies are those of rpa_prefill_async_kernel (K/V tiles of 64 tokens arrive through
// global_load_lds_dwordx4 into XOR-swizzled row-major LDS tiles, two ring slots per matrix).  A
// workgroup of 4 waves owns 128 * NQ query rows of one query head; wave w owns NQ blocks of 32 rows.
// With NQ = 2 every K and V^T fragment read from LDS feeds two MFMAs and a tile copied into LDS
// serves twice the rows; the wave then needs more than 256 registers, so one wave runs per SIMD and
// the overlap between matrix, vector and LDS work has to come from inside the wave.  A 64-token tile
// is handled as two halves of 32 tokens, and iteration i holds three independent instruction
// streams per block of rows:
//     matrix pipe   S(i+1) = K(i+1) . Q^T - m      8 MFMAs (one accumulator chain)
//     matrix pipe   O     += V(i-1)^T . P(i-1)^T   8 MFMAs (four accumulator chains)
//     vector pipe   P(i)   = 2^S(i)                exponentials, packing, row sum
// Step t of a workgroup is the pair of iterations (2t-1, 2t): it reads K tile t and V tile t-1, so
// two ring slots per matrix suffice (V lags K by one tile) and there is one barrier per tile.
//
// Scores leave the matrix pipe ready for v_exp_f32: the queries are multiplied by
// sm_scale * log2(e) once (and rounded to bf16 again: a relative change of 2^-9 per element, the
// size of the rounding they already carry), and the first MFMA of a score chain takes minus the
// running maximum as its C operand.  The running maximum is checked after the fact: a half's
// probabilities are taken against the maximum known before it; if a row sum of the half exceeds
// 2^8 the half is redone against its true maximum and everything accumulated is rescaled.
//
// The compiler does not keep such an interleave (it regroups the matrix instructions and spills),
// and it will not keep hundreds of registers in place around an assembly block that is only a loop
// body, so the whole run of steady-state steps of a wave is one assembly block with fixed
// registers, written by gen_prefill_pipe_loop.py into rpa_prefill_pipe_loop.inc; this file binds
// the kernel's variables to those registers.  Steps that touch the causal diagonal or a window
// edge, the first and the last steps run the same pipeline through a general iteration in C++ with
// masking and run-time flags.
//
// The global -> LDS copies are issued as assembly too, so the compiler knows of no store into the
// LDS ring and never waits for the copy queue on its own; the kernel waits (vmcnt(0)) in front of
// the barrier that ends a step.

#include <type_traits>

#include "rpa_prefill_common.h"
#include "rpa_prefill_pipe_loop.inc"

namespace rpa {

using namespace pf;

namespace {

constexpr int kRowB = 256;               // bytes of one K or V row of a head
constexpr int kTileB = kBN * kRowB;      // 16 KiB
constexpr int kHalfB = 32 * kRowB;       // byte distance between the halves of a tile
constexpr int kKSlot = 0;                // ring slots inside the LDS array: K0 K1 V0 V1
constexpr int kVSlot = 2 * kTileB;
constexpr float kRowSumLimit = 256.0f;   // a half's row sum above it: the stale maximum is too stale
constexpr float kSeenFloor = -1.0e30f;   // a row maximum below it: every token so far was masked

typedef uint32_t u32x32_t __attribute__((ext_vector_type(32)));
typedef uint32_t u32x8_t __attribute__((ext_vector_type(8)));
typedef int32_t i32x8_t __attribute__((ext_vector_type(8)));
typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4v_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ u32x4_t lds_ld16_at(int addr) {
  typedef const __attribute__((address_space(3))) u32x4_t* p_t;
  return *(p_t)(uintptr_t)(uint32_t)addr;
}
__device__ __forceinline__ u32x2_t lds_tr16_at(int addr) {
  typedef __attribute__((address_space(3))) s16x4v_t* p_t;
  return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((p_t)(uintptr_t)(uint32_t)addr));
}

// The registers of one block of 32 query rows.  The assembly loop expects them in the registers the
// RPA_PIPE_NQn_C_* constraints of rpa_prefill_pipe_loop.inc name.
struct RowBlock {
  f32x16_t O[4];    // accumulators, lane (c, h): row c, dims 32d + 8*(v/4) + 4h + v%4
  u32x32_t Q;       // Q^T operands of the 8 k-steps, scaled to log2 units
  f32x16_t S[2];    // scores of the even / odd half in flight, minus the running maximum
  u32x8_t P[2];     // probabilities of the even / odd half (two B operands of the second product each)
  f32x16_t NM;      // minus the running maximum in all 16 registers (C operand of a score chain's first MFMA)
  float m, l;       // running maximum (log2 units), running sum of this lane's tokens
  float seen;       // 1 once the row has met a token it may see (same in both lanes of a row)
  int qpos;         // position of this lane's row
};

struct Shared {   // what the row blocks of a wave share
  i32x8_t koff;   // LDS addresses of the K operand reads (slot 0, first half)
  i32x4_t voff;   // LDS addresses of the V^T operand reads (slot 0, first half, first k-step)
  u32x4_t ofs_k, ofs_v;  // per-lane byte offsets of this wave's four K / V copy instructions
};

template <int KS>
__device__ __forceinline__ u32x4_t q_frag(const u32x32_t& q) {
  return u32x4_t{q[4 * KS], q[4 * KS + 1], q[4 * KS + 2], q[4 * KS + 3]};
}

// K or V rows of one tile, global -> LDS: 4 instructions per wave.  `lds_wave` is the LDS address
// of this wave's first 1 KiB block of the slot.
template <bool IS_V>
__device__ __forceinline__ void copy_rows(uint32_t lds_wave, const TileSrc& s, const KvAddr& kv, const char* head, int tb,
                                          int wave, int lane, int page, const Shared& sh) {
  tb = min(tb, s.last_tok & ~(kBN - 1));
  if (tb + kBN - 1 <= s.last_tok) {
    const int64_t base = (int64_t)page * kv.page_stride + (int64_t)(tb - page_slot(s, tb) * s.page_size) * kv.tok_stride;
    const char* b = head + base;  // wave-uniform
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :: "s"(lds_wave + n * 1024), "v"(IS_V ? sh.ofs_v[n] : sh.ofs_k[n]), "s"(b)
                   : "memory", "m0");
    }
    return;
  }
  // last, partial tile: rows clamped to the last valid token
  const int cp = lane & 15;
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    const int t = (wave * 4 + n) * 4 + (lane >> 4);
    const int64_t ro = row_offset<true>(s, kv, tb, tb + t, page);
    const int j = IS_V ? (cp ^ ((t & 3) << 2)) : (cp ^ (t & 15));
    const char* g = head + ro + j * 16;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :: "s"(lds_wave + n * 1024), "v"(g)
                 : "memory", "m0");
  }
}

__device__ __forceinline__ int scalar_page(const TileSrc& s, int tb) {
  tb = min(tb, s.last_tok & ~(kBN - 1));
  return scalar_load_i32(s.pages + __builtin_amdgcn_readfirstlane(page_slot(s, tb)));
}

// first product of one 32-token half: one chain of 8 MFMAs starting from minus the running
// maximum; `off` = slot and half offset
__device__ __forceinline__ f32x16_t qk_half(const RowBlock& b, const Shared& sh, int off) {
  f32x16_t S = mfma32(lds_ld16_at(sh.koff[0] + off), q_frag<0>(b.Q), b.NM);
  S = mfma32(lds_ld16_at(sh.koff[1] + off), q_frag<1>(b.Q), S);
  S = mfma32(lds_ld16_at(sh.koff[2] + off), q_frag<2>(b.Q), S);
  S = mfma32(lds_ld16_at(sh.koff[3] + off), q_frag<3>(b.Q), S);
  S = mfma32(lds_ld16_at(sh.koff[4] + off), q_frag<4>(b.Q), S);
  S = mfma32(lds_ld16_at(sh.koff[5] + off), q_frag<5>(b.Q), S);
  S = mfma32(lds_ld16_at(sh.koff[6] + off), q_frag<6>(b.Q), S);
  S = mfma32(lds_ld16_at(sh.koff[7] + off), q_frag<7>(b.Q), S);
  return S;
}

// second product of one 32-token half: four chains of 2 MFMAs
__device__ __forceinline__ void pv_half(RowBlock& b, const Shared& sh, int off, const u32x8_t& P) {
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int vt = sh.voff[d] + off + kk * 16 * kRowB;
      const u32x2_t lo = lds_tr16_at(vt);
      const u32x2_t hi = lds_tr16_at(vt + 8 * kRowB);
      b.O[d] = mfma32(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, u32x4_t{P[4 * kk], P[4 * kk + 1], P[4 * kk + 2], P[4 * kk + 3]},
                      b.O[d]);
    }
}

// probabilities of 16 scores that are already relative to the running maximum: P = bf16(2^S), their sum
__device__ __forceinline__ float exp_pack(const f32x16_t& S, u32x8_t& P) {
  const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
  float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t w = pack_bf16x2(fast_exp2(S[2 * j]), fast_exp2(S[2 * j + 1]));
    P[j] = w;
    if (j & 1) ps1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), ones, ps1, false);
    else ps0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), ones, ps0, false);
  }
  return ps0 + ps1;
}

__device__ __forceinline__ float row_max16(const f32x16_t& S) {
  float mx = __builtin_fmaxf(__builtin_fmaxf(S[0], S[1]), S[2]);
#pragma unroll
  for (int v = 3; v < 15; v += 2) mx = __builtin_fmaxf(__builtin_fmaxf(mx, S[v]), S[v + 1]);
  mx = __builtin_fmaxf(mx, S[15]);
  return swap_max(mx);
}

// Softmax of a half with the maximum taken first (first halves of a row, masked halves).  Sc: the
// half's scores relative to the running maximum; Sn: the scores of the next half, already computed
// against the same maximum, which move with it.
__device__ __forceinline__ void softmax_half_general(f32x16_t& Sc, f32x16_t& Sn, RowBlock& b, bool need_mask, int tb, int h,
                                                     int window, u32x8_t& P) {
  if (need_mask) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int tok = tb + 8 * (v >> 2) + 4 * h + (v & 3);
      const bool masked = tok > b.qpos || (window > 0 && tok <= b.qpos - window);
      Sc[v] = masked ? kMaskRaw : Sc[v];
    }
  }
  const float mx = row_max16(Sc);
  // a row that has seen nothing yet takes the half's maximum as it is (nothing to rescale); afterwards
  // the maximum only rises, and only when it is off by more than the slack
  const bool real = mx > kSeenFloor;
  const float d = (b.seen == 0.f) ? (real ? mx : 0.f) : (mx > kMaxSlack ? mx : 0.f);
  if (__builtin_amdgcn_ballot_w64(d != 0.f) != 0) {
    const float alpha = (b.seen == 0.f) ? 1.0f : fast_exp2(-d);
    b.m += d;
    b.l *= alpha;
#pragma unroll
    for (int dd = 0; dd < 4; ++dd)
#pragma unroll
      for (int v = 0; v < 16; ++v) b.O[dd][v] *= alpha;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      b.NM[v] = -b.m;
      Sc[v] -= d;
      Sn[v] -= d;
    }
  }
  if (real) b.seen = 1.0f;
  b.l += exp_pack(Sc, P);
}

struct LoopScalars {
  int t_end, t_lo, pmask, pshift, tok_stride, last_tile_tok;
  uint32_t pstr, kh_lo, kh_hi, vh_lo, vh_hi, lds_wave;
  const int32_t* pages;
  float limit;
};

// Steady-state steps [t, t_end) in assembly.  On entry K tile t is in K slot t & 1 and V tile t - 1
// in V slot 1 - (t & 1), pg_a / pg_b are the pages of tiles t and t + 1; on exit the same holds for
// t = t_end.  Every tile the loop copies (up to t_end) lies completely inside the sequence.
#define RPA_PIPE_SCALARS(sc)                                                                                    \
  [ones] "s"(0x3f803f80u), [limit] "s"(sc.limit), [t_end] "s"(sc.t_end), [t_lo] "s"(sc.t_lo), [pmask] "s"(sc.pmask), \
      [pshift] "s"(sc.pshift), [tok_stride] "s"(sc.tok_stride), [last_tile_tok] "s"(sc.last_tile_tok),             \
      [pstr] "s"(sc.pstr), [kh_lo] "s"(sc.kh_lo), [kh_hi] "s"(sc.kh_hi), [vh_lo] "s"(sc.vh_lo),                    \
      [vh_hi] "s"(sc.vh_hi), [lds_wave] "s"(sc.lds_wave), [pages] "s"(sc.pages)

__device__ __forceinline__ void pipe_loop(RowBlock (&b)[1], const Shared& sh, int& t, int& pg_a, int& pg_b,
                                          const LoopScalars& sc) {
#define C(n) RPA_PIPE_NQ1_C_##n
  // t and the page ids change inside the block while inputs are still being read: early-clobber, so that no
  // input that happens to hold the same value on entry can share their registers
  asm volatile(RPA_PIPE_NQ1_ASM
               : "+" C(O00)(b[0].O[0]), "+" C(O01)(b[0].O[1]), "+" C(O02)(b[0].O[2]), "+" C(O03)(b[0].O[3]),
                 "+" C(S00)(b[0].S[0]), "+" C(S01)(b[0].S[1]), "+" C(P00)(b[0].P[0]), "+" C(P01)(b[0].P[1]),
                 "+" C(NM0)(b[0].NM), "+" C(M0)(b[0].m), "+" C(L0)(b[0].l),
                 [t] "+&s"(t), [pg_a] "+&s"(pg_a), [pg_b] "+&s"(pg_b)
               : C(Q0)(b[0].Q), C(KOFF)(sh.koff), C(VOFF)(sh.voff), C(OFSK)(sh.ofs_k), C(OFSV)(sh.ofs_v),
                 RPA_PIPE_SCALARS(sc)
               : RPA_PIPE_NQ1_CLOBBERS);
#undef C
}

// The same steps with the causal mask applied to every half before its exponentials (the steps on the
// diagonal).  thr: query position - first token of the half whose probabilities the block's first iteration
// takes (half 2t - 1) - 4 * (lane / 32); the block moves it on by 32 per half.
__device__ __forceinline__ void pipe_loop_masked(RowBlock (&b)[1], const Shared& sh, int& t, int& pg_a, int& pg_b,
                                                 const LoopScalars& sc, int thr) {
#define C(n) RPA_PIPE_NQ1M_C_##n
  const float ninf = -1.0e30f;
  asm volatile(RPA_PIPE_NQ1M_ASM
               : "+" C(O00)(b[0].O[0]), "+" C(O01)(b[0].O[1]), "+" C(O02)(b[0].O[2]), "+" C(O03)(b[0].O[3]),
                 "+" C(S00)(b[0].S[0]), "+" C(S01)(b[0].S[1]), "+" C(P00)(b[0].P[0]), "+" C(P01)(b[0].P[1]),
                 "+" C(NM0)(b[0].NM), "+" C(M0)(b[0].m), "+" C(L0)(b[0].l), "+" C(THR)(thr),
                 [t] "+&s"(t), [pg_a] "+&s"(pg_a), [pg_b] "+&s"(pg_b)
               : C(Q0)(b[0].Q), C(KOFF)(sh.koff), C(VOFF)(sh.voff), C(OFSK)(sh.ofs_k), C(OFSV)(sh.ofs_v), C(NINF)(ninf),
                 RPA_PIPE_SCALARS(sc)
               : RPA_PIPE_NQ1M_CLOBBERS);
#undef C
}
__device__ __forceinline__ void pipe_loop_masked(RowBlock (&)[2], const Shared&, int&, int&, int&, const LoopScalars&, int) {}

__device__ __forceinline__ void pipe_loop(RowBlock (&b)[2], const Shared& sh, int& t, int& pg_a, int& pg_b,
                                          const LoopScalars& sc) {
#define C(n) RPA_PIPE_NQ2_C_##n
  asm volatile(RPA_PIPE_NQ2_ASM
               : "+" C(O00)(b[0].O[0]), "+" C(O01)(b[0].O[1]), "+" C(O02)(b[0].O[2]), "+" C(O03)(b[0].O[3]),
                 "+" C(O10)(b[1].O[0]), "+" C(O11)(b[1].O[1]), "+" C(O12)(b[1].O[2]), "+" C(O13)(b[1].O[3]),
                 "+" C(S00)(b[0].S[0]), "+" C(S01)(b[0].S[1]), "+" C(P00)(b[0].P[0]), "+" C(P01)(b[0].P[1]),
                 "+" C(S10)(b[1].S[0]), "+" C(S11)(b[1].S[1]), "+" C(P10)(b[1].P[0]), "+" C(P11)(b[1].P[1]),
                 "+" C(NM0)(b[0].NM), "+" C(M0)(b[0].m), "+" C(L0)(b[0].l),
                 "+" C(NM1)(b[1].NM), "+" C(M1)(b[1].m), "+" C(L1)(b[1].l),
                 [t] "+&s"(t), [pg_a] "+&s"(pg_a), [pg_b] "+&s"(pg_b)
               : C(Q0)(b[0].Q), C(Q1)(b[1].Q), C(KOFF)(sh.koff), C(VOFF)(sh.voff), C(OFSK)(sh.ofs_k), C(OFSV)(sh.ofs_v),
                 RPA_PIPE_SCALARS(sc)
               : RPA_PIPE_NQ2_CLOBBERS);
#undef C
}

// HEADS4: the short-chunk tile.  A workgroup owns 32 query positions of FOUR query heads of a kv head, one
// head per wave, instead of 128 positions of one head: chunks of a few dozen tokens (a verify step, a short
// prompt, the tail of a long one) then fill their tiles, and the four waves still share every K/V tile.
//
// SPLIT: launches that would leave most of the GPU idle (one long prompt on a few heads, a verify step on a
// long context) cut every workgroup's run of K/V tiles into a.kv_splits pieces, blockIdx.y picks the piece,
// and the workgroup leaves unnormalised rows with their (reference, sum) in the workspace for
// rpa_prefill_combine_kernel instead of finished rows.
template <bool WIN, int NQ, bool HEADS4 = false, bool SPLIT = false>
__global__ __launch_bounds__(256, (NQ == 1 ? 2 : 1)) void rpa_prefill_pipe_kernel(const PrefillArgs a_in, int tiles, int nseq,
                                                                                 bool by_level, float row_sum_limit,
                                                                                 bool masked_steps) {
  PrefillArgs a = a_in;  // static-shape mode: the sequences to process come from the device
  if (a.dist) {
    a.seq_begin = (a.sm.mask_mode == 1) ? 0 : scalar_load_i32(a.dist);
    a.seq_end = min(a.seq_end, scalar_load_i32(a.dist + 2));
  }
  static_assert(!HEADS4 || NQ == 1, "the short-chunk tile has one block of rows per wave");
  constexpr int BM = HEADS4 ? 32 : 128 * NQ;  // query positions per workgroup
  __shared__ __attribute__((aligned(1024))) char lds[4 * kTileB];

  Work w = decompose(a, tiles, nseq, by_level, BM, HEADS4 ? 4 : 1);
  if (!w.valid) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if constexpr (HEADS4) w.head += wave;  // this wave's head
  const int c = lane & 31, h = lane >> 5;
  const TileSrc src = make_src(a, w);
  const char* kh = a.kv.k_base + (int64_t)w.hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)w.hk * a.kv.head_stride;
  typedef __attribute__((address_space(3))) char* lds_ptr_t;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)lds);

  // rows of the wave: NQ blocks of 32
  const int r_lo = w.q_start + (HEADS4 ? 0 : wave * 32 * NQ);
  const int r_hi = min(r_lo + 32 * NQ - 1, w.q_len - 1);
  const bool active = r_lo < w.q_len;
  const int W_ = WIN ? a.sm.window : 0;
  const float sc2 = a.sm.sm_scale * (a.k_scale ? a.k_scale[w.hk] : 1.0f) * kLog2e;

  const int wg_r_hi = min(w.q_start + BM, w.q_len) - 1;
  int t_hi = min(w.kv_len, w.prefix + wg_r_hi + 1);  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, w.prefix + w.q_start - W_ + 1) & ~(kBN - 1);
  int split = 0;
  if constexpr (SPLIT) {
    if (!kv_piece(a, t_lo, t_hi, split)) {  // nothing left for this piece
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        WaveRows wr;
        wr.r_lo = r_lo + 32 * q;
        wr.r_hi = min(wr.r_lo + 31, w.q_len - 1);
        wr.active = wr.r_lo < w.q_len;
        wr.row = wr.r_lo + c;
        wr.qpos = w.prefix + wr.row;
        write_empty_partial_rows<4>(a, w, wr, h, split);
      }
      return;
    }
    // the piece's bounds went through the vector pipe (a division); the assembly loop takes scalars
    t_lo = __builtin_amdgcn_readfirstlane(t_lo);
    t_hi = __builtin_amdgcn_readfirstlane(t_hi);
  }
  const int nT = (t_hi - t_lo + kBN - 1) / kBN;  // K/V tiles of the workgroup (of its piece)

  RowBlock b[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int row = r_lo + 32 * q + c;
    b[q].qpos = w.prefix + row;
    const int rr = min(row, w.q_len - 1);
    const uint16_t* qp = a.q + ((int64_t)(w.qg0 + rr) * a.Hq + w.head) * 128 + h * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const u32x4_t x = ld16(qp + ks * 16);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        b[q].Q[4 * ks + e] = pack_bf16x2(bf16_lo_to_f32(x[e]) * sc2, bf16_hi_to_f32(x[e]) * sc2);
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) b[q].O[d] = kZero16;
    b[q].S[0] = b[q].S[1] = b[q].NM = kZero16;
    b[q].P[0] = b[q].P[1] = u32x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    b[q].m = 0.f;
    b[q].l = 0.f;
    b[q].seen = 0.f;
  }

  // halves [0, n_w) of 32 tokens concern this wave; halves [i_f0, i_f1) need no mask for any of its rows
  int n_w = 0, i_f0 = 0, i_f1 = 0;
  if (active) {
    n_w = max(0, (min(t_hi, w.prefix + r_hi + 1) - t_lo + 31) >> 5);  // (t_hi <= kv_len; a piece may end before the wave's rows do)
    i_f1 = max(0, (w.prefix + r_lo - t_lo + 1) >> 5);
    if (W_ > 0) {
      const int y = w.prefix + r_hi - W_ - t_lo;
      i_f0 = y >= 0 ? (y >> 5) + 1 : 0;
    }
    i_f1 = min(i_f1, n_w);
  }
  n_w = __builtin_amdgcn_readfirstlane(n_w);
  i_f0 = __builtin_amdgcn_readfirstlane(i_f0);
  i_f1 = __builtin_amdgcn_readfirstlane(i_f1);

  // operand addresses inside the LDS array (see rpa_prefill_async_kernel for the swizzles)
  Shared sh;
  {
    const int k_row = c * kRowB;
    const int k_swz = (h ^ (c & 15)) << 4;
    const int r16 = lane & 15, b16 = lane >> 4;
    const int v_row = (4 * h + (r16 >> 2)) * kRowB;
    const int v_in = ((b16 & 1) << 5) + (((r16 & 3) >> 1) << 4) + ((r16 & 1) << 3);
    const int v_swz = (r16 >> 2) << 6;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) sh.koff[ks] = (int)lds_base + kKSlot + k_row + ((ks * 32) ^ k_swz);
#pragma unroll
    for (int d = 0; d < 4; ++d) sh.voff[d] = (int)lds_base + kVSlot + v_row + v_in + ((d * 64) ^ v_swz);
    const AsyncOffsets<128> ofs = make_async_offsets<128>(a.kv, wave, lane);
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      sh.ofs_k[n] = ofs.k[n];
      sh.ofs_v[n] = ofs.v[n];
    }
  }

  const uint32_t lds_wave = lds_base + wave * 4096;  // this wave's four 1 KiB blocks of slot K0
  int pg_a = scalar_page(src, t_lo);         // page of tile t
  copy_rows<false>(lds_wave + kKSlot, src, a.kv, kh, t_lo, wave, lane, pg_a, sh);
  int pg_b = scalar_page(src, t_lo + kBN);   // page of tile t + 1
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  // iteration i of the general kind, half i in buffer i & 1: scores of half i + 1, second product of
  // half i - 1, softmax of half i
  auto general_iter = [&](auto cur_tag, int i, int k_off, int v_off) __attribute__((always_inline)) {
    constexpr int cur = decltype(cur_tag)::value, nxt = cur ^ 1;  // half i lives in buffer i & 1
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (i + 1 < n_w) b[q].S[nxt] = qk_half(b[q], sh, k_off);
      if (i >= 1 && i - 1 < n_w) pv_half(b[q], sh, v_off, b[q].P[nxt]);
    }
    if (i >= 0 && i < n_w) {
      const bool need_mask = i < i_f0 || i >= i_f1;
#pragma unroll
      for (int q = 0; q < NQ; ++q)
        softmax_half_general(b[q].S[cur], b[q].S[nxt], b[q], need_mask, t_lo + 32 * i, h, W_, b[q].P[cur]);
    }
  };

  // step t: iterations 2t - 1 and 2t; with par = t & 1 it reads K tile t from K slot par and V tile
  // t - 1 from V slot 1 - par, fills K slot 1 - par with tile t + 1 and V slot par with tile t
  auto copies = [&](int t, int par) __attribute__((always_inline)) {
    if (t + 1 < nT)
      copy_rows<false>(lds_wave + kKSlot + (1 - par) * kTileB, src, a.kv, kh, t_lo + (t + 1) * kBN, wave, lane, pg_b, sh);
    if (t < nT) copy_rows<true>(lds_wave + kVSlot + par * kTileB, src, a.kv, vh, t_lo + t * kBN, wave, lane, pg_a, sh);
    pg_a = pg_b;
    if (t + 2 < nT) pg_b = scalar_page(src, t_lo + (t + 2) * kBN);
  };
  // Steps [t_fb, t_fe) of this wave are steady-state steps (no mask, every part present, the tiles
  // they copy lie completely inside the sequence); they run inside one assembly block.  All waves of
  // the workgroup run nT + 1 steps with one barrier each, whichever kind each wave's step is.
  const int t_fb = (max(i_f0, 1) + 2) >> 1;  // first t with 2t - 1 >= max(i_f0, 1)
  const int n_full = (w.kv_len - t_lo) >> 6;  // tiles completely inside the sequence
  const int t_fe = __builtin_amdgcn_readfirstlane(min((i_f1 + 1) >> 1, n_full - 1));  // 2t < i_f1, tile t + 1 is whole
  LoopScalars sc;
  sc.t_end = t_fe;
  sc.t_lo = __builtin_amdgcn_readfirstlane(t_lo);
  sc.pmask = src.page_size - 1;
  sc.pshift = src.page_shift;
  sc.tok_stride = a.kv.tok_stride;
  sc.last_tile_tok = __builtin_amdgcn_readfirstlane(src.last_tok & ~(kBN - 1));
  sc.pstr = (uint32_t)a.kv.page_stride;
  sc.kh_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)kh);
  sc.kh_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)kh >> 32));
  sc.vh_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)vh);
  sc.vh_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)vh >> 32));
  sc.lds_wave = lds_wave;
  sc.pages = src.pages;
  sc.limit = row_sum_limit;
  auto general_step = [&](int t) __attribute__((always_inline)) {
    const int par = t & 1;
    copies(t, par);
    const int k_off = par * kTileB, v_off = (1 - par) * kTileB;
    general_iter(std::integral_constant<int, 1>{}, 2 * t - 1, k_off, v_off);
    general_iter(std::integral_constant<int, 0>{}, 2 * t, k_off + kHalfB, v_off + kHalfB);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  };
  // Three phases, each a loop of its own (one loop that switches between the assembly block and the
  // general step would move the whole register state to a common place on every trip): general steps
  // up to the first steady-state step, the assembly loop, general steps to the end.
  const bool has_fast = t_fb < t_fe && row_sum_limit > -1.5f;  // (limit -2: a probe that keeps every step general)
  // Steps [t_mb, t_me): the ones behind the steady state that touch the causal diagonal, up to the wave's last
  // half, in the masked assembly loop (no window, or one far wider than a tile: the loop masks the diagonal only).
  // Every row has met a token it sees by then (half 0 at the latest, which step 0 takes), the tiles the steps copy
  // are whole, and halves past the wave's rows come out with every score masked, so they add nothing.
  int t_mb = nT + 1, t_me = nT + 1;
  if constexpr (NQ == 1) {
    // (without steady-state steps in front: only if the range starts at or before the wave's first row, so that
    // step 0 has shown every row a token and with it a real reference for its probabilities)
    const bool seen_early = W_ == 0 && t_lo <= w.prefix + r_lo;
    if (masked_steps && active && row_sum_limit > -1.5f && (W_ == 0 || W_ >= 4 * kBN) && (has_fast || seen_early)) {
      t_mb = has_fast ? t_fe : max(t_fb, 1);
      t_me = min(min(((n_w + 1) >> 1) + 1, n_full - 1), nT + 1);
    }
  }
  t_mb = __builtin_amdgcn_readfirstlane(t_mb);
  t_me = __builtin_amdgcn_readfirstlane(t_me);
  const bool has_masked = t_mb < t_me;
  const int t_first = has_fast ? t_fb : (has_masked ? t_mb : nT + 1);
  int t = 0;
  for (; t < t_first; ++t) general_step(t);
  if (has_fast) {
    pipe_loop(b, sh, t, pg_a, pg_b, sc);  // leaves t == t_fe
#pragma unroll
    for (int q = 0; q < NQ; ++q) b[q].seen = 1.0f;  // a steady-state half hides nothing from any row
  }
  if (has_masked) {
    sc.t_end = t_me;
    // (a piece of a K/V range may end in front of the diagonal: its end masks like a row's own position)
    pipe_loop_masked(b, sh, t, pg_a, pg_b, sc, min(b[0].qpos, t_hi - 1) - t_lo - 32 * (2 * t - 1) - 4 * h);  // leaves t == t_me
#pragma unroll
    for (int q = 0; q < NQ; ++q) b[q].seen = 1.0f;
  }
  if (has_fast || has_masked) {
    for (; t <= nT; ++t) general_step(t);
  }
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    WaveRows wr;
    wr.r_lo = r_lo + 32 * q;
    wr.r_hi = min(wr.r_lo + 31, w.q_len - 1);
    wr.active = wr.r_lo < w.q_len;
    wr.row = wr.r_lo + c;
    wr.qpos = b[q].qpos;
    if constexpr (SPLIT) write_partial_rows<4>(a, w, wr, b[q].O, b[q].l, h, b[q].seen != 0.f ? b[q].m : kNoReference, split);
    else write_rows<4>(a, w, wr, b[q].O, b[q].l, h, b[q].m);
  }
}

}  // namespace

// (what the assembly kernel can run is written down once, as the conditions of its rows in the shape table)
bool prefill_pipe_applies(const PrefillArgs& a) {
  return select_shape(prefill_shape_key(a)).kernel == kKernelPrefillPipe;
}

namespace {
int forced_nq() { return tuning().prefill_pipe_nq; }
// 32 positions x 4 heads per workgroup instead of 128 x 1: row "prefill_pipe_short" of the shape table
bool short_chunk_tile(const PrefillArgs& a, int nq) {
  return nq == 1 && select_shape(prefill_shape_key(a)).tile_q == 32;
}
}  // namespace

// Pieces per K/V range for a launch of the pipelined kernel (1 = whole ranges).
int prefill_pipe_kv_splits(const PrefillArgs& a, int nseq) {
  if (forced_nq() == 2) return 1;
  const bool heads4 = short_chunk_tile(a, 1);
  return kv_pieces(a, nseq, heads4 ? 32 : 128, heads4 ? 4 : 1, 0.8);
}

hipError_t launch_prefill_pipe(const PrefillArgs& a, int nseq, bool level_order, hipStream_t stream) {
  const int force_nq = forced_nq();
  // a half's row sum above the limit sends a wave through the rescaling path (testing knob: -1 = always)
  const float limit = tuning().prefill_pipe_limit != 0.f ? tuning().prefill_pipe_limit : kRowSumLimit;
  const bool masked = tuning().prefill_pipe_masked != 0;  // the steps on the causal diagonal in assembly too
  const int nq = force_nq ? force_nq : 1;
  // Tile by shape (the reference's per-shape block sizes, tuned_block_sizes.py, have this one counterpart
  // here): chunks of at most 64 tokens take 32 positions x 4 heads per workgroup when the heads come in fours
  const bool heads4 = short_chunk_tile(a, nq);
  const int bm = heads4 ? 32 : 128 * nq;
  int tiles = (a.max_q_len + bm - 1) / bm;
  const int levels = a.max_kv_len > 0 ? (a.max_kv_len + bm - 1) / bm + 1 : 0;
  const bool by_level = level_order && levels > tiles && levels <= 2 * tiles + 2;
  if (by_level) tiles = levels;
  const int64_t units = (int64_t)nseq * a.Hkv;
  const int64_t grid = (units >= 8 ? ((units + 7) / 8) * 8 : units) * (heads4 ? a.G / 4 : a.G) * tiles;
  if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
  const dim3 g((unsigned)grid), blk(256);
  const bool win = a.sm.window > 0;
  if (a.kv_splits > 1 && nq == 1) {  // pieces of the K/V ranges, then the merge
    if (!a.ws_o || !a.ws_ml || a.kv_splits > 64) return hipErrorInvalidValue;
    const dim3 gs((unsigned)grid, (unsigned)a.kv_splits);
#define RPA_LAUNCH_SPLIT(W, H4) \
  hipLaunchKernelGGL((rpa_prefill_pipe_kernel<W, 1, H4, true>), gs, blk, 0, stream, a, tiles, nseq, by_level, limit, masked)
    if (heads4) {
      if (win) RPA_LAUNCH_SPLIT(true, true);
      else RPA_LAUNCH_SPLIT(false, true);
    } else {
      if (win) RPA_LAUNCH_SPLIT(true, false);
      else RPA_LAUNCH_SPLIT(false, false);
    }
#undef RPA_LAUNCH_SPLIT
    return launch_prefill_combine(a, stream);
  }
#define RPA_LAUNCH(W, N) \
  hipLaunchKernelGGL((rpa_prefill_pipe_kernel<W, N>), g, blk, 0, stream, a, tiles, nseq, by_level, limit, masked)
  if (heads4) {
    if (win) hipLaunchKernelGGL((rpa_prefill_pipe_kernel<true, 1, true>), g, blk, 0, stream, a, tiles, nseq, by_level, limit, masked);
    else hipLaunchKernelGGL((rpa_prefill_pipe_kernel<false, 1, true>), g, blk, 0, stream, a, tiles, nseq, by_level, limit, masked);
  } else if (nq == 1) {
    if (win) RPA_LAUNCH(true, 1);
    else RPA_LAUNCH(false, 1);
  } else {
    if (win) RPA_LAUNCH(true, 2);
    else RPA_LAUNCH(false, 2);
  }
#undef RPA_LAUNCH
  return hipGetLastError();
}

}  // namespace rpa
