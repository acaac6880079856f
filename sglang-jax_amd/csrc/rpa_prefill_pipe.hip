// Software-pipelined flash kernel for the common prefill case on gfx950: bf16 cache, 128-wide
// heads, pages that hold whole 64-token tiles, causal mask (optionally with a sliding window),
// no score options.
//
// Work split and LDS layout are those of rpa_prefill_async_kernel (a workgroup of 4 waves owns
// 128 query rows of one query head, wave w owns 32 of them, K/V tiles of 64 tokens arrive through
// global_load_lds_dwordx4 into XOR-swizzled row-major LDS tiles).  What differs is the order of
// work inside a wave.  A 64-token tile is handled as two halves of 32 tokens, and iteration i
// holds three independent instruction streams:
//     matrix pipe   S(i+1) = K(i+1) . Q^T          8 MFMAs (one accumulator chain)
//     matrix pipe   O     += V(i-1)^T . P(i-1)^T   8 MFMAs (four accumulator chains)
//     vector pipe   P(i)   = 2^(S(i) c - m c)      exponentials, packing, row sum, row maximum
// so every vector instruction of the softmax has matrix instructions of the same wave to run
// under, instead of relying on another wave being in the other phase.  Step t of a workgroup is
// the pair of iterations (2t-1, 2t): it reads K tile t and V tile t-1, so two ring slots per
// matrix suffice (V lags K by one tile) and there is still one barrier per tile.
//
// The compiler does not keep such an interleave (it regroups the matrix instructions and spills),
// and it will not keep two hundred registers in place around an assembly block that is only a loop
// body, so the whole run of steady-state steps of a wave is one assembly block with fixed
// registers, written by gen_prefill_pipe_loop.py into rpa_prefill_pipe_loop.inc; this file binds
// the kernel's variables to those registers.  Steps that touch the causal diagonal or a window edge, the first and the
// last steps run the same pipeline through a general iteration in C++ with masking and run-time
// flags.
//
// The running maximum is checked after the fact: the exponentials of half i use the maximum known
// before it; the half's own maximum is taken by the vector pipe next to them, and only if it
// exceeds the stale one by more than 2^kMaxSlack is the half redone (its scores are still in
// registers) and the accumulators rescaled.
//
// The global -> LDS copies are issued as assembly too, so the compiler knows of no store into the
// LDS ring and never waits for the copy queue on its own; the kernel waits (vmcnt(0)) in front of
// the barrier that ends a step.

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

typedef uint32_t u32x16_t __attribute__((ext_vector_type(16)));
typedef int32_t i32x8_t __attribute__((ext_vector_type(8)));
typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4v_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ u32x4_t lds_ld16_at(int addr) {
  typedef const __attribute__((address_space(3))) u32x4_t* p_t;
  return *(p_t)(uint32_t)addr;
}
__device__ __forceinline__ u32x2_t lds_tr16_at(int addr) {
  typedef __attribute__((address_space(3))) s16x4v_t* p_t;
  return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((p_t)(uint32_t)addr));
}

template <int KS>
__device__ __forceinline__ u32x4_t q_frag(const u32x16_t& a, const u32x16_t& b) {
  const u32x16_t& s = KS < 4 ? a : b;
  constexpr int o = (KS & 3) * 4;
  return u32x4_t{s[o], s[o + 1], s[o + 2], s[o + 3]};
}

// The registers of one wave's pipeline.  The assembly loop expects them in the registers the
// RPA_PIPE_C_* constraints of rpa_prefill_pipe_loop.inc name.
struct Pipe {
  f32x16_t O[4];      // accumulators, lane (c, h): row c, dims 32d + 8*(v/4) + 4h + v%4
  f32x16_t S0, S1;    // scores of the even / odd half in flight
  u32x4_t P0[2], P1[2];  // probabilities of the even / odd half (B operands of the second product)
  u32x16_t Qa, Qb;    // Q^T operands of the 8 k-steps
  i32x8_t koff;       // LDS addresses of the K operand reads (slot 0, first half)
  i32x4_t voff;       // LDS addresses of the V^T operand reads (slot 0, first half, first k-step)
  float m, l;         // running maximum (raw score units), running sum
  u32x4_t ofs_k, ofs_v;  // per-lane byte offsets of this wave's four K / V copy instructions
  float sc2;          // raw score -> log2 units
};

// K or V rows of one tile, global -> LDS: 4 instructions per wave.  `lds_wave` is the LDS address
// of this wave's first 1 KiB block of the slot.
template <bool IS_V>
__device__ __forceinline__ void copy_rows(uint32_t lds_wave, const TileSrc& s, const KvAddr& kv, const char* head, int tb,
                                          int wave, int lane, int page, const AsyncOffsets<128>& ofs) {
  tb = min(tb, s.last_tok & ~(kBN - 1));
  if (tb + kBN - 1 <= s.last_tok) {
    const int64_t base = (int64_t)page * kv.page_stride + (int64_t)(tb - page_slot(s, tb) * s.page_size) * kv.tok_stride;
    const char* b = head + base;  // wave-uniform
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :: "s"(lds_wave + n * 1024), "v"(IS_V ? ofs.v[n] : ofs.k[n]), "s"(b)
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

// first product of one 32-token half: one chain of 8 MFMAs; `off` = slot and half offset
__device__ __forceinline__ f32x16_t qk_half(const Pipe& p, int off) {
  f32x16_t S = mfma32(lds_ld16_at(p.koff[0] + off), q_frag<0>(p.Qa, p.Qb), kZero16);
  S = mfma32(lds_ld16_at(p.koff[1] + off), q_frag<1>(p.Qa, p.Qb), S);
  S = mfma32(lds_ld16_at(p.koff[2] + off), q_frag<2>(p.Qa, p.Qb), S);
  S = mfma32(lds_ld16_at(p.koff[3] + off), q_frag<3>(p.Qa, p.Qb), S);
  S = mfma32(lds_ld16_at(p.koff[4] + off), q_frag<4>(p.Qa, p.Qb), S);
  S = mfma32(lds_ld16_at(p.koff[5] + off), q_frag<5>(p.Qa, p.Qb), S);
  S = mfma32(lds_ld16_at(p.koff[6] + off), q_frag<6>(p.Qa, p.Qb), S);
  S = mfma32(lds_ld16_at(p.koff[7] + off), q_frag<7>(p.Qa, p.Qb), S);
  return S;
}

// second product of one 32-token half: four chains of 2 MFMAs
__device__ __forceinline__ void pv_half(Pipe& p, int off, const u32x4_t (&P)[2]) {
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int vt = p.voff[d] + off + kk * 16 * kRowB;
      const u32x2_t lo = lds_tr16_at(vt);
      const u32x2_t hi = lds_tr16_at(vt + 8 * kRowB);
      p.O[d] = mfma32(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, P[kk], p.O[d]);
    }
}

// probabilities of 16 scores against a fixed reference: P = bf16(2^(S sc2 + neg_m)), their sum
__device__ __forceinline__ float exp_pack(const f32x16_t& S, float sc2, float neg_m, u32x4_t (&P)[2]) {
  const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
  float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float p0 = fast_exp2(__builtin_fmaf(S[8 * kk + 2 * j], sc2, neg_m));
      const float p1 = fast_exp2(__builtin_fmaf(S[8 * kk + 2 * j + 1], sc2, neg_m));
      w[j] = pack_bf16x2(p0, p1);
      if (j & 1) ps1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[j]), ones, ps1, false);
      else ps0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[j]), ones, ps0, false);
    }
    P[kk] = u32x4_t{w[0], w[1], w[2], w[3]};
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

// softmax of a half with the maximum taken first (first half of a row, masked halves)
__device__ __forceinline__ void softmax_half_general(f32x16_t& S, Pipe& p, bool need_mask, int tb, int h, int qpos,
                                                     int window, u32x4_t (&P)[2]) {
  if (need_mask) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int tok = tb + 8 * (v >> 2) + 4 * h + (v & 3);
      const bool masked = tok > qpos || (window > 0 && tok <= qpos - window);
      S[v] = masked ? kMaskRaw : S[v];
    }
  }
  const float mx = row_max16(S);
  if (__builtin_amdgcn_ballot_w64((mx - p.m) * p.sc2 > kMaxSlack) != 0) {
    const float m_new = fmaxf(p.m, mx);
    const float alpha = fast_exp2((p.m - m_new) * p.sc2);
    p.m = m_new;
    p.l *= alpha;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) p.O[d][v] *= alpha;
  }
  p.l += exp_pack(S, p.sc2, -p.m * p.sc2, P);
}

// Steady-state steps [t, t_end) in assembly.  On entry K tile t is in K slot t & 1 and V tile t - 1
// in V slot 1 - (t & 1), pg_a / pg_b are the pages of tiles t and t + 1; on exit the same holds for
// t = t_end.  Every tile the loop copies (up to t_end) lies completely inside the sequence.
struct LoopScalars {
  int t_end, t_lo, pmask, pshift, tok_stride, last_tile_tok;
  uint32_t pstr, kh_lo, kh_hi, vh_lo, vh_hi, lds_wave;
  const int32_t* pages;
};

#define RPA_PIPE_LOOP(p, t, pg_a, pg_b, sc)                                                                       \
  asm volatile(RPA_PIPE_LOOP_ASM                                                                                  \
               : "+" RPA_PIPE_C_O0(p.O[0]), "+" RPA_PIPE_C_O1(p.O[1]), "+" RPA_PIPE_C_O2(p.O[2]),                 \
                 "+" RPA_PIPE_C_O3(p.O[3]), "+" RPA_PIPE_C_S0(p.S0), "+" RPA_PIPE_C_S1(p.S1),                     \
                 "+" RPA_PIPE_C_P00(p.P0[0]), "+" RPA_PIPE_C_P01(p.P0[1]), "+" RPA_PIPE_C_P10(p.P1[0]),           \
                 "+" RPA_PIPE_C_P11(p.P1[1]), "+" RPA_PIPE_C_M(p.m), "+" RPA_PIPE_C_L(p.l),                       \
                 [t] "+s"(t), [pg_a] "+s"(pg_a), [pg_b] "+s"(pg_b)                                                \
               : RPA_PIPE_C_QA(p.Qa), RPA_PIPE_C_QB(p.Qb), RPA_PIPE_C_KOFF(p.koff), RPA_PIPE_C_VOFF(p.voff),      \
                 RPA_PIPE_C_OFSK(p.ofs_k), RPA_PIPE_C_OFSV(p.ofs_v), [sc2] "s"(p.sc2), [nsc2] "s"(-p.sc2),        \
                 [ones] "s"(0x3f803f80u), [t_end] "s"(sc.t_end), [t_lo] "s"(sc.t_lo), [pmask] "s"(sc.pmask),      \
                 [pshift] "s"(sc.pshift), [tok_stride] "s"(sc.tok_stride), [last_tile_tok] "s"(sc.last_tile_tok), \
                 [pstr] "s"(sc.pstr), [kh_lo] "s"(sc.kh_lo), [kh_hi] "s"(sc.kh_hi), [vh_lo] "s"(sc.vh_lo),        \
                 [vh_hi] "s"(sc.vh_hi), [lds_wave] "s"(sc.lds_wave), [pages] "s"(sc.pages)                        \
               : RPA_PIPE_LOOP_CLOBBERS)

template <bool WIN>
__global__ __launch_bounds__(256, 2) void rpa_prefill_pipe_kernel(const PrefillArgs a, int tiles, int nseq, bool by_level) {
  __shared__ __attribute__((aligned(1024))) char lds[4 * kTileB];

  const Work w = decompose(a, tiles, nseq, by_level);
  if (!w.valid) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, h = lane >> 5;
  const TileSrc src = make_src(a, w);
  const char* kh = a.kv.k_base + (int64_t)w.hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)w.hk * a.kv.head_stride;
  typedef __attribute__((address_space(3))) char* lds_ptr_t;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)lds);

  WaveRows wr;
  wr.r_lo = w.q_start + wave * 32;
  wr.r_hi = min(wr.r_lo + 31, w.q_len - 1);
  wr.active = wr.r_lo < w.q_len;
  wr.row = wr.r_lo + c;
  wr.qpos = w.prefix + wr.row;
  const int W_ = WIN ? a.sm.window : 0;

  Pipe p;
  {
    const int rr = min(wr.row, w.q_len - 1);
    const uint16_t* qp = a.q + ((int64_t)(w.qg0 + rr) * a.Hq + w.head) * 128 + h * 8;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const u32x4_t x = ld16(qp + ks * 16), y = ld16(qp + (ks + 4) * 16);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        p.Qa[4 * ks + e] = x[e];
        p.Qb[4 * ks + e] = y[e];
      }
    }
  }
  p.sc2 = a.sm.sm_scale * (a.k_scale ? a.k_scale[w.hk] : 1.0f) * kLog2e;
#pragma unroll
  for (int d = 0; d < 4; ++d) p.O[d] = kZero16;
  p.S0 = kZero16;
  p.S1 = kZero16;
  p.P0[0] = p.P0[1] = p.P1[0] = p.P1[1] = u32x4_t{0, 0, 0, 0};
  p.m = kMaxFloor;
  p.l = 0.f;

  const int wg_r_hi = min(w.q_start + kBM, w.q_len) - 1;
  const int t_hi = min(w.kv_len, w.prefix + wg_r_hi + 1);  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, w.prefix + w.q_start - W_ + 1) & ~(kBN - 1);
  const int nT = (t_hi - t_lo + kBN - 1) / kBN;  // K/V tiles of the workgroup

  // halves [0, n_w) of 32 tokens concern this wave; halves [i_f0, i_f1) need no mask
  int n_w = 0, i_f0 = 0, i_f1 = 0;
  if (wr.active) {
    n_w = (min(w.kv_len, w.prefix + wr.r_hi + 1) - t_lo + 31) >> 5;
    i_f1 = max(0, (w.prefix + wr.r_lo - t_lo + 1) >> 5);
    if (W_ > 0) {
      const int y = w.prefix + wr.r_hi - W_ - t_lo;
      i_f0 = y >= 0 ? (y >> 5) + 1 : 0;
    }
    i_f1 = min(i_f1, n_w);
  }
  n_w = __builtin_amdgcn_readfirstlane(n_w);
  i_f0 = __builtin_amdgcn_readfirstlane(i_f0);
  i_f1 = __builtin_amdgcn_readfirstlane(i_f1);

  // operand addresses inside the LDS array (see rpa_prefill_async_kernel for the swizzles)
  {
    const int k_row = c * kRowB;
    const int k_swz = (h ^ (c & 15)) << 4;
    const int r16 = lane & 15, b16 = lane >> 4;
    const int v_row = (4 * h + (r16 >> 2)) * kRowB;
    const int v_in = ((b16 & 1) << 5) + (((r16 & 3) >> 1) << 4) + ((r16 & 1) << 3);
    const int v_swz = (r16 >> 2) << 6;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) p.koff[ks] = (int)lds_base + kKSlot + k_row + ((ks * 32) ^ k_swz);
#pragma unroll
    for (int d = 0; d < 4; ++d) p.voff[d] = (int)lds_base + kVSlot + v_row + v_in + ((d * 64) ^ v_swz);
  }

  const AsyncOffsets<128> ofs = make_async_offsets<128>(a.kv, wave, lane);
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    p.ofs_k[n] = ofs.k[n];
    p.ofs_v[n] = ofs.v[n];
  }
  const uint32_t lds_wave = lds_base + wave * 4096;  // this wave's four 1 KiB blocks of slot K0
  int pg_a = scalar_page(src, t_lo);         // page of tile t
  copy_rows<false>(lds_wave + kKSlot, src, a.kv, kh, t_lo, wave, lane, pg_a, ofs);
  int pg_b = scalar_page(src, t_lo + kBN);   // page of tile t + 1
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  // iteration i of the general kind: Sn <- scores of half i + 1, Pc <- softmax of Sc (half i), O += P(i - 1) V
  auto general_iter = [&](int i, f32x16_t& Sc, f32x16_t& Sn, u32x4_t (&Pc)[2], const u32x4_t (&Pp)[2], int k_off,
                          int v_off) __attribute__((always_inline)) {
    if (i + 1 < n_w) Sn = qk_half(p, k_off);
    if (i >= 1 && i - 1 < n_w) pv_half(p, v_off, Pp);
    if (i >= 0 && i < n_w) {
      const bool need_mask = i < i_f0 || i >= i_f1;
      softmax_half_general(Sc, p, need_mask, t_lo + 32 * i, h, wr.qpos, W_, Pc);
    }
  };

  // step t: iterations 2t - 1 and 2t; with par = t & 1 it reads K tile t from K slot par and V tile
  // t - 1 from V slot 1 - par, fills K slot 1 - par with tile t + 1 and V slot par with tile t
  auto copies = [&](int t, int par) __attribute__((always_inline)) {
    if (t + 1 < nT)
      copy_rows<false>(lds_wave + kKSlot + (1 - par) * kTileB, src, a.kv, kh, t_lo + (t + 1) * kBN, wave, lane, pg_b, ofs);
    if (t < nT) copy_rows<true>(lds_wave + kVSlot + par * kTileB, src, a.kv, vh, t_lo + t * kBN, wave, lane, pg_a, ofs);
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
  int t = 0;
  while (t <= nT) {
    if (t >= t_fb && t < t_fe) {
      RPA_PIPE_LOOP(p, t, pg_a, pg_b, sc);  // leaves t == t_fe
    } else {
      const int par = t & 1;
      copies(t, par);
      const int i = 2 * t - 1;
      const int k_off = par * kTileB, v_off = (1 - par) * kTileB;
      general_iter(i, p.S1, p.S0, p.P1, p.P0, k_off, v_off);
      general_iter(i + 1, p.S0, p.S1, p.P0, p.P1, k_off + kHalfB, v_off + kHalfB);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      ++t;
    }
  }
  write_rows<4>(a, w, wr, p.O, p.l, h, p.m * p.sc2);
}

}  // namespace

bool prefill_pipe_applies(const PrefillArgs& a) {
  const int P = a.pt.page_size;
  return !a.fp8 && a.head_dim == 128 && P >= kBN && (P & (P - 1)) == 0 && a.kv.page_stride < (int64_t(1) << 32) &&
         a.sm.mask_mode == 0 && a.sm.soft_cap == 0.f &&
         a.sm.round_logits == 0 && !(a.sm.xai_len > 0.f) && !(a.sm.q_scale > 0.f);
}

hipError_t launch_prefill_pipe(const PrefillArgs& a, int tiles, int nseq, bool by_level, unsigned grid, hipStream_t stream) {
  const dim3 g(grid), blk(256);
  if (a.sm.window > 0) hipLaunchKernelGGL((rpa_prefill_pipe_kernel<true>), g, blk, 0, stream, a, tiles, nseq, by_level);
  else hipLaunchKernelGGL((rpa_prefill_pipe_kernel<false>), g, blk, 0, stream, a, tiles, nseq, by_level);
  return hipGetLastError();
}

}  // namespace rpa
