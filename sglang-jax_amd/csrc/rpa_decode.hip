// Split-KV decode for ragged paged attention on gfx950, plus the combine pass,
// the page-table gather and the new-token cache write.
//
// Decode is HBM-bound: every visible KV token is read exactly once.  One
// wavefront owns one (sequence, kv head, kv split) and streams that head's K
// and V rows (adjacent in the head-interleaved cache: K_h | V_h = 2*D elements)
// through the page table with 16-byte loads straight into the MFMA operand
// layout -- no LDS, no barriers, so every wave is independent and the grid is
// just "enough waves to keep ~16 KiB per wave in flight on every SIMD".
//
// Per 32-token block (bf16):
//   S^T[tok, qrow] = K[tok, :] . Q^T        2 x 4 MFMA 16x16x32 (A = K, B = Q^T)
//   online softmax on the 8 scores each lane holds (row stats need one
//   cross-lane max over the 4 lane groups)
//   O^T[dim, qrow] += V^T[dim, tok] . P^T   8 MFMA 16x16x32 (A = V^T, B = P^T)
// The S^T result layout (lane = q row, registers = tokens) is already the B
// operand layout of the second product when the 32 tokens of a block are
// enumerated as slot(g, i) = (i < 4 ? 4g + i : 16 + 4g + i - 4); V is loaded in
// that token order and transposed in registers with v_perm_b32 (two bf16 of
// neighbouring tokens -> one dword), 32 permutes per block.
// GQA: the G query heads of a kv head are the (zero padded) 16 columns of Q^T.

#include <cstdlib>

#include "rpa_common.h"
#include "rpa_kernels.h"

// The K / V rows a decode wave streams are read exactly once per launch: non-temporal loads (the `nt` bit: the
// lines are the first to leave the L2 and the memory-side cache again instead of pushing out what is reused).
// C2's decode rows 103.6 -> 90.6 us, C3 360 -> 327 us, C4 238 -> 214 us; -DRPA_DECODE_NT=0 repeats the comparison.
#ifndef RPA_DECODE_NT
#define RPA_DECODE_NT 1
#endif
#if RPA_DECODE_NT
#define RPA_KV_LD16(p) __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p))
#define RPA_KV_LD8(p) __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p))
#else
#define RPA_KV_LD16(p) ld16(p)
#define RPA_KV_LD8(p) ld8(p)
#endif

namespace rpa {

namespace {

constexpr int kBlk = 32;

__device__ __forceinline__ int tok_slot(int g, int i) {
  return (i < 4) ? (g * 4 + i) : (16 + g * 4 + (i - 4));
}

template <bool FP8>
struct KvRegs;
template <>
struct KvRegs<false> {
  u32x4_t k[2][4];  // [token half][k step]: 8 bf16 of dims 32*s + 8*g ..
  u32x4_t v[8];     // [slot]: 8 bf16 of dims 8*c ..
};
template <>
struct KvRegs<true> {
  u32x4_t k[2][2];  // 32 fp8 of dims 32*g ..
  u32x2_t v[8];     // 8 fp8 of dims 8*c ..
};

struct SeqView {
  const int32_t* pages;  // this sequence's page ids
  int32_t page_size;
  int32_t page_shift;  // >= 0 when page_size is a power of two
  int32_t last_tok;    // kv_len - 1
};

__device__ __forceinline__ int page_slot_of(const SeqView& s, int tok) {
  return s.page_shift >= 0 ? (tok >> s.page_shift) : (tok / s.page_size);
}

// Issue the global loads of one 32-token block.  Token indices are clamped to
// the last valid token so that nothing past kv_len (and nothing past the
// sequence's page list) is ever dereferenced; clamped rows are masked later.
// WINDOW, win / win_first: for pages that do not hold whole blocks, the LDS window the caller keeps of this
// row's page ids (entry 0 = page slot win_first); without it every lane fetches the ids of its tokens from
// memory, a dependent round trip in front of the block's loads.
// (A compile-time choice: with both lookups in the code the compiler's wait-count bookkeeping sees a possible
// page-id load behind every block and drains the whole queue in front of each block's use.)
template <bool FP8, bool UNIFORM_PAGE, bool WINDOW = false>
__device__ __forceinline__ void load_block(KvRegs<FP8>& r, const SeqView& s, const KvAddr& kv,
                                           const char* kh, const char* vh, int tb, int page, int c, int g,
                                           const int32_t* win = nullptr, int win_first = 0) {
  constexpr int kLaneK = FP8 ? 32 : 16;  // byte offset step of lane group g inside a K row
  constexpr int kLaneV = FP8 ? 8 : 16;   // byte offset step of lane c inside a V row
  if constexpr (UNIFORM_PAGE) {
    // the whole block lies in one page whose id the caller fetched a block ahead
    const int slot = page_slot_of(s, tb);
    const char* kp = kh + (int64_t)page * kv.page_stride;
    const char* vp = vh + (int64_t)page * kv.page_stride;
    const int t0 = slot * s.page_size;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int tin = min(tb + b * 16 + c, s.last_tok) - t0;
      const uint32_t off = (uint32_t)(tin * kv.tok_stride + g * kLaneK);
      if constexpr (FP8) {
        r.k[b][0] = RPA_KV_LD16(kp + off);
        r.k[b][1] = RPA_KV_LD16(kp + off + 16);
      } else {
#pragma unroll
        for (int st = 0; st < 4; ++st) r.k[b][st] = RPA_KV_LD16(kp + off + st * 64);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tin = min(tb + tok_slot(g, i), s.last_tok) - t0;
      const uint32_t off = (uint32_t)(tin * kv.tok_stride + c * kLaneV);
      if constexpr (FP8) r.v[i] = RPA_KV_LD8(vp + off);
      else r.v[i] = RPA_KV_LD16(vp + off);
    }
  } else {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int tok = min(tb + b * 16 + c, s.last_tok);
      const int slot = page_slot_of(s, tok);
      const int page = WINDOW ? win[slot - win_first] : s.pages[slot];
      const char* kp = kh + (int64_t)page * kv.page_stride +
                       (int64_t)((tok - slot * s.page_size) * kv.tok_stride + g * kLaneK);
      if constexpr (FP8) {
        r.k[b][0] = RPA_KV_LD16(kp);
        r.k[b][1] = RPA_KV_LD16(kp + 16);
      } else {
#pragma unroll
        for (int st = 0; st < 4; ++st) r.k[b][st] = RPA_KV_LD16(kp + st * 64);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tok = min(tb + tok_slot(g, i), s.last_tok);
      const int slot = page_slot_of(s, tok);
      const int page = WINDOW ? win[slot - win_first] : s.pages[slot];
      const char* vp = vh + (int64_t)page * kv.page_stride +
                       (int64_t)((tok - slot * s.page_size) * kv.tok_stride + c * kLaneV);
      if constexpr (FP8) r.v[i] = RPA_KV_LD8(vp);
      else r.v[i] = RPA_KV_LD16(vp);
    }
  }
}

struct ScoreOpts {
  float scale;      // sm_scale * k_scale            (soft-cap path)
  float scale2;     // sm_scale * k_scale * log2(e)  (plain path)
  float cap, inv_cap;
  float temp;       // temperature factor                (soft-cap path; the plain path folds it into scale2)
  int round_mode;   // logits rounded to bf16 (1) or f16 (2) before the softmax (soft-cap path)
  float mask2;      // mask value in log2 units (finite)
  int t_lo;         // first visible token (sliding window), 0 otherwise
  int kv_len;
};

// K operands (A of S^T = K Q^T) of one 32-token block: [token half][k step]
template <bool FP8>
__device__ __forceinline__ void k_operands(const KvRegs<FP8>& r, u32x4_t (&kA)[2][4]) {
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    if constexpr (FP8) {
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const uint32_t w0 = r.k[b][st >> 1][(st & 1) * 2 + 0];
        const uint32_t w1 = r.k[b][st >> 1][(st & 1) * 2 + 1];
        const u32x2_t lo = fp8x4_to_bf16x4(w0);
        const u32x2_t hi = fp8x4_to_bf16x4(w1);
        kA[b][st] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
      }
    } else {
#pragma unroll
      for (int st = 0; st < 4; ++st) kA[b][st] = r.k[b][st];
    }
  }
}

// V^T operands (A of O^T = V^T P^T), one per output dim j of the lane's 8-dim chunk
template <bool FP8>
__device__ __forceinline__ void v_operands(const KvRegs<FP8>& r, u32x4_t (&vA)[8]) {
  if constexpr (FP8) {
    // r.v[i] = 8 fp8 (dims 8c .. 8c+7) of token slot i.  A byte permute first pairs the bytes of
    // two neighbouring tokens for two dims (t0 d, t1 d, t0 d+1, t1 d+1), then each half converts
    // straight to a bf16 pair: 3 instructions per 4 values.
#pragma unroll
    for (int tp = 0; tp < 4; ++tp)
#pragma unroll
      for (int dp = 0; dp < 4; ++dp) {
        const uint32_t lo_tok = r.v[2 * tp][dp >> 1], hi_tok = r.v[2 * tp + 1][dp >> 1];
        // selector bytes: 0-3 pick from lo_tok (second operand), 4-7 from hi_tok (first operand)
        const uint32_t sel = (dp & 1) ? 0x07030602u : 0x05010400u;
        const uint32_t mixed = __builtin_amdgcn_perm(hi_tok, lo_tok, sel);
        vA[2 * dp][tp] = fp8x2_to_bf16x2(mixed, false);
        vA[2 * dp + 1][tp] = fp8x2_to_bf16x2(mixed, true);
      }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      const int jj = j >> 1;
      vA[j] = u32x4_t{__builtin_amdgcn_perm(r.v[1][jj], r.v[0][jj], sel),
                      __builtin_amdgcn_perm(r.v[3][jj], r.v[2][jj], sel),
                      __builtin_amdgcn_perm(r.v[5][jj], r.v[4][jj], sel),
                      __builtin_amdgcn_perm(r.v[7][jj], r.v[6][jj], sel)};
    }
  }
}

template <int MT, bool FP8, bool CAP>
__device__ __forceinline__ void compute_block(const KvRegs<FP8>& r, const u32x4_t (&qB)[MT][4],
                                              f32x4_t (&acc)[MT][8], float (&m)[MT], float (&l)[MT],
                                              const ScoreOpts& so, int tb, int g) {
  u32x4_t kA[2][4];
  k_operands<FP8>(r, kA);
  u32x4_t vA[8];
  v_operands<FP8>(r, vA);
  const bool need_mask = (tb + kBlk > so.kv_len) || (tb < so.t_lo);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    f32x4_t s[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      s[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < 4; ++st) s[b] = mfma16(kA[b][st], qB[mt][st], s[b]);
    }
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = s[i >> 2][i & 3];
      if constexpr (CAP) {
        // the general path: soft cap (if any), temperature, rounding of the logit (if asked)
        v = v * so.scale;
        if (so.cap != 0.f) v = soft_cap_f(v, so.cap, so.inv_cap);
        v = v * so.temp;
        if (so.round_mode) v = round_logit(v, so.round_mode);
        v = v * kLog2e;
      } else {
        v = v * so.scale2;
      }
      x[i] = v;
    }
    if (need_mask) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int tok = tb + tok_slot(g, i);
        if (tok >= so.kv_len || tok < so.t_lo) x[i] = so.mask2;
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])),
                     fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m[mt], mx);
    const float alpha = fast_exp2(m[mt] - m_new);
    float p[8];
    float ps = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      p[i] = fast_exp2(x[i] - m_new);
      ps += p[i];
    }
    l[mt] = l[mt] * alpha + ps;
    m[mt] = m_new;
    const u32x4_t pB = u32x4_t{pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]),
                               pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7])};
    if constexpr (FP8) {
      // fp8 blocks are VALU-bound (dequantisation): skip the accumulator rescale unless the
      // running max moved in some lane, which is rare after the first blocks
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[mt][j] = acc[mt][j] * alpha;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[mt][j] = mfma16(vA[j], pB, acc[mt][j]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        acc[mt][j] = acc[mt][j] * alpha;
        acc[mt][j] = mfma16(vA[j], pB, acc[mt][j]);
      }
    }
  }
}

__device__ __forceinline__ int first_block_token(int kv_len, int window) {
  const int t_lo = (window > 0) ? max(0, kv_len - window) : 0;
  return t_lo & ~(kBlk - 1);
}

// Where a wave leaves the result of one piece of work: the finished bf16 rows in `out`, or
// unnormalised partial rows plus (max, sum) in the workspace, slot `base` + query head
// (fixed split plan) or `base` + row inside the group of 16 (balanced plan).
struct PartDest {
  bool final_rows;
  bool by_head;
  int64_t base;
};

// Q^T operands of one (query token, kv head, group of 16 query heads): column c = query head
// row0 + 16*mt + c of the kv head, zero beyond the G real ones.
template <int MT, bool FP8>
__device__ __forceinline__ void load_queries(const DecodeArgs& a, int tq, int hk, int row0, int c, int g,
                                             u32x4_t (&qB)[MT][4]) {
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = row0 + mt * 16 + c;
    const uint16_t* qp = a.q + ((int64_t)tq * a.Hq + (int64_t)hk * a.G + row) * 128;
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const int d0 = FP8 ? (g * 32 + st * 8) : (st * 32 + g * 8);
      qB[mt][st] = (row < a.G) ? ld16(qp + d0) : u32x4_t{0u, 0u, 0u, 0u};
    }
  }
}

template <int MT, bool FP8>
__device__ __forceinline__ void requantise_queries(const DecodeArgs& a, u32x4_t (&qB)[MT][4]) {
  if (a.sm.q_scale > 0.f) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int st = 0; st < 4; ++st) qB[mt][st] = requantise_q(qB[mt][st], a.sm.q_scale, FP8);
  }
}

// Leave the result of one piece of work: lane (c, g) holds q row c, dims 32g + 8r + j in
// acc[mt][j][r].
template <int MT, bool THROUGH = false>
__device__ __forceinline__ void write_rows(const DecodeArgs& a, const f32x4_t (&acc)[MT][8], const float (&m)[MT],
                                           const float (&l)[MT], int tq, int hk, int row0, const PartDest dest,
                                           int c, int g) {
  const float vs = a.v_scale ? a.v_scale[hk] : 1.0f;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float lt = l[mt];
    lt += __shfl_xor(lt, 16);
    lt += __shfl_xor(lt, 32);
    const int row = row0 + mt * 16 + c;
    if (row >= a.G) continue;
    const int head = hk * a.G + row;
    if (dest.final_rows) {
      const float inv = a.sm.sink ? vs * sink_inverse(m[mt], lt, sink_logit(a.sm.sink, a.sm.round_logits, head)) : vs / lt;
      uint16_t* op = a.out + ((int64_t)tq * a.Hq + head) * 128 + g * 32;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        u32x4_t w;
#pragma unroll
        for (int jp = 0; jp < 4; ++jp)
          w[jp] = pack_bf16x2(acc[mt][2 * jp][r] * inv, acc[mt][2 * jp + 1][r] * inv);
        st16(op + r * 8, w);
      }
    } else {
      const int64_t slot = dest.base + (dest.by_head ? head : row - row0);
      float* wo = a.ws_o + slot * 128 + g * 32;
      // merged inside the same launch: the rows are written through to device scope, so that the
      // merging wave (on another part of the GPU, behind another L2) reads them without any
      // cache-wide write-back or invalidate
      constexpr bool through = THROUGH;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        f32x4_t w0 = {acc[mt][0][r] * vs, acc[mt][1][r] * vs, acc[mt][2][r] * vs, acc[mt][3][r] * vs};
        f32x4_t w1 = {acc[mt][4][r] * vs, acc[mt][5][r] * vs, acc[mt][6][r] * vs, acc[mt][7][r] * vs};
        if (through) {
          asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(wo + r * 8), "v"(w0) : "memory");
          asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(wo + r * 8 + 4), "v"(w1) : "memory");
        } else {
          *reinterpret_cast<f32x4_t*>(wo + r * 8) = w0;
          *reinterpret_cast<f32x4_t*>(wo + r * 8 + 4) = w1;
        }
      }
      if (g == 0) {
        if (through) {
          __hip_atomic_store(a.ws_ml + slot * 2 + 0, m[mt], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(a.ws_ml + slot * 2 + 1, lt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          a.ws_ml[slot * 2 + 0] = m[mt];
          a.ws_ml[slot * 2 + 1] = lt;
        }
      }
    }
  }
}

// One wave, one (sequence, kv head, group of 16 query heads), tokens [t_begin, t_end).
template <int MT, bool FP8, bool UNIFORM_PAGE, bool CAP>
__device__ __forceinline__ void decode_segment(const DecodeArgs& a, int seq, int hk, int rg, int kv_len, int t_lo,
                                               int t_begin, int t_end, const PartDest dest, int lane) {
  const int c = lane & 15, g = lane >> 4;
  const int nblk = (t_end - t_begin + kBlk - 1) / kBlk;

  SeqView sv;
  sv.page_size = a.pt.page_size;
  sv.page_shift = ((sv.page_size & (sv.page_size - 1)) == 0) ? (31 - __builtin_clz(sv.page_size)) : -1;
  sv.last_tok = kv_len - 1;
  // Sequence metadata and page ids go through the scalar cache: nothing writes them while the
  // kernel runs, and a scalar load is not counted by vmcnt, so waiting for a page id never
  // drains the block prefetch issued just before it.
  seq = __builtin_amdgcn_readfirstlane(seq);
  sv.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (scalar_load_i32(a.pt.cu_kv_lens + seq) / a.pt.page_size)
                                                  : (int64_t)seq * a.pt.pages_per_seq);

  const char* kh = a.kv.k_base + (int64_t)hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)hk * a.kv.head_stride;

  // ---- Q^T operands: column c = query head (row0 + 16*mt + c) of this kv head ----
  const int tq = scalar_load_i32(a.pt.cu_q_lens + seq);
  const int row0 = rg * 16 * MT;
  u32x4_t qB[MT][4];
  load_queries<MT, FP8>(a, tq, hk, row0, c, g, qB);
  requantise_queries<MT, FP8>(a, qB);

  ScoreOpts so;
  const float ks = a.k_scale ? a.k_scale[hk] : 1.0f;
  // the one query of a decode row sits at position kv_len - 1
  const float temp = xai_factor(kv_len - 1, a.sm.xai_len);
  so.scale = a.sm.sm_scale * ks * (a.sm.q_scale > 0.f ? a.sm.q_scale : 1.0f);
  so.scale2 = so.scale * kLog2e * temp;
  so.temp = temp;
  so.round_mode = a.sm.round_logits;
  so.cap = a.sm.soft_cap;
  so.inv_cap = (so.cap != 0.f) ? 1.0f / so.cap : 0.f;
  so.mask2 = fmaxf(a.sm.mask_value * kLog2e, -3.0e38f);
  so.t_lo = t_lo;
  so.kv_len = kv_len;

  f32x4_t acc[MT][8];
  float m[MT], l[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    m[mt] = -INFINITY;
    l[mt] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[mt][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // ---- software pipeline: the loads of block i+1 are in flight while block i is consumed.
  // The prefetch is unconditional (past the end it re-reads the last block) so that the
  // number of outstanding loads is the same on every path and the waits stay partial; the
  // page id of block i+2 is fetched while block i is consumed.
  const int t_last = t_begin + (nblk - 1) * kBlk;
  auto block_tok = [&](int b) { return min(t_begin + b * kBlk, t_last); };
  auto page_of = [&](int tb) -> int {
    if constexpr (UNIFORM_PAGE) return scalar_load_i32(sv.pages + __builtin_amdgcn_readfirstlane(page_slot_of(sv, tb)));
    else return 0;
  };
  // Pages smaller than a block: the ids of the next kWinSmallPages pages wait in the wave's LDS window and
  // every lane looks its token rows up there; fetched from memory per block they were a dependent round
  // trip in front of every block's loads, behind which the loads already in flight had to drain (page size
  // 16: 2.6 TB/s where pages of 64 stream 5.8).  The window moves on every kWinSmallPages pages, at the
  // price of one drained queue.
  __shared__ int32_t seg_windows[UNIFORM_PAGE ? 1 : 4][UNIFORM_PAGE ? 1 : kWinSmallPages];  // [wave][entry]
  const int32_t* win = nullptr;
  int win_first = 0;
  auto cover = [&](int tb) __attribute__((always_inline)) {  // make the window hold the pages of block tb
    if constexpr (!UNIFORM_PAGE) {
      const int last_slot = page_slot_of(sv, sv.last_tok);
      if (!win || page_slot_of(sv, min(tb + kBlk - 1, sv.last_tok)) - win_first >= kWinSmallPages) {
        int32_t* mine = seg_windows[__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)];
        win_first = __builtin_amdgcn_readfirstlane(page_slot_of(sv, tb));
        copy_page_window<kWinSmallPages>(sv.pages, last_slot, mine, win_first, lane);
        wait_all_loads();
        win = mine;
      }
    }
  };
  KvRegs<FP8> ra, rb;
  int pg_next = page_of(block_tok(1));
  cover(t_begin);
  load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(ra, sv, a.kv, kh, vh, t_begin, page_of(t_begin), c, g, win, win_first);
  for (int blk = 0; blk < nblk; blk += 2) {
    cover(block_tok(blk + 1));
    load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(rb, sv, a.kv, kh, vh, block_tok(blk + 1), pg_next, c, g, win, win_first);
    pg_next = page_of(block_tok(blk + 2));
    compute_block<MT, FP8, CAP>(ra, qB, acc, m, l, so, t_begin + blk * kBlk, g);
    if (blk + 1 >= nblk) break;
    cover(block_tok(blk + 2));
    load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(ra, sv, a.kv, kh, vh, block_tok(blk + 2), pg_next, c, g, win, win_first);
    pg_next = page_of(block_tok(blk + 3));
    compute_block<MT, FP8, CAP>(rb, qB, acc, m, l, so, t_begin + (blk + 1) * kBlk, g);
  }

  write_rows<MT>(a, acc, m, l, tq, hk, row0, dest, c, g);
}

// ---- fixed split plan: grid = (max_splits * decode rows, 1, head groups * row groups), splits fastest (rows do
// not sit on a grid dimension of their own: that one ends at 65535); block = NW waves
template <int MT, bool FP8, bool UNIFORM_PAGE, bool CAP>
__global__ __launch_bounds__(256, 2) void rpa_decode_splitkv_kernel(const DecodeArgs a_in) {
  DecodeArgs a = a_in;  // static-shape mode: the number of decode rows comes from the device
  if (a.dist) a.num_rows = min(a.num_rows, scalar_load_i32(a.dist));
  const int nsp = max(a.max_splits, 1);
  const int seq = (int)(blockIdx.x / (unsigned)nsp);
  const int split = (int)blockIdx.x - seq * nsp;
  if (seq >= a.num_rows) return;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int head_groups = (a.Hkv + nw - 1) / nw;
  const int hg = blockIdx.z % head_groups;
  const int rg = blockIdx.z / head_groups;
  const int hk = hg * nw + wave;
  if (hk >= a.Hkv) return;

  const int kv_len = a.pt.kv_lens[seq];
  const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
  const int t0 = t_lo & ~(kBlk - 1);
  const int t_begin = t0 + split * a.chunk;
  if (t_begin >= kv_len) return;
  // the last split runs to kv_len even if the host's length bound was too small
  const int t_end = (split == a.max_splits - 1) ? kv_len : min(kv_len, t_begin + a.chunk);
  PartDest dest;
  dest.final_rows = a.max_splits == 1;
  dest.by_head = true;
  dest.base = ((int64_t)seq * a.max_splits + split) * a.Hq;
  decode_segment<MT, FP8, UNIFORM_PAGE, CAP>(a, seq, hk, rg, kv_len, t_lo, t_begin, t_end, dest, lane);
}

// ---- balanced plan ------------------------------------------------------------------------
// All 32-token blocks of the batch are laid out in one line -- sequence by sequence, inside a
// sequence unit by unit, inside a unit block by block -- and workgroup j takes blocks
// [j * pw, (j + 1) * pw): every workgroup streams the same number of KV bytes whatever the
// ragged lengths are, and nothing about the lengths has to be known on the host.  A unit is a
// group of NW neighbouring kv heads (x a group of 16 query heads): the NW waves of a workgroup
// walk the same tokens of neighbouring heads, whose rows are adjacent in the head-interleaved
// cache.  A workgroup crosses at most a few unit borders; units it covers completely are
// finished in place, the cut ones (at most its first and its last) leave partial rows in the
// workspace slots 2w and 2w + 1 of its waves w.
__device__ __forceinline__ int seq_blocks(int kv_len, int window) {
  return kv_len > 0 ? (kv_len - first_block_token(kv_len, window) + kBlk - 1) / kBlk : 0;
}

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int n = __shfl_up(v, off);
    if (lane >= off) v += n;
  }
  return v;
}

// Linear block indices are 32-bit: a batch holds fewer than 2^31 (32-token block, unit) pairs.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// total number of blocks of sequences [0, upto) -- all lanes of the wave must call it
__device__ __forceinline__ int blocks_before(const DecodeArgs& a, int upto, int lane) {
  int total = 0;
  for (int s0 = 0; s0 < upto; s0 += 64) {
    const int s = s0 + lane;
    int nb = (s < upto) ? seq_blocks(a.pt.kv_lens[s], a.sm.window) : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) nb += __shfl_xor(nb, off);
    total += nb;
  }
  return uniform(total);
}

__device__ __forceinline__ int blocks_per_wave(const DecodeArgs& a, int total_blocks) {
  // never fewer than the even share: the grid has exactly num_wgs workgroups
  const int even = (total_blocks + a.num_wgs - 1) / a.num_wgs;
  const int floor_ = a.forced_blocks_per_wave > 0 ? a.forced_blocks_per_wave : a.min_blocks_per_wave;
  return max(floor_, even);
}

// sequence that holds linear block x (x < total): first s with (blocks of [0, s]) * units > x
__device__ __forceinline__ void locate_block(const DecodeArgs& a, int x, int units, int lane, int& seq,
                                             int& seq_first_block) {
  int base = 0;
  seq = a.num_rows - 1;
  seq_first_block = 0;
  for (int s0 = 0; s0 < a.num_rows; s0 += 64) {
    const int s = s0 + lane;
    const int nb = (s < a.num_rows) ? seq_blocks(a.pt.kv_lens[s], a.sm.window) : 0;
    const int incl = wave_inclusive_scan(nb, lane);
    const uint64_t hit = __builtin_amdgcn_ballot_w64((base + incl) * units > x);
    if (hit != 0) {
      const int first = __builtin_ctzll(hit);
      seq = s0 + first;
      seq_first_block = uniform((base + __shfl(incl - nb, first)) * units);
      return;
    }
    base += uniform(__shfl(incl, 63));
  }
}

// Wave-uniform facts of one decode row.
struct RowMeta {
  int seq;
  int kv_len;
  int nb;         // its 32-token blocks (0: nothing to read)
  int64_t page0;  // index of its first page id in page_indices
  int tq;         // its query token
};

struct RowLoads {  // the three words of a row, as loaded
  int kv_len, cu_kv, tq;
};

__device__ __forceinline__ RowLoads row_issue_scalar(const DecodeArgs& a, int seq) {
  RowLoads r;
  r.kv_len = scalar_load_i32(a.pt.kv_lens + seq);
  r.cu_kv = a.pt.cu_kv_lens ? scalar_load_i32(a.pt.cu_kv_lens + seq) : 0;
  r.tq = scalar_load_i32(a.pt.cu_q_lens + seq);
  return r;
}

__device__ __forceinline__ RowMeta row_resolve(const DecodeArgs& a, int seq, const RowLoads& r) {
  RowMeta m;
  m.seq = seq;
  m.kv_len = r.kv_len;
  m.nb = seq_blocks(r.kv_len, a.sm.window);
  m.page0 = a.pt.cu_kv_lens ? (int64_t)(r.cu_kv / a.pt.page_size) : (int64_t)seq * a.pt.pages_per_seq;
  m.tq = r.tq;
  return m;
}

// The balanced plan's window of a row's page ids (copy_page_window), looked up with a uniform LDS read
// when pages hold whole blocks and with one LDS read per lane and token row when they are smaller:
// the steady state of a wave issues no small dependent global loads at all, and because no
// register ever waits for the copy, the compiler never drains the vector-memory queue for it.
struct PageWindow {
  int32_t* lds;  // ids of this wave: 64 (whole blocks per page, one uniform lookup per block) or kWinSmallPages
  int first;     // slot of entry 0
};

template <int ENTRIES>
__device__ __forceinline__ void request_window(const DecodeArgs& a, const RowMeta& row, PageWindow& w,
                                               int first_slot, int page_shift, int lane) {
  w.first = first_slot;
  const int last_tok = max(row.kv_len - 1, 0);
  const int last_slot = page_shift >= 0 ? (last_tok >> page_shift) : (last_tok / a.pt.page_size);
  copy_page_window<ENTRIES>(a.pt.page_indices + row.page0, last_slot, w.lds, first_slot, lane);
}

// One piece of work of a wave: tokens of one (row, kv head, group of 16 query heads).
struct Piece {
  RowMeta row;
  int hk, rg;
  int t_lo;     // first visible token (sliding window)
  int t_first;  // first token of the piece (a multiple of 32 past the window's first block)
  int nblk;     // its 32-token blocks
  bool final_rows;
};

// The wave that arrives last at a cut unit merges it.  A unit (row, kv head, group of 16 query
// heads) whose blocks n workgroups share leaves n groups of 16 partial rows; each wave, once its
// rows are written and fenced, adds one to the unit's arrival word, and the wave that brings it
// to n reads all n groups back and writes the 16 finished rows.  The word carries the call's
// generation in its upper 48 bits: a word left by another call (or by nothing: the memory is
// never cleared) counts as zero, and the merging wave sets the count back to zero so that a
// replay of the same launch with the same generation starts clean.
//
// A wave has at most two cut units, the first and the last piece of its share, and merges what
// falls to it after its last block: the registers of the block pipeline are free by then, so
// four groups of partial rows are in flight at a time, and no other wave waits for the rows.
struct PendingMerge {
  int n;  // 0: nothing to merge
  int w_first;
  int64_t first_block;
  int tq, head0, rows;
  unsigned long long* ctr;
};

// Every access is a device-scope atomic (relaxed): it reads what the other waves wrote through,
// whatever this part of the GPU still caches of an earlier call.  Lanes: dims 2 lane, 2 lane + 1
// of each of the 16 rows; lane r < 16 also owns the (max, sum) of row r.
__device__ __forceinline__ float load_agent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void load2_agent(const float* p, float& x, float& y) {
  const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
  x = __uint_as_float((uint32_t)v);
  y = __uint_as_float((uint32_t)(v >> 32));
}

__device__ __forceinline__ void merge_unit(const DecodeArgs& a, const PendingMerge& pm, int pw, int wave, int nw,
                                           unsigned long long generation, int lane) {
  const int n = pm.n;
  const int r = lane & 15;
  auto slot16 = [&](int j) -> int64_t {
    const int wj = pm.w_first + min(j, n - 1);
    const int part = ((int64_t)wj * pw >= pm.first_block) ? 0 : 1;
    return (((int64_t)wj * nw + wave) * 2 + part) * 16;
  };
  float mstar = -INFINITY;
  for (int j = 0; j < n; ++j) mstar = fmaxf(mstar, load_agent(a.ws_ml + (slot16(j) + r) * 2));
  float den = 0.f;
  float acc[16][2];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i][0] = acc[i][1] = 0.f;
  for (int j0 = 0; j0 < n; j0 += 4) {  // four groups of partial rows in flight
    float o[4][16][2];
    float wgt[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t s = slot16(j0 + u);
#pragma unroll
      for (int i = 0; i < 16; ++i) load2_agent(a.ws_o + (s + i) * 128 + 2 * lane, o[u][i][0], o[u][i][1]);
      float mj, lj;
      load2_agent(a.ws_ml + (s + r) * 2, mj, lj);
      wgt[u] = (j0 + u < n) ? fast_exp2(mj - mstar) : 0.f;  // a repeated group counts nothing
      den += lj * wgt[u];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float wu = __shfl(wgt[u], i);
        acc[i][0] += o[u][i][0] * wu;
        acc[i][1] += o[u][i][1] * wu;
      }
  }
  const float inv_r =
      a.sm.sink ? sink_inverse(mstar, den, sink_logit(a.sm.sink, a.sm.round_logits, pm.head0 + min(r, pm.rows - 1)))
                : 1.0f / den;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float inv = __shfl(inv_r, i);
    if (i < pm.rows) {
      uint32_t* op = reinterpret_cast<uint32_t*>(a.out + ((int64_t)pm.tq * a.Hq + pm.head0 + i) * 128 + 2 * lane);
      *op = pack_bf16x2(acc[i][0] * inv, acc[i][1] * inv);
    }
  }
  if (lane == 0) __hip_atomic_store(pm.ctr, generation << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// grid = num_wgs workgroups of NW = waves_per_wg waves.
//
// A wave treats its share as one stream of blocks: the block prefetched behind the last block of
// a piece is the first block of the next piece, the next row's lengths are fetched as scalar
// loads while the current piece streams, its page ids arrive as one window load and its queries
// are requested right behind that first block.  A piece border costs no round trip to memory,
// and neither does a block: under load a small dependent load waits behind megabytes of queued
// KV traffic (10 us and more), so there are none after the first block.
template <int MT, bool FP8, bool UNIFORM_PAGE, bool CAP, bool MERGE>
__global__ __launch_bounds__(256, 2) void rpa_decode_balanced_kernel(const DecodeArgs a_in) {
  DecodeArgs a = a_in;  // static-shape mode: the number of decode rows comes from the device
  if (a.dist) a.num_rows = min(a.num_rows, scalar_load_i32(a.dist));
  if (a.num_rows <= 0) return;
  const int lane = threadIdx.x & 63;
  const int wave = uniform(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int nw = a.waves_per_wg;
  const int wg = blockIdx.x;
  const int w = wg * nw + wave;
  const int row_groups = (a.G + 15) / 16;
  const int head_groups = (a.Hkv + nw - 1) / nw;
  const int units = head_groups * row_groups;
  const int page_size = a.pt.page_size;
  const int page_shift = ((page_size & (page_size - 1)) == 0) ? (31 - __builtin_clz(page_size)) : -1;

  // ---- one pass over the rows: lengths, page offsets and query tokens of rows 0..63 stay in
  // registers (most batches end there), the rest only adds to the total
  int kv0 = 0, cu0 = 0, tq0 = 0;
  if (lane < a.num_rows) {
    kv0 = a.pt.kv_lens[lane];
    cu0 = a.pt.cu_kv_lens ? a.pt.cu_kv_lens[lane] : 0;
    tq0 = a.pt.cu_q_lens[lane];
  }
  const int nb0 = seq_blocks(kv0, a.sm.window);
  const int incl0 = wave_inclusive_scan(nb0, lane);
  int total_rows = uniform(__shfl(incl0, 63));
  for (int s0 = 64; s0 < a.num_rows; s0 += 64) {
    const int s = s0 + lane;
    int nb = (s < a.num_rows) ? seq_blocks(a.pt.kv_lens[s], a.sm.window) : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) nb += __shfl_xor(nb, off);
    total_rows += uniform(nb);
  }
  const int total = total_rows * units;
  const int pw = blocks_per_wave(a, total);
  if (wg == 0 && wave == 0) {
    // the merge pass looks its rows up in this prefix sum instead of scanning again
    if (lane < a.num_rows) a.cu_blocks[lane + 1] = incl0;
    int base = uniform(__shfl(incl0, 63));
    for (int s0 = 64; s0 < a.num_rows; s0 += 64) {
      const int s = s0 + lane;
      const int nb = (s < a.num_rows) ? seq_blocks(a.pt.kv_lens[s], a.sm.window) : 0;
      const int incl = wave_inclusive_scan(nb, lane);
      if (s < a.num_rows) a.cu_blocks[s + 1] = base + incl;
      base += uniform(__shfl(incl, 63));
    }
    if (lane == 0) a.cu_blocks[0] = 0;
  }
  if ((int64_t)wg * pw >= total) return;
  int x = wg * pw;
  const int x_end = min(total, x + pw);
  const int x_first = x;

  // ---- the row that holds block x
  RowMeta row;
  int row_first;  // linear index of the row's first block
  {
    const uint64_t hit = __builtin_amdgcn_ballot_w64(incl0 * units > x);
    if (hit != 0) {
      const int first = __builtin_ctzll(hit);
      RowLoads rl;
      rl.kv_len = __builtin_amdgcn_readlane(kv0, first);
      rl.cu_kv = __builtin_amdgcn_readlane(cu0, first);
      rl.tq = __builtin_amdgcn_readlane(tq0, first);
      row = row_resolve(a, first, rl);
      row_first = uniform(__builtin_amdgcn_readlane(incl0 - nb0, first) * units);
    } else {
      int seq;
      locate_block(a, x, units, lane, seq, row_first);
      seq = uniform(seq);
      row = row_resolve(a, seq, row_issue_scalar(a, seq));
    }
  }

  auto make_piece = [&](const RowMeta& r, int unit, int blk, int take) {
    Piece p;
    p.row = r;
    const int hg = unit / row_groups;
    p.rg = unit - hg * row_groups;
    // a head group may reach past the last kv head: such a wave repeats the last head and its
    // result is dropped
    p.hk = hg * nw + wave;
    p.t_lo = (a.sm.window > 0) ? max(0, r.kv_len - a.sm.window) : 0;
    p.t_first = (p.t_lo & ~(kBlk - 1)) + blk * kBlk;
    p.nblk = take;
    p.final_rows = (blk == 0) && (take == r.nb);
    return p;
  };
  auto view_of = [&](const RowMeta& r) {
    SeqView sv;
    sv.page_size = page_size;
    sv.page_shift = page_shift;
    sv.last_tok = r.kv_len - 1;
    sv.pages = a.pt.page_indices + r.page0;
    return sv;
  };
  auto slot_of_tok = [&](int tok) { return page_shift >= 0 ? (tok >> page_shift) : (tok / page_size); };
  auto page_in = [&](const PageWindow& pwn, int tok) -> int {
    if constexpr (UNIFORM_PAGE) return uniform(pwn.lds[uniform(slot_of_tok(tok) - pwn.first)]);
    else return 0;
  };

  Piece cur;
  {
    const int r = x - row_first;
    const int unit = r / row.nb;
    const int blk = r - unit * row.nb;
    cur = make_piece(row, unit, blk, min(row.nb - blk, x_end - x));
  }
  int cur_unit = (x - row_first) / row.nb;
  constexpr int kWin = UNIFORM_PAGE ? 64 : kWinSmallPages;
  __shared__ int32_t lds_windows[4][2][kWin];  // [wave][current / next piece][entry]
  PageWindow win = {lds_windows[wave][0], 0};
  PageWindow nwin = {lds_windows[wave][1], 0};
  // what load_block takes besides the uniform page id: the window itself when pages are smaller than a block
  auto lanes_win = [&](const PageWindow& pwn) -> const int32_t* { return UNIFORM_PAGE ? nullptr : pwn.lds; };
  request_window<kWin>(a, cur.row, win, slot_of_tok(cur.t_first), page_shift, lane);
  u32x4_t qB[MT][4];
  load_queries<MT, FP8>(a, cur.row.tq, min(cur.hk, a.Hkv - 1), cur.rg * 16 * MT, c, g, qB);
  wait_all_loads();  // the window (and the queries behind it)

  KvRegs<FP8> ra, rb;
  bool in_b = false;  // which register set holds the block about to be consumed
  {
    const SeqView sv = view_of(cur.row);
    const int hk = min(cur.hk, a.Hkv - 1);
    load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(ra, sv, a.kv, a.kv.k_base + (int64_t)hk * a.kv.head_stride,
                                  a.kv.v_base + (int64_t)hk * a.kv.head_stride, cur.t_first,
                                  page_in(win, cur.t_first), c, g, lanes_win(win), win.first);
  }

  PendingMerge pm_first = {}, pm_last = {};
  for (;;) {
    // ---- this piece
    const int hk = min(cur.hk, a.Hkv - 1);
    const SeqView sv = view_of(cur.row);
    const char* kh = a.kv.k_base + (int64_t)hk * a.kv.head_stride;
    const char* vh = a.kv.v_base + (int64_t)hk * a.kv.head_stride;
    requantise_queries<MT, FP8>(a, qB);
    ScoreOpts so;
    {
      const float ks = a.k_scale ? a.k_scale[hk] : 1.0f;
      const float temp = xai_factor(cur.row.kv_len - 1, a.sm.xai_len);  // the one query sits at kv_len - 1
      so.scale = a.sm.sm_scale * ks * (a.sm.q_scale > 0.f ? a.sm.q_scale : 1.0f);
      so.scale2 = so.scale * kLog2e * temp;
      so.temp = temp;
      so.round_mode = a.sm.round_logits;
      so.cap = a.sm.soft_cap;
      so.inv_cap = (so.cap != 0.f) ? 1.0f / so.cap : 0.f;
      so.mask2 = fmaxf(a.sm.mask_value * kLog2e, -3.0e38f);
      so.t_lo = cur.t_lo;
      so.kv_len = cur.row.kv_len;
    }
    f32x4_t acc[MT][8];
    float m[MT], l[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      m[mt] = -INFINITY;
      l[mt] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[mt][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // ---- the piece after it: the next unit of the same row, or the first unit of the next row
    // that has any block (has_next guarantees there is one)
    const bool has_next = x + cur.nblk < x_end;
    const bool next_row = has_next && (cur_unit == units - 1);
    int nseq = cur.row.seq + 1;
    RowLoads nl = {0, 0, 0};
    if (next_row) nl = row_issue_scalar(a, nseq);
    Piece nxt = cur;
    SeqView nsv = sv;
    const char* nkh = kh;
    const char* nvh = vh;
    // resolved one block into the piece when it has more than one block, at once otherwise
    const int resolve_at = (cur.nblk > 1) ? 1 : 0;

    auto step = [&](int i, const KvRegs<FP8>& use, KvRegs<FP8>& fill) __attribute__((always_inline)) {
      if (has_next && i == resolve_at) {
        RowMeta nrow = cur.row;
        int nunit = cur_unit + 1;
        if (next_row) {
          nrow = row_resolve(a, nseq, nl);
          while (nrow.nb == 0) {  // rows without tokens (padding)
            ++nseq;
            nrow = row_resolve(a, nseq, row_issue_scalar(a, nseq));
          }
          nunit = 0;
        }
        const int x_next = x + cur.nblk;
        nxt = make_piece(nrow, nunit, 0, min(nrow.nb, x_end - x_next));
        request_window<kWin>(a, nrow, nwin, slot_of_tok(nxt.t_first), page_shift, lane);
        nsv = view_of(nrow);
        const int nhk = min(nxt.hk, a.Hkv - 1);
        nkh = a.kv.k_base + (int64_t)nhk * a.kv.head_stride;
        nvh = a.kv.v_base + (int64_t)nhk * a.kv.head_stride;
      }
      const int tb = cur.t_first + i * kBlk;
      const bool last = (i + 1 == cur.nblk);
      // the block to request now: the next one of this piece, the first one of the next piece,
      // or (nothing left) this block again, so that every path has the same loads in flight
      // the window moves on when the next block's last page lies beyond it
      if (!last && slot_of_tok(tb + kBlk + (UNIFORM_PAGE ? 0 : kBlk - 1)) - win.first >= kWin) {
        request_window<kWin>(a, cur.row, win, slot_of_tok(tb + kBlk), page_shift, lane);
        wait_all_loads();
      }
      // real branches, not selects: looking a page up in the next piece's window must not make
      // every block wait for that window
      if (last && has_next) {
        // The next piece's window was requested at block resolve_at, in front of that block's
        // prefetch.  Two blocks later a wait for younger loads has passed; earlier it has not.
        if (i <= resolve_at + 1) wait_all_loads();
        load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(fill, nsv, a.kv, nkh, nvh, nxt.t_first, page_in(nwin, nxt.t_first), c, g,
                                      lanes_win(nwin), nwin.first);
      } else {
        const int ptb = last ? tb : tb + kBlk;
        load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(fill, sv, a.kv, kh, vh, ptb, page_in(win, ptb), c, g, lanes_win(win), win.first);
      }
      compute_block<MT, FP8, CAP>(use, qB, acc, m, l, so, tb, g);
    };
    // the piece's first block sits in ra or in rb, wherever the piece before it ended
    {
      int i = 0;
      bool skip_a = in_b;
      for (;;) {
        if (!skip_a) {
          step(i, ra, rb);
          if (++i == cur.nblk) {
            in_b = true;
            break;
          }
        }
        skip_a = false;
        step(i, rb, ra);
        if (++i == cur.nblk) {
          in_b = false;
          break;
        }
      }
    }

    if (cur.hk < a.Hkv) {
      PartDest dest;
      dest.final_rows = cur.final_rows;
      dest.by_head = false;
      dest.base = ((int64_t)w * 2 + (x == x_first ? 0 : 1)) * 16;
      write_rows<MT, MERGE>(a, acc, m, l, cur.row.tq, hk, cur.rg * 16 * MT, dest, c, g);
      if (MERGE && !cur.final_rows) {
        // the unit's first block in the linear order, and the workgroups that share the unit
        const int64_t first_block = (int64_t)x - (cur.t_first - (cur.t_lo & ~(kBlk - 1))) / kBlk;
        const int w_first = (int)(first_block / pw), w_last = (int)((first_block + cur.row.nb - 1) / pw);
        const unsigned long long n = (unsigned long long)(w_last - w_first + 1);
        unsigned long long* ctr = a.merge_counters + ((int64_t)cur.row.seq * units + cur_unit) * nw + wave;
        // this wave's rows, written through, have reached device scope before it arrives
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        int is_last = 0;
        if (lane == 0) {
          unsigned long long old = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          for (;;) {
            const unsigned long long cnt = ((old >> 16) == a.generation) ? (old & 0xffffull) : 0ull;
            const unsigned long long neu = (a.generation << 16) | (cnt + 1);
            if (__hip_atomic_compare_exchange_strong(ctr, &old, neu, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT)) {
              is_last = (cnt + 1 == n) ? 1 : 0;
              break;
            }
          }
        }
        is_last = __builtin_amdgcn_readfirstlane(is_last);
        if (is_last) {
          PendingMerge& pm = (x == x_first) ? pm_first : pm_last;
          pm.n = (int)n;
          pm.w_first = w_first;
          pm.first_block = first_block;
          pm.tq = cur.row.tq;
          pm.head0 = hk * a.G + cur.rg * 16;
          pm.rows = min(16, a.G - cur.rg * 16);
          pm.ctr = ctr;
        }
      }
    }
    if (!has_next) break;
    x += cur.nblk;
    cur_unit = next_row ? 0 : cur_unit + 1;
    cur = nxt;
    {  // the two LDS windows trade places
      const PageWindow t = win;
      win = nwin;
      nwin = t;
    }
    // the queries queue up right behind the piece's first block, which is already on its way
    load_queries<MT, FP8>(a, cur.row.tq, min(cur.hk, a.Hkv - 1), cur.rg * 16 * MT, c, g, qB);
  }
  if (MERGE && (pm_first.n | pm_last.n)) {
    if (pm_first.n) merge_unit(a, pm_first, pw, wave, nw, a.generation, lane);
    if (pm_last.n) merge_unit(a, pm_last, pw, wave, nw, a.generation, lane);
  }
}

// Merge the n partial rows of one (decode row, query head) and write the finished row.
// slot_of(j) is the workspace slot of partial j.  One wave, 2 dims per lane.  Up to 16 partials
// (nearly always) everything is requested at once -- the (max, sum) pairs by lanes 0..n-1, the
// partial rows by all lanes, the row's query token before either -- so the merge costs one round
// trip to memory instead of three dependent ones.
template <int N, int HD, typename SlotOf>
__device__ __forceinline__ void merge_few(const DecodeArgs& a, int n, int lane, SlotOf slot_of, float& mstar,
                                          float& den, float (&acc)[HD / 64]) {
  constexpr int kDpl = HD / 64;  // dims per lane
  typedef float fvec_t __attribute__((ext_vector_type(kDpl)));
  const int d = lane * kDpl;
  float mj = -INFINITY, lj = 0.f;
  if (lane < n) {
    const int64_t slot = slot_of(lane);
    mj = a.ws_ml[slot * 2];
    lj = a.ws_ml[slot * 2 + 1];
  }
  fvec_t o[N];
#pragma unroll
  for (int u = 0; u < N; ++u) o[u] = *reinterpret_cast<const fvec_t*>(a.ws_o + slot_of(min(u, n - 1)) * HD + d);
  mstar = mj;
#pragma unroll
  for (int off = N / 2; off > 0; off >>= 1) mstar = fmaxf(mstar, __shfl_xor(mstar, off));
  mstar = __shfl(mstar, 0);
  const float wj = (lane < n) ? fast_exp2(mj - mstar) : 0.f;
  den = lj * wj;
#pragma unroll
  for (int off = N / 2; off > 0; off >>= 1) den += __shfl_xor(den, off);
  den = __shfl(den, 0);
#pragma unroll
  for (int e = 0; e < kDpl; ++e) acc[e] = 0.f;
#pragma unroll
  for (int u = 0; u < N; ++u) {
    const float wu = __shfl(wj, u);  // 0 beyond n: the repeated last row does not count
#pragma unroll
    for (int e = 0; e < kDpl; ++e) acc[e] += o[u][e] * wu;
  }
}

template <int HD = 128, typename SlotOf>
__device__ __forceinline__ void merge_rows(const DecodeArgs& a, int seq, int head, int n, int lane, SlotOf slot_of) {
  constexpr int kDpl = HD / 64;  // dims per lane
  typedef float fvec_t __attribute__((ext_vector_type(kDpl)));
  const int d = lane * kDpl;
  const int tq = scalar_load_i32(a.pt.cu_q_lens + seq);
  float mstar = -INFINITY, den = 0.f;
  float acc[kDpl];
#pragma unroll
  for (int e = 0; e < kDpl; ++e) acc[e] = 0.f;
  if (n <= 8) {
    merge_few<8, HD>(a, n, lane, slot_of, mstar, den, acc);
  } else if (n <= 16) {
    merge_few<16, HD>(a, n, lane, slot_of, mstar, den, acc);
  } else {
    for (int j0 = 0; j0 < n; j0 += 64) {
      const int j = j0 + lane;
      float mj = (j < n) ? a.ws_ml[slot_of(j) * 2] : -INFINITY;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) mj = fmaxf(mj, __shfl_xor(mj, off));
      mstar = fmaxf(mstar, mj);
    }
    for (int j0 = 0; j0 < n; j0 += 64) {
      const int j = j0 + lane;
      float wj = 0.f, lj = 0.f;
      if (j < n) {
        const int64_t slot = slot_of(j);
        wj = fast_exp2(a.ws_ml[slot * 2] - mstar);
        lj = a.ws_ml[slot * 2 + 1] * wj;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) lj += __shfl_xor(lj, off);
      den += lj;
      // 32 partial rows requested at a time: a row with hundreds of partials (one long
      // sequence cut over the whole GPU) is a chain of such round trips
      const int cnt = min(64, n - j0);
      for (int jj = 0; jj < cnt; jj += 32) {
        fvec_t o[32];
        float wv[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          const int js = min(jj + u, cnt - 1);
          wv[u] = (jj + u < cnt) ? __shfl(wj, js) : 0.f;
          o[u] = *reinterpret_cast<const fvec_t*>(a.ws_o + slot_of(j0 + js) * HD + d);
        }
#pragma unroll
        for (int u = 0; u < 32; ++u)
#pragma unroll
          for (int e = 0; e < kDpl; ++e) acc[e] += o[u][e] * wv[u];
      }
    }
  }
  const float inv = a.sm.sink ? sink_inverse(mstar, den, sink_logit(a.sm.sink, a.sm.round_logits, head)) : 1.0f / den;
  uint32_t* op = reinterpret_cast<uint32_t*>(a.out + ((int64_t)tq * a.Hq + head) * HD + d);
#pragma unroll
  for (int e = 0; e < kDpl; e += 2) op[e / 2] = pack_bf16x2(acc[e] * inv, acc[e + 1] * inv);
}

// Merge the partial rows of the balanced plan.  grid = (Hq * decode rows); block = one wave.
__global__ __launch_bounds__(64) void rpa_combine_balanced_kernel(const DecodeArgs a_in) {
  DecodeArgs a = a_in;  // static-shape mode: the number of decode rows comes from the device
  if (a.dist) a.num_rows = min(a.num_rows, scalar_load_i32(a.dist));
  const int seq = (int)(blockIdx.x / (unsigned)a.Hq);  // grid.x = Hq * rows, heads fastest
  const int head = (int)blockIdx.x - seq * a.Hq;
  if (seq >= a.num_rows) return;
  const int lane = threadIdx.x;
  const int nw = a.waves_per_wg;
  const int row_groups = (a.G + 15) / 16;
  const int units = ((a.Hkv + nw - 1) / nw) * row_groups;
  const int nb = seq_blocks(a.pt.kv_lens[seq], a.sm.window);
  if (nb == 0) return;
  const int before = scalar_load_i32(a.cu_blocks + seq);
  const int total = scalar_load_i32(a.cu_blocks + a.num_rows) * units;
  const int pw = blocks_per_wave(a, total);
  const int hk = head / a.G, row = head - hk * a.G;
  const int unit = (hk / nw) * row_groups + row / 16;
  const int wv = hk % nw;
  const int first_block = before * units + unit * nb;
  const int w_first = first_block / pw, w_last = (first_block + nb - 1) / pw;
  if (w_first == w_last) return;  // one wave covered the unit and wrote the finished rows
  const int n = w_last - w_first + 1;
  const int r16 = row & 15;
  auto slot_of = [&](int j) -> int64_t {
    const int wj = w_first + j;  // workgroup
    // a workgroup's first piece of work goes to slot 0 of its waves: that is this unit iff it starts inside it
    const int part = ((int64_t)wj * pw >= first_block) ? 0 : 1;
    return (((int64_t)wj * nw + wv) * 2 + part) * 16 + r16;
  };
  merge_rows(a, seq, head, n, lane, slot_of);
}

// ---- head_dim 256 ---------------------------------------------------------------------------
// One wave per (query token, kv head, group of 16 query heads): a query token of a chunk is a
// decode row over the first kv_len - q_len + j + 1 tokens, so one kernel serves decode rows and
// prefill chunks alike.  The two 128-dim halves of a head reuse the register layouts and the
// loads of the 128-dim kernel (a half is 128 contiguous elements of the head's row); scores sum
// over both halves, each half has its own accumulators.  No split over tokens, no prefetch
// ahead of the block being consumed, and a chunk's tokens each stream the prefix again: this
// path exists so that 256-dim heads work, it is not tuned.
__device__ __forceinline__ int owner_of_token(const int32_t* cu_q_lens, int num_seqs, int tok) {
  int lo = 0, hi = num_seqs;  // last i with cu_q_lens[i] <= tok (zero-length sequences are skipped)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_q_lens[mid] <= tok) lo = mid; else hi = mid;
  }
  return lo;
}

// grid = (token rows, Hkv, row groups of 16 query heads); block = one wave.
// With the composition on the device (a.dist) seq_end is only a bound: dist_role 1 = the decode partition
// [0, dist[0]), 2 = everything behind it [dist[0], dist[2]) (custom-mask calls: [0, dist[2])).
template <bool FP8, bool UNIFORM_PAGE>
__global__ __launch_bounds__(64) void rpa_rows256_kernel(const DecodeArgs a, int seq_begin, int seq_end, int dist_role) {
  if (a.dist && dist_role == 1) {
    seq_end = min(seq_end, scalar_load_i32(a.dist));
  } else if (a.dist && dist_role == 2) {
    seq_begin = (a.sm.mask_mode == 1) ? 0 : min(seq_end, scalar_load_i32(a.dist));
    seq_end = min(seq_end, scalar_load_i32(a.dist + 2));
  }
  if (seq_end <= seq_begin) return;
  const int lane = threadIdx.x;
  const int c = lane & 15, g = lane >> 4;
  const int rg = blockIdx.z, hk = blockIdx.y;
  // decode rows may be cut into max_splits pieces of `chunk` tokens (one token per row then, and
  // row = sequence); partial rows go to the workspace in the fixed plan's layout
  const int nsplit = max(a.max_splits, 1);
  const int split = blockIdx.x % nsplit;
  const int tok_row = blockIdx.x / nsplit + a.pt.cu_q_lens[seq_begin];
  if (tok_row >= a.pt.cu_q_lens[seq_end]) return;
  const int seq = owner_of_token(a.pt.cu_q_lens, seq_end, tok_row);
  const int q0 = a.pt.cu_q_lens[seq];
  const int q_len = a.pt.cu_q_lens[seq + 1] - q0;
  const int kv_len = a.pt.kv_lens[seq];
  const int qpos = kv_len - q_len + (tok_row - q0);
  // tokens this row sees: [t_lo, t_hi)
  const int t_hi = (a.sm.mask_mode == 0) ? qpos + 1 : kv_len;
  if (t_hi <= 0) return;
  const int t_lo = (a.sm.window > 0) ? max(0, qpos - a.sm.window + 1) : 0;
  // the caller's own mask: one i32 per (query token, kv token), rows kv_len wide or padded to whole pages
  const int32_t* mask_row = nullptr;
  if (a.sm.mask_mode == 1) {
    const int width = a.sm.mask_rows_page_aligned ? (a.pt.cu_kv_lens[seq + 1] - a.pt.cu_kv_lens[seq]) : kv_len;
    mask_row = a.sm.custom_mask + a.sm.cu_mask_lens[seq] + (int64_t)(tok_row - q0) * width;
  }

  SeqView sv;
  sv.page_size = a.pt.page_size;
  sv.page_shift = ((sv.page_size & (sv.page_size - 1)) == 0) ? (31 - __builtin_clz(sv.page_size)) : -1;
  sv.last_tok = t_hi - 1;
  sv.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / a.pt.page_size)
                                                  : (int64_t)seq * a.pt.pages_per_seq);
  constexpr int kHalfB = FP8 ? 128 : 256;  // bytes of 128 cached elements
  const char* kh = a.kv.k_base + (int64_t)hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)hk * a.kv.head_stride;

  // ---- Q^T operands: column c = query head (16 rg + c) of this kv head, both halves ----
  const int row = rg * 16 + c;
  u32x4_t qB[2][4];
  {
    const uint16_t* qp = a.q + ((int64_t)tok_row * a.Hq + (int64_t)hk * a.G + min(row, a.G - 1)) * 256;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const int d0 = hf * 128 + (FP8 ? (g * 32 + st * 8) : (st * 32 + g * 8));
        qB[hf][st] = ld16(qp + d0);
        if (a.sm.q_scale > 0.f) qB[hf][st] = requantise_q(qB[hf][st], a.sm.q_scale, FP8);
      }
  }
  const float scale = a.sm.sm_scale * (a.k_scale ? a.k_scale[hk] : 1.0f) * (a.sm.q_scale > 0.f ? a.sm.q_scale : 1.0f);
  const float temp = xai_factor(qpos, a.sm.xai_len);
  const float cap = a.sm.soft_cap;
  const float inv_cap = (cap != 0.f) ? 1.0f / cap : 0.f;
  const float mask2 = fmaxf(a.sm.mask_value * kLog2e, -3.0e38f);
  const int round_mode = a.sm.round_logits;

  f32x4_t acc[2][8];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[hf][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  int tb_begin = t_lo & ~(kBlk - 1), tb_end = t_hi;
  if (nsplit > 1) {
    tb_begin += split * a.chunk;
    if (tb_begin >= t_hi) return;  // the merge pass knows how many pieces a row has
    if (split < nsplit - 1) tb_end = min(t_hi, tb_begin + a.chunk);
  }
  // pages smaller than a block: the lanes look their token rows' pages up in an LDS window of the row's page
  // ids (see decode_segment) instead of fetching them from memory in front of every block
  __shared__ int32_t win_ids[UNIFORM_PAGE ? 1 : kWinSmallPages];
  const int32_t* win = nullptr;
  int win_first = 0;
  for (int tb = tb_begin; tb < tb_end; tb += kBlk) {
    int page = 0;
    if constexpr (UNIFORM_PAGE) page = __builtin_amdgcn_readfirstlane(sv.pages[page_slot_of(sv, tb)]);
    else if (!win || page_slot_of(sv, min(tb + kBlk - 1, sv.last_tok)) - win_first >= kWinSmallPages) {
      win_first = __builtin_amdgcn_readfirstlane(page_slot_of(sv, tb));
      copy_page_window<kWinSmallPages>(sv.pages, page_slot_of(sv, sv.last_tok), win_ids, win_first, lane);
      wait_all_loads();
      win = win_ids;
    }
    KvRegs<FP8> r0, r1;
    load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(r0, sv, a.kv, kh, vh, tb, page, c, g, win, win_first);
    load_block<FP8, UNIFORM_PAGE, !UNIFORM_PAGE>(r1, sv, a.kv, kh + kHalfB, vh + kHalfB, tb, page, c, g, win, win_first);
    f32x4_t s[2];
    {
      u32x4_t kA[2][4];
      k_operands<FP8>(r0, kA);
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        s[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < 4; ++st) s[b] = mfma16(kA[b][st], qB[0][st], s[b]);
      }
      k_operands<FP8>(r1, kA);
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int st = 0; st < 4; ++st) s[b] = mfma16(kA[b][st], qB[1][st], s[b]);
    }
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = s[i >> 2][i & 3] * scale;
      if (cap != 0.f) v = soft_cap_f(v, cap, inv_cap);
      v = v * temp;
      if (round_mode) v = round_logit(v, round_mode);
      v = v * kLog2e;
      const int tok = tb + tok_slot(g, i);
      bool dead = tok >= tb_end || tok < t_lo;
      if (mask_row && !dead) dead = mask_row[tok] < 1;
      x[i] = dead ? mask2 : v;
    }
    float mx = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2(m - m_new);
    float p[8], ps = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      p[i] = fast_exp2(x[i] - m_new);
      ps += p[i];
    }
    l = l * alpha + ps;
    m = m_new;
    const u32x4_t pB = u32x4_t{pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                               pack_bf16x2(p[6], p[7])};
    {
      u32x4_t vA[8];
      v_operands<FP8>(r0, vA);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[0][j] = mfma16(vA[j], pB, acc[0][j] * alpha);
      v_operands<FP8>(r1, vA);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[1][j] = mfma16(vA[j], pB, acc[1][j] * alpha);
    }
  }

  // ---- epilogue: lane (c, g) holds q row c, dims 128 hf + 32g + 8r + j in acc[hf][j][r] ----
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  if (row >= a.G) return;
  const int head = hk * a.G + row;
  const float vs = a.v_scale ? a.v_scale[hk] : 1.0f;
  if (nsplit > 1) {
    const int64_t slot = ((int64_t)seq * nsplit + split) * a.Hq + head;
    float* wo = a.ws_o + slot * 256 + g * 32;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        f32x4_t w0 = {acc[hf][0][r] * vs, acc[hf][1][r] * vs, acc[hf][2][r] * vs, acc[hf][3][r] * vs};
        f32x4_t w1 = {acc[hf][4][r] * vs, acc[hf][5][r] * vs, acc[hf][6][r] * vs, acc[hf][7][r] * vs};
        *reinterpret_cast<f32x4_t*>(wo + hf * 128 + r * 8) = w0;
        *reinterpret_cast<f32x4_t*>(wo + hf * 128 + r * 8 + 4) = w1;
      }
    if (g == 0) {
      a.ws_ml[slot * 2 + 0] = m;
      a.ws_ml[slot * 2 + 1] = l;
    }
    return;
  }
  const float inv = a.sm.sink ? vs * sink_inverse(m, l, sink_logit(a.sm.sink, a.sm.round_logits, head)) : vs / l;
  uint16_t* op = a.out + ((int64_t)tok_row * a.Hq + head) * 256 + g * 32;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      u32x4_t w;
#pragma unroll
      for (int jp = 0; jp < 4; ++jp) w[jp] = pack_bf16x2(acc[hf][2 * jp][r] * inv, acc[hf][2 * jp + 1][r] * inv);
      st16(op + hf * 128 + r * 8, w);
    }
}

// Merge the split partials: out = sum_j o_j 2^(m_j - m*) / sum_j l_j 2^(m_j - m*).
// grid = (Hq * decode rows); block = one wave, 2 dims per lane (D = 128).  Lane j
// first fetches (m_j, l_j) of split j, the wave reduces m* and the denominator
// with shuffles, then the weights are broadcast lane by lane while the partial
// rows stream in with independent loads.
template <int HD>
__global__ __launch_bounds__(64) void rpa_combine_kernel(const DecodeArgs a_in) {
  DecodeArgs a = a_in;  // static-shape mode: the number of decode rows comes from the device
  if (a.dist) a.num_rows = min(a.num_rows, scalar_load_i32(a.dist));
  const int seq = (int)(blockIdx.x / (unsigned)a.Hq);  // grid.x = Hq * rows, heads fastest
  const int head = (int)blockIdx.x - seq * a.Hq;
  if (seq >= a.num_rows) return;
  const int lane = threadIdx.x;
  const int kv_len = a.pt.kv_lens[seq];
  const int t0 = first_block_token(kv_len, a.sm.window);
  const int n = min(a.max_splits, (kv_len - t0 + a.chunk - 1) / a.chunk);
  if (n <= 0) return;
  const int64_t base = ((int64_t)seq * a.max_splits) * a.Hq + head;
  merge_rows<HD>(a, seq, head, n, lane, [&](int j) -> int64_t { return base + (int64_t)j * a.Hq; });
}

// One thread copies one 16-byte piece of one gathered row.
__global__ __launch_bounds__(256) void rpa_gather_kernel(const GatherArgs a) {
  const int kv_len = min(a.pt.kv_lens[a.seq], a.max_tokens);
  const int pieces = a.row_bytes / 16;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)kv_len * pieces;
  if (idx >= total) return;
  const int tok = (int)(idx / pieces);
  const int byte = (int)(idx % pieces) * 16;
  const int head = byte / a.head_bytes;
  const int inner = byte % a.head_bytes;
  const int32_t* pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[a.seq] / a.pt.page_size)
                                                              : (int64_t)a.seq * a.pt.pages_per_seq);
  const int slot = tok / a.pt.page_size;
  const int64_t off = (int64_t)pages[slot] * a.kv.page_stride +
                      (int64_t)(tok - slot * a.pt.page_size) * a.kv.tok_stride +
                      (int64_t)head * a.kv.head_stride + inner;
  st16((char*)a.k_out + (int64_t)tok * a.row_bytes + byte, ld16(a.kv.k_base + off));
  st16((char*)a.v_out + (int64_t)tok * a.row_bytes + byte, ld16(a.kv.v_base + off));
}

// New-token cache write: token j of sequence i lands at position kv_len-q_len+j.
// grid.x covers (token, 16-byte piece); the sequence of a token is found by
// binary search in cu_q_lens.
__global__ __launch_bounds__(256) void rpa_kv_write_kernel(const KvWriteArgs a_in) {
  KvWriteArgs a = a_in;
  if (a.dist) a.num_seqs = min(a.num_seqs, a.dist[2]);
  const int pieces = a.Hkv * a.head_bytes / 16;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int total_tokens = min(a.num_tokens, a.pt.cu_q_lens[a.num_seqs]);
  if (idx >= (int64_t)total_tokens * pieces) return;
  const int t = (int)(idx / pieces);
  const int byte = (int)(idx % pieces) * 16;
  int lo = 0, hi = a.num_seqs;  // last i with cu_q_lens[i] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.pt.cu_q_lens[mid] <= t) lo = mid; else hi = mid;
  }
  const int seq = lo;
  const int q0 = a.pt.cu_q_lens[seq], q1 = a.pt.cu_q_lens[seq + 1];
  const int pos = a.pt.kv_lens[seq] - (q1 - q0) + (t - q0);
  if (pos < 0) return;
  const int32_t* pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / a.pt.page_size)
                                                              : (int64_t)seq * a.pt.pages_per_seq);
  const int slot = pos / a.pt.page_size;
  const int head = byte / a.head_bytes;
  const int inner = byte % a.head_bytes;
  const int64_t off = (int64_t)pages[slot] * a.kv.page_stride +
                      (int64_t)(pos - slot * a.pt.page_size) * a.kv.tok_stride +
                      (int64_t)head * a.kv.head_stride + inner;
  const int64_t src = (int64_t)t * a.Hkv * a.head_bytes + byte;
  st16(const_cast<char*>(a.kv.k_base) + off, ld16(a.keys + src));
  st16(const_cast<char*>(a.kv.v_base) + off, ld16(a.values + src));
}

template <bool FP8, bool UNIFORM, bool CAP>
void launch_decode_variant(const DecodeArgs& a, dim3 grid, dim3 block, hipStream_t st) {
  if (a.balanced && a.merge_counters)
    hipLaunchKernelGGL((rpa_decode_balanced_kernel<1, FP8, UNIFORM, CAP, true>), grid, block, 0, st, a);
  else if (a.balanced)
    hipLaunchKernelGGL((rpa_decode_balanced_kernel<1, FP8, UNIFORM, CAP, false>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((rpa_decode_splitkv_kernel<1, FP8, UNIFORM, CAP>), grid, block, 0, st, a);
}

hipError_t launch_decode_mt(const DecodeArgs& a, dim3 grid, dim3 block, bool uniform, hipStream_t st) {
  // soft cap and logit rounding share the general score path
  const bool cap = a.sm.soft_cap != 0.f || a.sm.round_logits != 0;
  const int key = (a.fp8 ? 4 : 0) | (uniform ? 2 : 0) | (cap ? 1 : 0);
  switch (key) {
    case 0: launch_decode_variant<false, false, false>(a, grid, block, st); break;
    case 1: launch_decode_variant<false, false, true>(a, grid, block, st); break;
    case 2: launch_decode_variant<false, true, false>(a, grid, block, st); break;
    case 3: launch_decode_variant<false, true, true>(a, grid, block, st); break;
    case 4: launch_decode_variant<true, false, false>(a, grid, block, st); break;
    case 5: launch_decode_variant<true, false, true>(a, grid, block, st); break;
    case 6: launch_decode_variant<true, true, false>(a, grid, block, st); break;
    default: launch_decode_variant<true, true, true>(a, grid, block, st); break;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_decode(const DecodeArgs& a, hipStream_t stream) {
  if (a.num_rows <= 0) return hipSuccess;
  const int nw = min(max(a.waves_per_wg, 1), min(4, a.Hkv));  // kv heads walked together by one workgroup
  const int head_groups = (a.Hkv + nw - 1) / nw;
  // more than 16 query heads per kv head: further groups of 16 re-walk the KV (rare: MQA-like shapes)
  const int row_groups = (a.G + 15) / 16;
  const bool uniform = (a.pt.page_size % kBlk) == 0;
  if (a.balanced) {
    hipError_t e = launch_decode_mt(a, dim3(a.num_wgs), dim3(a.waves_per_wg * 64), uniform, stream);
    if (e != hipSuccess) return e;
    if (!a.merge_counters)
      hipLaunchKernelGGL(rpa_combine_balanced_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(64), 0, stream, a);
    return hipGetLastError();
  }
  if ((int64_t)a.max_splits * a.num_rows > 0x7fffffffLL || (int64_t)a.Hq * a.num_rows > 0x7fffffffLL)
    return hipErrorInvalidValue;
  dim3 grid((unsigned)max(a.max_splits, 1) * (unsigned)a.num_rows, 1, head_groups * row_groups);
  dim3 block(nw * 64);
  hipError_t e = launch_decode_mt(a, grid, block, uniform, stream);
  if (e != hipSuccess) return e;
  if (a.max_splits > 1) {
    hipLaunchKernelGGL(rpa_combine_kernel<128>, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(64), 0, stream, a);
    e = hipGetLastError();
  }
  return e;
}

hipError_t launch_gather(const GatherArgs& a, hipStream_t stream) {
  if (a.max_tokens <= 0) return hipSuccess;
  const int64_t total = (int64_t)a.max_tokens * (a.row_bytes / 16);
  const int blocks = (int)((total + 255) / 256);
  hipLaunchKernelGGL(rpa_gather_kernel, dim3(blocks), dim3(256), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_rows256(const DecodeArgs& a, int seq_begin, int seq_end, int max_token_rows, int dist_role,
                          hipStream_t stream) {
  if (seq_end <= seq_begin || max_token_rows <= 0) return hipSuccess;
  if (a.Hkv > 65535) return hipErrorInvalidValue;  // grid.y
  const int nsplit = a.max_splits > 1 ? a.max_splits : 1;
  if ((int64_t)max_token_rows * nsplit > 0x7fffffffLL) return hipErrorInvalidValue;
  const dim3 grid(max_token_rows * nsplit, a.Hkv, (a.G + 15) / 16), block(64);
  const bool uniform = (a.pt.page_size % kBlk) == 0;
  if (a.fp8) {
    if (uniform) hipLaunchKernelGGL((rpa_rows256_kernel<true, true>), grid, block, 0, stream, a, seq_begin, seq_end, dist_role);
    else hipLaunchKernelGGL((rpa_rows256_kernel<true, false>), grid, block, 0, stream, a, seq_begin, seq_end, dist_role);
  } else {
    if (uniform) hipLaunchKernelGGL((rpa_rows256_kernel<false, true>), grid, block, 0, stream, a, seq_begin, seq_end, dist_role);
    else hipLaunchKernelGGL((rpa_rows256_kernel<false, false>), grid, block, 0, stream, a, seq_begin, seq_end, dist_role);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || nsplit == 1) return e;
  if ((int64_t)a.Hq * a.num_rows > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(rpa_combine_kernel<256>, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(64), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_kv_write(const KvWriteArgs& a, hipStream_t stream) {
  if (a.num_tokens <= 0 || a.num_seqs <= 0) return hipSuccess;
  const int64_t total = (int64_t)a.num_tokens * (a.Hkv * a.head_bytes / 16);
  const int blocks = (int)((total + 255) / 256);
  hipLaunchKernelGGL(rpa_kv_write_kernel, dim3(blocks), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace rpa
