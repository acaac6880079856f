// Pieces shared by the prefill kernels (rpa_prefill.hip, rpa_prefill_pipe.hip): work
// decomposition, tile geometry in LDS, the asynchronous global -> LDS tile copy, the online
// softmax of a 64-token tile and the final row write.
#pragma once

#include "rpa_common.h"
#include "rpa_kernels.h"
#include "rpa_shapes.h"
#include "rpa_tuning.h"

namespace rpa {
namespace pf {

constexpr int kBM = 128;  // query rows per workgroup
constexpr int kBN = 64;   // kv tokens per tile

__device__ __forceinline__ u32x4_t lds_ld16(const char* p) { return *reinterpret_cast<const u32x4_t*>(p); }
__device__ __forceinline__ void lds_st16(char* p, u32x4_t v) { *reinterpret_cast<u32x4_t*>(p) = v; }

typedef short s16x4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: inside every block of 16 lanes, lane i receives
//   out[e] = M[(i >> 2) + 4e][i & 3],  e = 0..3,
// where M[r][0..3] are the four 16-bit elements at the address supplied by lane r of
// the block.  With lane r pointing at (token r >> 2, dims 4*(r & 3) ..) of a row-major
// tile, lane i ends up with dim i of four tokens: the k-contiguous MFMA operand.
__device__ __forceinline__ u32x2_t lds_tr16(const char* p) {
  typedef __attribute__((address_space(3))) s16x4_t* lds_ptr_t;
  const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
  return __builtin_bit_cast(u32x2_t, v);
}

// token (inside a 64-token tile) that lands at LDS position 8*tg + i of a staged V^T row
__device__ __forceinline__ int vt_token(int tg, int i) {
  return (tg >> 1) * 16 + (i >> 2) * 8 + (tg & 1) * 4 + (i & 3);
}

struct TileSrc {
  const int32_t* pages;
  int32_t page_size;
  int32_t page_shift;
  int32_t last_tok;
};

__device__ __forceinline__ int page_slot(const TileSrc& s, int tok) {
  return s.page_shift >= 0 ? (tok >> s.page_shift) : (tok / s.page_size);
}

// Byte offset of token `tok` of the tile starting at `tb`.  UNIFORM (page_size % 64 == 0):
// the tile lies inside the page `page`.
template <bool UNIFORM>
__device__ __forceinline__ int64_t row_offset(const TileSrc& s, const KvAddr& kv, int tb, int tok, int page) {
  tok = min(tok, s.last_tok);
  if constexpr (UNIFORM) {
    const int page_tok0 = page_slot(s, tb) * s.page_size;  // wave-uniform
    return (int64_t)page * kv.page_stride + (int64_t)((tok - page_tok0) * kv.tok_stride);
  } else {
    return (int64_t)page * kv.page_stride + (int64_t)(tok - page_slot(s, tok) * s.page_size) * kv.tok_stride;
  }
}

// ------------------------------------------------------------------ work decomposition
// A unit is one (sequence, kv head): its G query heads and all their query tiles read the
// same K/V, so a unit stays on one XCD (one L2).  Hardware deals workgroup n to XCD n % 8;
// XCD x owns units x, x+8, ...: units of one sequence cost the same, so the XCDs stay
// balanced whatever the ragged lengths are.  Inside an XCD the G heads of a unit sit next to
// each other and the most expensive query tiles are issued first, so that the last workgroups
// to start are short ones.  A causal tile costs what its last row sees: with a bound on kv_len
// from the host, tiles are ordered by level = tile index + ceil(prefix / tile rows), i.e. by
// that extent across sequences; without one, by position inside their own sequence.
struct Work {
  int seq, hk, head, q_start, qg0, q_len, kv_len, prefix;
  bool valid;
};

// `heads` query heads of a kv head per workgroup (1, or 4 when the waves of a workgroup take a head each):
// Work.head is then the first of them.
__device__ __forceinline__ Work decompose(const PrefillArgs& a, int tiles, int nseq, bool by_level, int bm = kBM,
                                          int heads = 1) {
  Work w;
  w.valid = false;
  const int units = nseq * a.Hkv;
  const int groups = a.G / heads;  // workgroups per (sequence, kv head, tile)
  int tile_rev, u, gi;
  if (units >= 8) {
    const int xcd = blockIdx.x & 7, r = blockIdx.x >> 3;
    const int units_per_xcd = (units + 7) >> 3;
    const int per_tile = units_per_xcd * groups;
    tile_rev = r / per_tile;
    const int rest = r - tile_rev * per_tile;
    u = xcd + 8 * (rest / groups);
    gi = (rest % groups) * heads;
  } else {
    const int per_tile = units * groups;
    tile_rev = blockIdx.x / per_tile;
    const int rest = blockIdx.x - tile_rev * per_tile;
    u = rest / groups;
    gi = (rest % groups) * heads;
  }
  if (u >= units || tile_rev >= tiles) return w;
  const int si = u / a.Hkv;
  w.hk = u - si * a.Hkv;
  w.head = w.hk * a.G + gi;
  w.seq = a.seq_begin + si;
  if (w.seq >= a.seq_end) return w;  // the grid was sized for a bound on the number of sequences
  w.qg0 = a.pt.cu_q_lens[w.seq];
  w.q_len = a.pt.cu_q_lens[w.seq + 1] - w.qg0;
  w.kv_len = a.pt.kv_lens[w.seq];
  w.prefix = w.kv_len - w.q_len;
  int tile = tiles - 1 - tile_rev;
  if (by_level) tile -= (max(w.prefix, 0) + bm - 1) / bm;
  w.q_start = tile * bm;
  if (tile < 0 || w.q_start >= w.q_len) return w;
  w.valid = true;
  return w;
}

__device__ __forceinline__ TileSrc make_src(const PrefillArgs& a, const Work& w) {
  TileSrc src;
  src.page_size = a.pt.page_size;
  src.page_shift = ((src.page_size & (src.page_size - 1)) == 0) ? (31 - __builtin_clz(src.page_size)) : -1;
  src.last_tok = w.kv_len - 1;
  src.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[w.seq] / a.pt.page_size)
                                                  : (int64_t)w.seq * a.pt.pages_per_seq);
  return src;
}

// ------------------------------------------------------------------ per-wave state and softmax
struct WaveRows {
  int r_lo, r_hi, row, qpos;
  bool active;
};

template <bool CAP>
struct Softmax {
  float scale, cap, inv_cap;
  float sc2;   // raw score -> log2 units inside the exponent (per row: carries the temperature factor)
  float temp;  // soft-cap path: temperature factor
  int round_mode;   // soft-cap path: logits rounded to bf16 (1) or f16 (2) before the softmax
};

// Online-softmax update of one 64-token tile.  On entry S holds raw scores (MFMA units); on
// exit it holds the probabilities.  Scores stay in MFMA units; sc2 turns them into log2 units
// inside the exponent: p = 2^(s*sc2 - m*sc2) is one fused multiply-add per score (soft-capped
// scores are already in log2 units, sc2 = 1).  The running max starts at a finite floor far
// above the mask value, so a row whose tokens are all masked in this tile gets p = 0, not 2^0.
constexpr f32x16_t kZero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
constexpr float kMaxFloor = -1.0e30f;
constexpr float kMaskRaw = -3.0e38f;

// The running max is allowed to go stale: it is raised (and the accumulators rescaled) only
// when some row's new maximum exceeds it by more than 2^kMaxSlack, so probabilities stay
// below 2^kMaxSlack -- harmless in f32 sums and bf16 operands -- and the 64-register rescale
// of O happens a handful of times per row instead of once per tile.
constexpr float kMaxSlack = 8.0f;

template <int ND>
__device__ __forceinline__ void update_running_max(float mx, float& m, float& l, f32x16_t (&O)[ND], float sc2) {
  if (__builtin_amdgcn_ballot_w64((mx - m) * sc2 > kMaxSlack) != 0) {
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2((m - m_new) * sc2);
    m = m_new;
    l *= alpha;
#pragma unroll
    for (int d = 0; d < ND; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) O[d][v] *= alpha;
  }
}

// xor-32 lane exchange of a maximum through v_permlane32_swap (no LDS round trip)
__device__ __forceinline__ float swap_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// Which tokens a query row may see.  mode 0: causal (token <= row position); mode 1: the
// caller's mask row (>= 1 keeps), mode 2: everything; modes 1 and 2 still hide the tokens of a
// partial last tile beyond kv_len.  The sliding window applies on top in every mode.
struct MaskCtx {
  int mode;
  int kv_len;
  const int32_t* row;    // mode 1: this lane's mask row (token t at row[t])
  const uint64_t* bits;  // mode 1: the same row as bits (token t = bit t % 64 of word t / 64), or nullptr
  int bit_words;         // words per bit row
};

__device__ __forceinline__ MaskCtx make_mask_ctx(const PrefillArgs& a, const Work& w, int row) {
  MaskCtx mc;
  mc.mode = a.sm.mask_mode;
  mc.kv_len = w.kv_len;
  mc.row = nullptr;
  mc.bits = nullptr;
  mc.bit_words = a.mask_pitch;
  if (mc.mode == 1 && a.mask_bits) mc.bits = a.mask_bits + (int64_t)(w.qg0 + min(row, w.q_len - 1)) * a.mask_pitch;
  if (mc.mode == 1) {
    const int width = a.sm.mask_rows_page_aligned ? (a.pt.cu_kv_lens[w.seq + 1] - a.pt.cu_kv_lens[w.seq]) : w.kv_len;
    mc.row = a.sm.custom_mask + a.sm.cu_mask_lens[w.seq] + (int64_t)min(row, w.q_len - 1) * width;
  }
  return mc;
}

// mask_word: with a caller's mask turned into bits (mc.bits), the word of this tile's 64 tokens, which the
// caller fetches at the top of the tile's step, in FRONT of the next tile's copy: loads return in order, so
// the wait for it leaves the copy in flight.  Without the bits, one 4-byte load per score, here, behind the
// first product (which waits for the copy as well).
template <bool CAP, bool EXT, int ND = 4>
__device__ __forceinline__ void softmax_tile(f32x16_t (&S)[2], f32x16_t (&O)[ND], float& m, float& l,
                                             const Softmax<CAP>& sm, bool need_mask, int tb, int h, int qpos,
                                             int window, u32x4_t (&pB)[2][2], const MaskCtx& mc,
                                             uint64_t mask_word = 0) {
  if constexpr (CAP && ND != 4) {
    // 256-wide heads: one loop with run-time choices (those kernels have no register to spare for variants)
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float x = S[mt][v] * sm.scale;
        if (sm.cap != 0.f) x = soft_cap_f(x, sm.cap, sm.inv_cap);
        x = x * sm.temp;
        if (sm.round_mode) x = round_logit(x, sm.round_mode);
        S[mt][v] = x * kLog2e;
      }
  } else if constexpr (CAP) {
    if (sm.cap != 0.f && !sm.round_mode) {
      // soft cap alone (the usual case), constants folded: five instructions per score.
      // cap tanh(s scale / cap) temp log2e = k2 - 2 k2 / (2^(s k1) + 1)
      const float k1 = sm.scale * sm.inv_cap * (2.0f * kLog2e), k2 = sm.cap * sm.temp * kLog2e;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          S[mt][v] = __builtin_fmaf(__builtin_amdgcn_rcpf(fast_exp2(S[mt][v] * k1) + 1.0f), -2.0f * k2, k2);
    } else {
      // the general path: soft cap (if any), temperature, then the logit rounded to the softmax dtype.  One loop
      // per combination, so that no score pays for a choice that is the same for the whole call.
      const bool capped = sm.cap != 0.f;
      const float k1 = sm.scale * sm.inv_cap * (2.0f * kLog2e), k2 = (capped ? sm.cap : sm.scale) * sm.temp;
      auto all_scores = [&](auto logit, auto rounded) __attribute__((always_inline)) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int v = 0; v < 16; ++v) S[mt][v] = rounded(logit(S[mt][v])) * kLog2e;
      };
      auto with_cap = [&](float s) { return __builtin_fmaf(__builtin_amdgcn_rcpf(fast_exp2(s * k1) + 1.0f), -2.0f * k2, k2); };
      auto no_cap = [&](float s) { return s * k2; };
      auto as_is = [](float x) { return x; };
      auto to_bf16 = [](float x) { return bf16_round(x); };
      auto to_f16 = [](float x) { return f16_round(x); };
      if (capped) {  // (rounded: the unrounded capped case is the branch above)
        if (sm.round_mode == 1) all_scores(with_cap, to_bf16);
        else all_scores(with_cap, to_f16);
      } else {
        if (sm.round_mode == 1) all_scores(no_cap, to_bf16);
        else if (sm.round_mode == 2) all_scores(no_cap, to_f16);
        else all_scores(no_cap, as_is);
      }
    }
  }
  if (EXT && ND == 4 && need_mask && mc.mode == 1 && mc.bits) {  // (128-wide heads: the 256-wide kernels have no register to spare)
    // the caller's mask as bits: the tile's 64 tokens are one word, fetched by the caller at the top of the step
    const uint32_t half[2] = {(uint32_t)mask_word >> (4 * h), (uint32_t)(mask_word >> 32) >> (4 * h)};
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int tok = tb + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        bool masked = (tok >= mc.kv_len) || !((half[mt] >> (8 * (v >> 2) + (v & 3))) & 1u);
        masked = masked || (window > 0 && tok <= qpos - window);
        S[mt][v] = masked ? kMaskRaw : S[mt][v];
      }
  } else if (need_mask) {
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int tok = tb + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        bool masked;
        if (!EXT || mc.mode == 0) masked = tok > qpos;
        else masked = (tok >= mc.kv_len) || (mc.mode == 1 && mc.row[tok] < 1);
        masked = masked || (window > 0 && tok <= qpos - window);
        S[mt][v] = masked ? kMaskRaw : S[mt][v];
      }
  }
  // 32 scores -> 1 with three-operand maxima: 16 instructions instead of 31
  float mx = __builtin_fmaxf(__builtin_fmaxf(S[0][0], S[0][1]), S[1][0]);
#pragma unroll
  for (int v = 1; v < 16; ++v) {
    if (v < 15) mx = __builtin_fmaxf(__builtin_fmaxf(mx, S[0][v + 1]), S[1][v]);
    else mx = __builtin_fmaxf(mx, S[1][v]);
  }
  mx = swap_max(mx);
  update_running_max<ND>(mx, m, l, O, sm.sc2);
  const float neg_m = -m * sm.sc2;
  // probabilities go straight into bf16 pairs (the B operands of the second product); the row
  // sum is taken over the rounded pairs, one dot instruction per pair
  const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
  float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p0 = fast_exp2(__builtin_fmaf(S[mt][8 * kk + 2 * j], sm.sc2, neg_m));
        const float p1 = fast_exp2(__builtin_fmaf(S[mt][8 * kk + 2 * j + 1], sm.sc2, neg_m));
        w[j] = pack_bf16x2(p0, p1);
        if (j & 1) ps1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[j]), ones, ps1, false);
        else ps0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[j]), ones, ps0, false);
      }
      pB[mt][kk] = u32x4_t{w[0], w[1], w[2], w[3]};
    }
  l += ps0 + ps1;
}

// lane (c, h) holds query row c, dims 32d + 8*(v/4) + 4h + v%4 in O[d][v]
template <int ND = 4>
__device__ __forceinline__ void write_rows(const PrefillArgs& a, const Work& w, const WaveRows& wr,
                                           const f32x16_t (&O)[ND], float l, int h, float m2) {
  l += __shfl_xor(l, 32);
  if (!wr.active || wr.row >= w.q_len) return;
  const float vs = a.v_scale ? a.v_scale[w.hk] : 1.0f;
  const float inv = a.sm.sink ? vs * sink_inverse(m2, l, sink_logit(a.sm.sink, a.sm.round_logits, w.head)) : vs / l;
  uint16_t* op = a.out + ((int64_t)(w.qg0 + wr.row) * a.Hq + w.head) * (ND * 32) + 4 * h;
#pragma unroll
  for (int d = 0; d < ND; ++d)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      u32x2_t o = {pack_bf16x2(O[d][4 * vq + 0] * inv, O[d][4 * vq + 1] * inv),
                   pack_bf16x2(O[d][4 * vq + 2] * inv, O[d][4 * vq + 3] * inv)};
      *reinterpret_cast<u32x2_t*>(op + d * 32 + vq * 8) = o;
    }
}

// -------------------------------------------------- the launch shape of a prefill call (rpa_shapes.h)
// RPA_PREFILL_PIPE=0 / RPA_PREFILL_STAGED=1 take the assembly kernel out of the selection, RPA_PREFILL_PIPE_TILE
// = 32 | 128 and RPA_PREFILL_PIPE_NQ=2 decide the short-chunk question by hand.
inline ShapeKey prefill_shape_key(const PrefillArgs& a) {
  const Tuning& tune = tuning();
  const int P = a.pt.page_size;
  ShapeKey k = {};
  k.stage = kStagePrefill;
  k.kv_bits = a.fp8 ? 8 : 16;
  k.head_dim = a.head_dim;
  k.heads = a.G;
  k.max_q_len = a.max_q_len;
  if (tune.prefill_pipe_tile == 32) k.max_q_len = 1;
  else if (tune.prefill_pipe_tile != 0 || tune.prefill_pipe_nq == 2) k.max_q_len = 0;
  k.options = ((a.sm.soft_cap != 0.f || a.sm.round_logits != 0) ? kOptSoftCap : 0u) |
              (a.sm.mask_mode != 0 ? kOptMaskOther : 0u) | (a.sm.xai_len > 0.f ? kOptTemperature : 0u) |
              (a.sm.q_scale > 0.f ? kOptQScale : 0u) | ((P % kBN) != 0 ? kOptOddPages : 0u) |
              ((P & (P - 1)) != 0 ? kOptNotPow2Pages : 0u) |
              (a.kv.page_stride >= (int64_t(1) << 32) ? kOptWidePages : 0u);
  return k;
}

inline const ShapeRule& prefill_shape(const PrefillArgs& a) {
  const Tuning& tune = tuning();
  const unsigned skip = (tune.prefill_pipe == 0 || tune.prefill_staged == 1) ? (1u << kKernelPrefillPipe) : 0u;
  return select_shape(prefill_shape_key(a), skip);
}

// -------------------------------------------------- K/V ranges cut into pieces (under-filled launches)
// A launch with far fewer workgroups than CUs (one long prompt on a few heads, a chunk on a long prefix, a
// verify step on a long context) cuts every workgroup's run of K/V tiles into a.kv_splits pieces; blockIdx.y
// picks the piece, which leaves its rows as they stand -- unnormalised accumulators, (reference, sum) of the
// probabilities in log2 units -- in workspace slot ((token, head), piece), and rpa_prefill_combine_kernel
// finishes them.
constexpr float kNoReference = -1.0e30f;  // reference of a row that met no visible token: weighs nothing in the merge

// The piece of [t_lo, t_hi) that this workgroup runs; false when nothing is left for it.
__device__ __forceinline__ bool kv_piece(const PrefillArgs& a, int& t_lo, int& t_hi, int& split) {
  split = blockIdx.y;
  const int nT = (t_hi - t_lo + kBN - 1) / kBN;
  // The host chose the number of pieces for the longest range it knew a bound of; a shorter range is cut into
  // fewer (no piece under four tiles), the workgroups of the others leave rows that weigh nothing.
  const int pieces = max(1, min(a.kv_splits, nT >> 2));
  // (the division runs on the vector pipe: say that its result is the same in every lane)
  const int per = __builtin_amdgcn_readfirstlane((nT + pieces - 1) / pieces);
  const int lo = split * per, hi = min(nT, lo + per);
  if (lo >= hi) return false;
  t_hi = min(t_hi, t_lo + hi * kBN);
  t_lo += lo * kBN;
  return true;
}

// lane (c, h) holds query row c, dims 32d + 8*(v/4) + 4h + v%4 in O[d][v]
template <int ND>
__device__ __forceinline__ void write_partial_rows(const PrefillArgs& a, const Work& w, const WaveRows& wr,
                                                   const f32x16_t (&O)[ND], float l, int h, float m2, int split) {
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  l += __shfl_xor(l, 32);
  if (!wr.active || wr.row >= w.q_len) return;
  const int64_t slot = ((int64_t)(w.qg0 + wr.row) * a.Hq + w.head) * a.kv_splits + split;
  float* op = a.ws_o + slot * (ND * 32) + 4 * h;
#pragma unroll
  for (int d = 0; d < ND; ++d)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq)
      *reinterpret_cast<f32x4_t*>(op + d * 32 + vq * 8) =
          f32x4_t{O[d][4 * vq + 0], O[d][4 * vq + 1], O[d][4 * vq + 2], O[d][4 * vq + 3]};
  if (h == 0) {
    a.ws_ml[slot * 2] = fmaxf(m2, kNoReference);
    a.ws_ml[slot * 2 + 1] = l;
  }
}

template <int ND>
__device__ __forceinline__ void write_empty_partial_rows(const PrefillArgs& a, const Work& w, const WaveRows& wr, int h,
                                                         int split) {
  f32x16_t zero[ND];
#pragma unroll
  for (int d = 0; d < ND; ++d) zero[d] = kZero16;
  write_partial_rows<ND>(a, w, wr, zero, 0.f, h, kNoReference, split);
}

// Merge the kv_splits partial rows of one (query token, query head): out = sum_j O_j 2^(m_j - m*) /
// sum_j l_j 2^(m_j - m*).  grid = (tokens, Hq); one wave, HD / 64 dims per lane; lane j fetches (m_j, l_j).
template <int HD>
static __global__ __launch_bounds__(64) void rpa_prefill_combine_kernel(const PrefillArgs a) {
  constexpr int kDpl = HD / 64;
  typedef float fvec_t __attribute__((ext_vector_type(kDpl)));
  // (with the call's composition on the device the sequences to process are read there, as in the kernels)
  int seq_begin = a.seq_begin, seq_end = a.seq_end;
  if (a.dist) {
    seq_begin = (a.sm.mask_mode == 1) ? 0 : scalar_load_i32(a.dist);
    seq_end = min(seq_end, scalar_load_i32(a.dist + 2));
  }
  const int tok0 = scalar_load_i32(a.pt.cu_q_lens + seq_begin);
  const int tok1 = scalar_load_i32(a.pt.cu_q_lens + seq_end);
  const int token = tok0 + (int)blockIdx.x;
  if (token >= tok1) return;
  const int head = blockIdx.y, lane = threadIdx.x, n = a.kv_splits;
  const int64_t base = ((int64_t)token * a.Hq + head) * n;
  float mj = -INFINITY, lj = 0.f;
  if (lane < n) {
    mj = a.ws_ml[(base + lane) * 2];
    lj = a.ws_ml[(base + lane) * 2 + 1];
  }
  float mstar = mj;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mstar = fmaxf(mstar, __shfl_xor(mstar, off));
  const float wj = (lane < n) ? fast_exp2(mj - mstar) : 0.f;
  float den = lj * wj;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) den += __shfl_xor(den, off);
  float acc[kDpl];
#pragma unroll
  for (int e = 0; e < kDpl; ++e) acc[e] = 0.f;
  for (int j0 = 0; j0 < n; j0 += 8) {  // eight partial rows requested at a time
    fvec_t o[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      o[u] = *reinterpret_cast<const fvec_t*>(a.ws_o + (base + min(j0 + u, n - 1)) * HD + kDpl * lane);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float wu = (j0 + u < n) ? __shfl(wj, j0 + u) : 0.f;  // the repeated last row does not count
#pragma unroll
      for (int e = 0; e < kDpl; ++e) acc[e] += o[u][e] * wu;
    }
  }
  const float vs = a.v_scale ? a.v_scale[head / a.G] : 1.0f;
  const float inv = a.sm.sink ? vs * sink_inverse(mstar, den, sink_logit(a.sm.sink, a.sm.round_logits, head)) : vs / den;
  uint32_t* op = reinterpret_cast<uint32_t*>(a.out + ((int64_t)token * a.Hq + head) * HD + kDpl * lane);
#pragma unroll
  for (int e = 0; e < kDpl; e += 2) op[e / 2] = pack_bf16x2(acc[e] * inv, acc[e + 1] * inv);
}

inline hipError_t launch_prefill_combine(const PrefillArgs& a, hipStream_t stream) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int64_t tokens = std::max<int64_t>(1, (int64_t)a.num_tokens - a.seq_begin);  // decode rows hold one token each
  const dim3 g((unsigned)tokens, (unsigned)a.Hq);
  if (a.head_dim == 256) hipLaunchKernelGGL(rpa_prefill_combine_kernel<256>, g, dim3(64), 0, stream, a);
  else hipLaunchKernelGGL(rpa_prefill_combine_kernel<128>, g, dim3(64), 0, stream, a);
  return hipGetLastError();
}

// How many pieces (1 = whole ranges): the count that minimises a small model of the launch, fitted to
// measurements of the pipelined kernel.  The critical path is the longest range, chain / n tiles per piece; a
// tile takes ~tile_us while every workgroup has a CU to itself (up to ~192 workgroups: the dispatcher does
// not spread them perfectly), 2.6 x that once two share every CU (512), in proportion in between, and the
// launch runs in rounds of 512 workgroups beyond; the merge costs a launch (~1.5 us) plus the partial rows'
// way to memory and back (~0.29 ns per (token, head, piece) of 128 dims).  A cut must save at least 2 us,
// leaves no piece under four tiles and makes at most 64 pieces.  bm / heads: query positions and query heads
// per workgroup.  RPA_PREFILL_SPLITS: 0 / 1 never, n forces n.
inline int kv_pieces(const PrefillArgs& a, int nseq, int bm, int heads, double tile_us) {
  // (with the composition on the device nseq, max_q_len, max_kv_len and num_tokens are bounds: a launch that is
  // under-filled even by its bounds is cut, and every workgroup fits the piece count to its own range)
  if (nseq <= 0 || a.max_q_len <= 0 || a.max_kv_len <= 0 || a.num_tokens <= 0) return 1;
  const int forced = tuning().prefill_splits;
  if (forced == 0 || forced == 1) return 1;
  if (forced > 1) return std::min(forced, 64);
  const int64_t tokens = std::max<int64_t>(1, (int64_t)a.num_tokens - a.seq_begin);
  const int64_t blocks = std::min<int64_t>((int64_t)nseq * ((a.max_q_len + bm - 1) / bm), tokens / bm + nseq);
  const int64_t wgs = blocks * a.Hkv * (a.G / heads);
  int64_t longest = a.max_kv_len;  // tokens of the longest range
  if (a.sm.window > 0) longest = std::min<int64_t>(longest, (int64_t)a.sm.window + bm + kBN);
  const int64_t chain = (longest + kBN - 1) / kBN;
  const int64_t cap = std::min<int64_t>(64, chain / 4);
  const double per_piece = 0.29e-3 * (double)tokens * a.Hq * (a.head_dim / 128);  // us per piece for the partial rows
  auto launch_us = [&](int n) {
    const double w = (double)wgs * n;
    const double rate = w <= 192 ? 1.0 : w <= 512 ? 1.0 + (w - 192) * (1.6 / 320) : 2.6 * (w / 512);
    return tile_us * rate * chain / n + (n > 1 ? 1.5 + per_piece * n : 0.0);
  };
  // (and the partial rows stay under 256 MB)
  const int64_t row_bytes = (int64_t)a.num_tokens * a.Hq * (a.head_dim + 2) * 4;
  const int64_t cap_ws = row_bytes > 0 ? ((int64_t)256 << 20) / row_bytes : 64;
  int best = 1;
  double best_us = launch_us(1) - 2.0;
  for (int n = 2; n <= cap && n <= cap_ws; ++n) {
    const double us = launch_us(n);
    if (us < best_us) {
      best_us = us;
      best = n;
    }
  }
  return best;
}

// ==================================================================== async path (bf16 cache)
// Geometry of a tile for head dim HD (128 or 256): rows stay row-major and unpadded in LDS.
template <int HD>
struct Tile {
  static constexpr int kRowB = HD * 2;          // one K or V row of a head, bf16
  static constexpr int kTileB = kBN * kRowB;    // 16 or 32 KiB
  static constexpr int kChunks = HD / 8;        // 16-byte chunks per row
  static constexpr int kSteps = HD / 16;        // k-steps of the first product
  static constexpr int kDimTiles = HD / 32;     // 32-dim output tiles of the second product
  static constexpr int kCopies = kChunks / 4;   // copy instructions per wave, for K and for V
  static constexpr int kRowsPerCopy = 64 / kChunks;
};

// 16-byte chunk j of row t sits at chunk position j ^ swizzle(t):
//   K: swizzle = t & 15      (ds_read_b128: 16 consecutive tokens -> 16 distinct chunk columns)
//   V: swizzle = 4 * (t & 3) (transposing read: 4 consecutive tokens -> 4 distinct 64-byte windows)
template <bool UNIFORM, int HD>
struct AsyncPages {
  int32_t id[UNIFORM ? 1 : Tile<HD>::kCopies];
};

template <bool UNIFORM, int HD>
__device__ __forceinline__ void async_fetch_pages(AsyncPages<UNIFORM, HD>& pg, const TileSrc& s, int tb, int wave,
                                                  int lane) {
  using T = Tile<HD>;
  tb = min(tb, s.last_tok & ~(kBN - 1));
  if constexpr (UNIFORM) {
    pg.id[0] = scalar_load_i32(s.pages + __builtin_amdgcn_readfirstlane(page_slot(s, tb)));
  } else {
#pragma unroll
    for (int n = 0; n < T::kCopies; ++n) {
      const int t = (wave * T::kCopies + n) * T::kRowsPerCopy + lane / T::kChunks;
      pg.id[n] = s.pages[page_slot(s, min(tb + t, s.last_tok))];
    }
  }
}

// Every wave copies kCopies x 64 chunks of K and of V: chunk position p = 64*(kCopies*wave + n) +
// lane of the tile, i.e. row p / kChunks, chunk column p % kChunks.  For a full tile inside one
// page the byte offset of a lane's chunk from the tile's first row never changes: it is computed
// once (AsyncOffsets) and a copy costs no vector ALU work, only a scalar tile base.
template <int HD>
struct AsyncOffsets {
  uint32_t k[Tile<HD>::kCopies], v[Tile<HD>::kCopies];
};

template <int HD>
__device__ __forceinline__ AsyncOffsets<HD> make_async_offsets(const KvAddr& kv, int wave, int lane) {
  using T = Tile<HD>;
  AsyncOffsets<HD> o;
  const int cp = lane % T::kChunks;
#pragma unroll
  for (int n = 0; n < T::kCopies; ++n) {
    const int t = (wave * T::kCopies + n) * T::kRowsPerCopy + lane / T::kChunks;
    o.k[n] = (uint32_t)(t * kv.tok_stride + ((cp ^ (t & 15)) << 4));
    o.v[n] = (uint32_t)(t * kv.tok_stride + ((cp ^ ((t & 3) << 2)) << 4));
  }
  return o;
}

template <bool UNIFORM, int HD>
__device__ __forceinline__ void async_copy_tile(char* lds_k, char* lds_v, const TileSrc& s, const KvAddr& kv,
                                                const char* kh, const char* vh, int tb, int wave, int lane,
                                                const AsyncPages<UNIFORM, HD>& pg, const AsyncOffsets<HD>& ofs) {
  using T = Tile<HD>;
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  tb = min(tb, s.last_tok & ~(kBN - 1));  // past the end: re-copy the last tile
  if constexpr (UNIFORM) {
    if (tb + kBN - 1 <= s.last_tok) {
      const int64_t base = (int64_t)pg.id[0] * kv.page_stride +
                           (int64_t)(tb - page_slot(s, tb) * s.page_size) * kv.tok_stride;  // scalar
      const char* kb = kh + base;
      const char* vb = vh + base;
#pragma unroll
      for (int n = 0; n < T::kCopies; ++n) {
        const int blk = wave * T::kCopies + n;
        __builtin_amdgcn_global_load_lds((gptr_t)(kb + ofs.k[n]), (lptr_t)(lds_k + blk * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(vb + ofs.v[n]), (lptr_t)(lds_v + blk * 1024), 16, 0, 0);
      }
      return;
    }
  }
  // last, partial tile (rows clamped to the last valid token) or pages smaller than a tile
  const int cp = lane % T::kChunks;
#pragma unroll
  for (int n = 0; n < T::kCopies; ++n) {
    const int blk = wave * T::kCopies + n;
    const int t = blk * T::kRowsPerCopy + lane / T::kChunks;
    const int64_t ro = row_offset<UNIFORM>(s, kv, tb, tb + t, pg.id[UNIFORM ? 0 : n]);
    const int jk = cp ^ (t & 15);
    const int jv = cp ^ ((t & 3) << 2);
    __builtin_amdgcn_global_load_lds((gptr_t)(kh + ro + jk * 16), (lptr_t)(lds_k + blk * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(vh + ro + jv * 16), (lptr_t)(lds_v + blk * 1024), 16, 0, 0);
  }
}
}  // namespace pf

// rpa_prefill_pipe.hip: the software-pipelined kernel for the plain causal bf16 case
bool prefill_pipe_applies(const PrefillArgs& a);
hipError_t launch_prefill_pipe(const PrefillArgs& a, int nseq, bool level_order, hipStream_t stream);
int prefill_pipe_kv_splits(const PrefillArgs& a, int nseq);

}  // namespace rpa
