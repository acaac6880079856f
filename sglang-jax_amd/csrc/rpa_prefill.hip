// Flash-style prefill / mixed kernel for ragged paged attention on gfx950.
//
// One workgroup (4 waves) owns a tile of 128 query positions of one query head
// of one sequence; wave w owns 32 of them.  KV is walked in tiles of 64 tokens
// gathered through the page table into a two-deep LDS ring (tile t+1 arrives
// while tile t is consumed, one barrier per tile):
//   S^T[tok, q]  = K . Q^T        v_mfma_f32_32x32x16_bf16, A = K rows from LDS,
//                                 B = Q^T held in registers for the whole loop
//   online softmax per query column (in-lane over tokens + one lane swap)
//   O^T[dim, q] += V^T . P^T      A = V^T from LDS, B = P^T straight from the
//                                 S^T result registers
// The S^T result layout (lane = query, registers = tokens) is the B operand
// layout of the second product when the 16 tokens of a k-step are ordered
// 16kk + 8*(i/4) + 4h + i%4 -- no data crosses lanes between the two products.
//
// Two data paths feed the LDS ring:
//   * bf16 cache ("async"): global_load_lds_dwordx4 copies 16-byte chunks straight
//     into LDS, rows kept row-major with XOR-swizzled chunk positions (no padding,
//     no staging registers).  K operands are ds_read_b128; V^T operands come from
//     the row-major V rows through the transposing LDS read ds_read_b64_tr_b16.
//   * fp8 cache ("staged"): rows pass through registers, are dequantised to bf16
//     once, and V is transposed in registers (v_perm_b32) before it is written.
//
// Workgroup ids are remapped so that everything that reads one kv head of one
// sequence runs on the same XCD (same L2) while the ragged sequences are spread
// evenly over the 8 XCDs: hardware deals workgroup n to XCD n % 8.

#include <cstdlib>

#include "rpa_common.h"
#include "rpa_kernels.h"

namespace rpa {

namespace {

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

__device__ __forceinline__ Work decompose(const PrefillArgs& a, int tiles, int nseq, bool by_level) {
  Work w;
  w.valid = false;
  const int units = nseq * a.Hkv;
  int tile_rev, u, gi;
  if (units >= 8) {
    const int xcd = blockIdx.x & 7, r = blockIdx.x >> 3;
    const int units_per_xcd = (units + 7) >> 3;
    const int per_tile = units_per_xcd * a.G;
    tile_rev = r / per_tile;
    const int rest = r - tile_rev * per_tile;
    u = xcd + 8 * (rest / a.G);
    gi = rest % a.G;
  } else {
    const int per_tile = units * a.G;
    tile_rev = blockIdx.x / per_tile;
    const int rest = blockIdx.x - tile_rev * per_tile;
    u = rest / a.G;
    gi = rest % a.G;
  }
  if (u >= units || tile_rev >= tiles) return w;
  const int si = u / a.Hkv;
  w.hk = u - si * a.Hkv;
  w.head = w.hk * a.G + gi;
  w.seq = a.seq_begin + si;
  w.qg0 = a.pt.cu_q_lens[w.seq];
  w.q_len = a.pt.cu_q_lens[w.seq + 1] - w.qg0;
  w.kv_len = a.pt.kv_lens[w.seq];
  w.prefix = w.kv_len - w.q_len;
  int tile = tiles - 1 - tile_rev;
  if (by_level) tile -= (max(w.prefix, 0) + kBM - 1) / kBM;
  w.q_start = tile * kBM;
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
  const int32_t* row;  // mode 1: this lane's mask row (token t at row[t])
};

__device__ __forceinline__ MaskCtx make_mask_ctx(const PrefillArgs& a, const Work& w, int row) {
  MaskCtx mc;
  mc.mode = a.sm.mask_mode;
  mc.kv_len = w.kv_len;
  mc.row = nullptr;
  if (mc.mode == 1) {
    const int width = a.sm.mask_rows_page_aligned ? (a.pt.cu_kv_lens[w.seq + 1] - a.pt.cu_kv_lens[w.seq]) : w.kv_len;
    mc.row = a.sm.custom_mask + a.sm.cu_mask_lens[w.seq] + (int64_t)min(row, w.q_len - 1) * width;
  }
  return mc;
}

template <bool CAP, bool EXT, int ND = 4>
__device__ __forceinline__ void softmax_tile(f32x16_t (&S)[2], f32x16_t (&O)[ND], float& m, float& l,
                                             const Softmax<CAP>& sm, bool need_mask, int tb, int h, int qpos,
                                             int window, u32x4_t (&pB)[2][2], const MaskCtx& mc) {
  if constexpr (CAP) {
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        // the general path: soft cap (if any), temperature, rounding of the logit (if asked)
        float x = S[mt][v] * sm.scale;
        if (sm.cap != 0.f) x = soft_cap_f(x, sm.cap, sm.inv_cap);
        x = x * sm.temp;
        if (sm.round_mode) x = round_logit(x, sm.round_mode);
        S[mt][v] = x * kLog2e;
      }
  }
  if (need_mask) {
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

// EXT compiles in the rarely used options (temperature factor, custom mask / no mask); the
// plain causal instantiation keeps its scale in a scalar register and its mask test to one compare.
// HD = 256 doubles the rows in LDS (two 64 KiB slots), the Q^T operands and the accumulators: one
// workgroup per CU, one wave per SIMD with up to 512 registers.
template <bool UNIFORM, bool CAP, bool EXT, int HD = 128>
__global__ __launch_bounds__(256, (HD == 128 ? 2 : 1)) void rpa_prefill_async_kernel(const PrefillArgs a, int tiles, int nseq,
                                                                                  bool by_level) {
  using T = Tile<HD>;
  constexpr int kRowB = T::kRowB;
  constexpr int kTileB = T::kTileB;
  // Four separate arrays (not one indexed array): the compiler can then prove that the
  // asynchronous copy into one ring slot does not alias the LDS reads of the other slot and
  // does not drain the vector-memory queue in the middle of a tile.
  __shared__ __attribute__((aligned(1024))) char lds_k0[kTileB];
  __shared__ __attribute__((aligned(1024))) char lds_k1[kTileB];
  __shared__ __attribute__((aligned(1024))) char lds_v0[kTileB];
  __shared__ __attribute__((aligned(1024))) char lds_v1[kTileB];

  const Work w = decompose(a, tiles, nseq, by_level);
  if (!w.valid) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, h = lane >> 5;
  const TileSrc src = make_src(a, w);
  const char* kh = a.kv.k_base + (int64_t)w.hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)w.hk * a.kv.head_stride;

  WaveRows wr;
  wr.r_lo = w.q_start + wave * 32;
  wr.r_hi = min(wr.r_lo + 31, w.q_len - 1);
  wr.active = wr.r_lo < w.q_len;
  wr.row = wr.r_lo + c;
  wr.qpos = w.prefix + wr.row;
  const int W_ = a.sm.window;

  u32x4_t qB[T::kSteps];
  {
    const int rr = min(wr.row, w.q_len - 1);
    const uint16_t* qp = a.q + ((int64_t)(w.qg0 + rr) * a.Hq + w.head) * HD + h * 8;
#pragma unroll
    for (int ks = 0; ks < T::kSteps; ++ks) qB[ks] = ld16(qp + ks * 16);
    if (EXT && a.sm.q_scale > 0.f) {
#pragma unroll
      for (int ks = 0; ks < T::kSteps; ++ks) qB[ks] = requantise_q(qB[ks], a.sm.q_scale, false);
    }
  }
  Softmax<CAP> sm;
  sm.scale = a.sm.sm_scale * (a.k_scale ? a.k_scale[w.hk] : 1.0f) *
             ((EXT && a.sm.q_scale > 0.f) ? a.sm.q_scale : 1.0f);
  sm.cap = a.sm.soft_cap;
  sm.inv_cap = (sm.cap != 0.f) ? 1.0f / sm.cap : 0.f;
  {
    const float temp = EXT ? xai_factor(wr.qpos, a.sm.xai_len) : 1.0f;  // per query row
    sm.sc2 = CAP ? 1.0f : sm.scale * kLog2e * temp;
    sm.temp = temp;
    sm.round_mode = a.sm.round_logits;
  }

  f32x16_t O[T::kDimTiles];
#pragma unroll
  for (int d = 0; d < T::kDimTiles; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) O[d][v] = 0.f;
  float m = kMaxFloor, l = 0.f;

  const int wg_r_hi = min(w.q_start + kBM, w.q_len) - 1;
  const bool causal = !EXT || a.sm.mask_mode == 0;
  MaskCtx mc;
  mc.mode = 0;
  if constexpr (EXT) mc = make_mask_ctx(a, w, wr.row);
  const int t_hi = causal ? min(w.kv_len, w.prefix + wg_r_hi + 1) : w.kv_len;  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, w.prefix + w.q_start - W_ + 1) & ~(kBN - 1);

  // ---- operand addresses inside a tile (bytes) ----
  // K operand of (m-tile mt, k-step ks): row 32mt + c, chunk (2ks + h) ^ (c & 15)
  const int k_row = c * kRowB;
  const int k_swz = (h ^ (c & 15)) << 4;  // chunk = (2ks) ^ (h ^ (c & 15)), in bytes: (32ks) ^ k_swz
  // V^T operand of (dim tile d, m-tile mt, k-step kk), first / second half of the k-step:
  //   source lane r = lane & 15 of its 16-lane block points at token 32mt + 16kk + 4h + (r >> 2) (+ 8),
  //   dims 32d + 16*(block & 1) + 4*(r & 3); chunk = (4d + 2*(block & 1) + ((r & 3) >> 1)) ^ (4*(r >> 2))
  const int r16 = lane & 15, b16 = lane >> 4;
  const int v_row = (4 * h + (r16 >> 2)) * kRowB;
  const int v_in = ((b16 & 1) << 5) + (((r16 & 3) >> 1) << 4) + ((r16 & 1) << 3);
  const int v_swz = (r16 >> 2) << 6;  // byte offset of the 64-byte window: (64d) ^ v_swz
  // The swizzled offsets are kept in registers for the whole loop (12 of them) instead of being
  // recomputed in front of each of the 48 LDS reads of a tile; slot bases and row steps fold
  // into the instructions' immediate offsets.
  int koff[T::kSteps], voff[T::kDimTiles];
#pragma unroll
  for (int ks = 0; ks < T::kSteps; ++ks) {
    koff[ks] = k_row + ((ks * 32) ^ k_swz);
    asm volatile("" : "+v"(koff[ks]));
  }
#pragma unroll
  for (int d = 0; d < T::kDimTiles; ++d) {
    voff[d] = v_row + v_in + ((d * 64) ^ v_swz);
    asm volatile("" : "+v"(voff[d]));
  }

  // ---- pipeline: page ids two tiles ahead, the asynchronous copy one tile ahead ----
  const AsyncOffsets<HD> ofs = make_async_offsets<HD>(a.kv, wave, lane);
  AsyncPages<UNIFORM, HD> pg;
  async_fetch_pages<UNIFORM, HD>(pg, src, t_lo, wave, lane);
  async_copy_tile<UNIFORM, HD>(lds_k0, lds_v0, src, a.kv, kh, vh, t_lo, wave, lane, pg, ofs);
  async_fetch_pages<UNIFORM, HD>(pg, src, t_lo + kBN, wave, lane);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the copies have landed in LDS
  __syncthreads();

  // one tile: consume (lds_k, lds_v), fill (nxt_k, nxt_v) with the tile after it
  auto tile_step = [&](const char* lds_k, const char* lds_v, char* nxt_k, char* nxt_v, int tb) {
    if (tb + kBN < t_hi) {
      // the other slot was last read before the barrier that ended the previous tile
      async_copy_tile<UNIFORM, HD>(nxt_k, nxt_v, src, a.kv, kh, vh, tb + kBN, wave, lane, pg, ofs);
      async_fetch_pages<UNIFORM, HD>(pg, src, tb + 2 * kBN, wave, lane);
    }
    // visible to this wave?  causal: some token <= last row's position; window: some token
    // newer than the first row's horizon
    const bool vis = wr.active && (!causal || tb <= w.prefix + wr.r_hi) &&
                     (W_ <= 0 || tb + kBN - 1 > w.prefix + wr.r_lo - W_);
    if (vis) {
      const bool need_mask = (causal ? (tb + kBN - 1 > w.prefix + wr.r_lo) : (mc.mode == 1 || tb + kBN > w.kv_len)) ||
                             (W_ > 0 && tb <= w.prefix + wr.r_hi - W_);
      {
        // the two 32-token halves form two independent accumulator chains, issued alternately
        f32x16_t S[2];
        S[0] = mfma32(lds_ld16(lds_k + koff[0]), qB[0], kZero16);  // zero accumulator as an inline constant
        S[1] = mfma32(lds_ld16(lds_k + koff[0] + 32 * kRowB), qB[0], kZero16);
#pragma unroll
        for (int ks = 1; ks < T::kSteps; ++ks) {
          S[0] = mfma32(lds_ld16(lds_k + koff[ks]), qB[ks], S[0]);
          S[1] = mfma32(lds_ld16(lds_k + koff[ks] + 32 * kRowB), qB[ks], S[1]);
        }
        u32x4_t pB[2][2];
        softmax_tile<CAP, EXT, T::kDimTiles>(S, O, m, l, sm, need_mask, tb, h, wr.qpos, W_, pB, mc);
        // independent accumulator chains (dim tiles), issued round-robin
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int d = 0; d < T::kDimTiles; ++d) {
              const char* vt = lds_v + voff[d] + (mt * 32 + kk * 16) * kRowB;
              const u32x2_t lo = lds_tr16(vt);
              const u32x2_t hi = lds_tr16(vt + 8 * kRowB);
              O[d] = mfma32(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, pB[mt][kk], O[d]);
            }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the next tile has landed
    __syncthreads();
  };
  for (int tb = t_lo; tb < t_hi; tb += 2 * kBN) {
    tile_step(lds_k0, lds_v0, lds_k1, lds_v1, tb);
    if (tb + kBN >= t_hi) break;
    tile_step(lds_k1, lds_v1, lds_k0, lds_v0, tb + kBN);
  }
  write_rows<T::kDimTiles>(a, w, wr, O, l, h, m * sm.sc2);
}

// ==================================================================== staged path (fp8 cache)
constexpr int kKPitch = 272;  // bytes per K row in LDS (256 + 16 pad: conflict-free b128 reads)
constexpr int kVPitch = 144;  // bytes per V^T row in LDS (128 + 16 pad)

template <bool UNIFORM>
struct PageIds {
  int32_t id[UNIFORM ? 1 : 8];
};

template <bool FP8>
struct Stage {
  u32x4_t r[FP8 ? 4 : 8];
};

template <bool UNIFORM>
__device__ __forceinline__ void fetch_page_ids(PageIds<UNIFORM>& pg, const TileSrc& s, int tb, int tid) {
  tb = min(tb, s.last_tok & ~(kBN - 1));
  if constexpr (UNIFORM) {
    pg.id[0] = scalar_load_i32(s.pages + __builtin_amdgcn_readfirstlane(page_slot(s, tb)));
  } else {
    if (tid < 128) {
      pg.id[0] = s.pages[page_slot(s, min(tb + (tid >> 1), s.last_tok))];
    } else {
      const int tg = (tid - 128) & 7;
#pragma unroll
      for (int i = 0; i < 8; ++i) pg.id[i] = s.pages[page_slot(s, min(tb + vt_token(tg, i), s.last_tok))];
    }
  }
}

// Threads 0..127 stage K (one half row each), threads 128..255 stage V (8 tokens x 8 dims each).
template <bool FP8, bool UNIFORM>
__device__ __forceinline__ void tile_gload(Stage<FP8>& st, const TileSrc& s, const KvAddr& kv, const char* kh,
                                           const char* vh, int tb, int tid, const PageIds<UNIFORM>& pg) {
  tb = min(tb, s.last_tok & ~(kBN - 1));  // past the end: re-read the last tile
  if (tid < 128) {
    const int tl = tid >> 1, half = tid & 1;
    const char* p = kh + row_offset<UNIFORM>(s, kv, tb, tb + tl, pg.id[0]) + half * (FP8 ? 64 : 128);
#pragma unroll
    for (int i = 0; i < (FP8 ? 4 : 8); ++i) st.r[i] = ld16(p + i * 16);
  } else {
    const int u = tid - 128;
    const int tg = u & 7, dc = u >> 3;
    if constexpr (FP8) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const u32x2_t x =
            ld8(vh + row_offset<UNIFORM>(s, kv, tb, tb + vt_token(tg, i), pg.id[UNIFORM ? 0 : i]) + dc * 8);
        st.r[i >> 1][(i & 1) * 2 + 0] = x[0];
        st.r[i >> 1][(i & 1) * 2 + 1] = x[1];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        st.r[i] = ld16(vh + row_offset<UNIFORM>(s, kv, tb, tb + vt_token(tg, i), pg.id[UNIFORM ? 0 : i]) + dc * 16);
    }
  }
}

template <bool FP8>
__device__ __forceinline__ void tile_lstore(const Stage<FP8>& st, char* lds_k, char* lds_v, int tid) {
  if (tid < 128) {
    const int tl = tid >> 1, half = tid & 1;
    char* p = lds_k + tl * kKPitch + half * 128;
    if constexpr (FP8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32x2_t a = fp8x4_to_bf16x4(st.r[i][0]);
        const u32x2_t b = fp8x4_to_bf16x4(st.r[i][1]);
        const u32x2_t c = fp8x4_to_bf16x4(st.r[i][2]);
        const u32x2_t d = fp8x4_to_bf16x4(st.r[i][3]);
        lds_st16(p + i * 32, u32x4_t{a[0], a[1], b[0], b[1]});
        lds_st16(p + i * 32 + 16, u32x4_t{c[0], c[1], d[0], d[1]});
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) lds_st16(p + i * 16, st.r[i]);
    }
  } else {
    const int u = tid - 128;
    const int tg = u & 7, dc = u >> 3;
    char* p = lds_v + (dc * 8) * kVPitch + tg * 16;
    if constexpr (FP8) {
      float f[8][8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t w0 = st.r[i >> 1][(i & 1) * 2 + 0];
        const uint32_t w1 = st.r[i >> 1][(i & 1) * 2 + 1];
        const f32x2_t a0 = __builtin_amdgcn_cvt_pk_f32_fp8(w0, false);
        const f32x2_t a1 = __builtin_amdgcn_cvt_pk_f32_fp8(w0, true);
        const f32x2_t a2 = __builtin_amdgcn_cvt_pk_f32_fp8(w1, false);
        const f32x2_t a3 = __builtin_amdgcn_cvt_pk_f32_fp8(w1, true);
        f[i][0] = a0[0]; f[i][1] = a0[1]; f[i][2] = a1[0]; f[i][3] = a1[1];
        f[i][4] = a2[0]; f[i][5] = a2[1]; f[i][6] = a3[0]; f[i][7] = a3[1];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        lds_st16(p + j * kVPitch, u32x4_t{pack_bf16x2(f[0][j], f[1][j]), pack_bf16x2(f[2][j], f[3][j]),
                                          pack_bf16x2(f[4][j], f[5][j]), pack_bf16x2(f[6][j], f[7][j])});
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
        const int jj = j >> 1;
        lds_st16(p + j * kVPitch,
                 u32x4_t{__builtin_amdgcn_perm(st.r[1][jj], st.r[0][jj], sel),
                         __builtin_amdgcn_perm(st.r[3][jj], st.r[2][jj], sel),
                         __builtin_amdgcn_perm(st.r[5][jj], st.r[4][jj], sel),
                         __builtin_amdgcn_perm(st.r[7][jj], st.r[6][jj], sel)});
      }
    }
  }
}

template <bool FP8, bool UNIFORM, bool CAP, bool EXT>
__global__ __launch_bounds__(256, 2) void rpa_prefill_staged_kernel(const PrefillArgs a, int tiles, int nseq, bool by_level) {
  __shared__ __attribute__((aligned(16))) char lds_k_buf[2][kBN * kKPitch];
  __shared__ __attribute__((aligned(16))) char lds_v_buf[2][128 * kVPitch];

  const Work w = decompose(a, tiles, nseq, by_level);
  if (!w.valid) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5;
  const TileSrc src = make_src(a, w);
  const char* kh = a.kv.k_base + (int64_t)w.hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)w.hk * a.kv.head_stride;

  WaveRows wr;
  wr.r_lo = w.q_start + wave * 32;
  wr.r_hi = min(wr.r_lo + 31, w.q_len - 1);
  wr.active = wr.r_lo < w.q_len;
  wr.row = wr.r_lo + c;
  wr.qpos = w.prefix + wr.row;
  const int W_ = a.sm.window;

  u32x4_t qB[8];
  {
    const int rr = min(wr.row, w.q_len - 1);
    const uint16_t* qp = a.q + ((int64_t)(w.qg0 + rr) * a.Hq + w.head) * 128 + h * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qB[ks] = ld16(qp + ks * 16);
    if (EXT && a.sm.q_scale > 0.f) {
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) qB[ks] = requantise_q(qB[ks], a.sm.q_scale, FP8);
    }
  }
  Softmax<CAP> sm;
  sm.scale = a.sm.sm_scale * (a.k_scale ? a.k_scale[w.hk] : 1.0f) *
             ((EXT && a.sm.q_scale > 0.f) ? a.sm.q_scale : 1.0f);
  sm.cap = a.sm.soft_cap;
  sm.inv_cap = (sm.cap != 0.f) ? 1.0f / sm.cap : 0.f;
  {
    const float temp = EXT ? xai_factor(wr.qpos, a.sm.xai_len) : 1.0f;  // per query row
    sm.sc2 = CAP ? 1.0f : sm.scale * kLog2e * temp;
    sm.temp = temp;
    sm.round_mode = a.sm.round_logits;
  }

  f32x16_t O[4];
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) O[d][v] = 0.f;
  float m = kMaxFloor, l = 0.f;

  const int wg_r_hi = min(w.q_start + kBM, w.q_len) - 1;
  const bool causal = !EXT || a.sm.mask_mode == 0;
  MaskCtx mc;
  mc.mode = 0;
  if constexpr (EXT) mc = make_mask_ctx(a, w, wr.row);
  const int t_hi = causal ? min(w.kv_len, w.prefix + wg_r_hi + 1) : w.kv_len;  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, w.prefix + w.q_start - W_ + 1) & ~(kBN - 1);

  // ---- pipeline: page ids run two tiles ahead, rows one tile ahead (in registers), LDS one
  // tile ahead of the MFMAs.  Loads past the last tile re-read the last tile.
  Stage<FP8> stg;
  PageIds<UNIFORM> pg;
  fetch_page_ids<UNIFORM>(pg, src, t_lo, tid);
  tile_gload<FP8, UNIFORM>(stg, src, a.kv, kh, vh, t_lo, tid, pg);
  fetch_page_ids<UNIFORM>(pg, src, t_lo + kBN, tid);
  tile_lstore<FP8>(stg, lds_k_buf[0], lds_v_buf[0], tid);
  tile_gload<FP8, UNIFORM>(stg, src, a.kv, kh, vh, t_lo + kBN, tid, pg);
  fetch_page_ids<UNIFORM>(pg, src, t_lo + 2 * kBN, tid);
  __syncthreads();
  int buf = 0;
  for (int tb = t_lo; tb < t_hi; tb += kBN, buf ^= 1) {
    const char* lds_k = lds_k_buf[buf];
    const char* lds_v = lds_v_buf[buf];
    if (tb + kBN < t_hi) {
      // the other buffer was last read before the barrier that ended the previous tile
      tile_lstore<FP8>(stg, lds_k_buf[buf ^ 1], lds_v_buf[buf ^ 1], tid);
      tile_gload<FP8, UNIFORM>(stg, src, a.kv, kh, vh, tb + 2 * kBN, tid, pg);
      fetch_page_ids<UNIFORM>(pg, src, tb + 3 * kBN, tid);
    }
    const bool vis = wr.active && (!causal || tb <= w.prefix + wr.r_hi) &&
                     (W_ <= 0 || tb + kBN - 1 > w.prefix + wr.r_lo - W_);
    if (vis) {
      const bool need_mask = (causal ? (tb + kBN - 1 > w.prefix + wr.r_lo) : (mc.mode == 1 || tb + kBN > w.kv_len)) ||
                             (W_ > 0 && tb <= w.prefix + wr.r_hi - W_);
      f32x16_t S[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const char* kp = lds_k + (mt * 32 + c) * kKPitch + h * 16;
        S[mt] = mfma32(lds_ld16(kp), qB[0], kZero16);
#pragma unroll
        for (int ks = 1; ks < 8; ++ks) S[mt] = mfma32(lds_ld16(kp + ks * 32), qB[ks], S[mt]);
      }
      u32x4_t pB[2][2];
      softmax_tile<CAP, EXT>(S, O, m, l, sm, need_mask, tb, h, wr.qpos, W_, pB, mc);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const char* vp = lds_v + (d * 32 + c) * kVPitch + h * 16;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk)
            O[d] = mfma32(lds_ld16(vp + (mt * 32 + kk * 16) * 2), pB[mt][kk], O[d]);
      }
    }
    __syncthreads();
  }
  write_rows(a, w, wr, O, l, h, m * sm.sc2);
}

}  // namespace

hipError_t launch_prefill(const PrefillArgs& a, hipStream_t stream) {
  const int nseq = a.seq_end - a.seq_begin;
  if (nseq <= 0 || a.max_q_len <= 0) return hipSuccess;
  int tiles = (a.max_q_len + kBM - 1) / kBM;
  // levels 0 .. ceil(max_kv_len / rows): only worth their empty workgroups when prefixes are
  // not much longer than the chunks (else every tile of a sequence costs about the same anyway)
  static const bool level_order = [] { const char* v = getenv("RPA_PREFILL_LEVEL_ORDER"); return !(v && *v == '0'); }();
  const int levels = a.max_kv_len > 0 ? (a.max_kv_len + kBM - 1) / kBM + 1 : 0;
  const bool by_level = level_order && a.sm.mask_mode == 0 && levels > tiles && levels <= 2 * tiles + 2;
  if (by_level) tiles = levels;
  const int64_t units = (int64_t)nseq * a.Hkv;
  const int64_t grid = (units >= 8 ? ((units + 7) / 8) * 8 : units) * a.G * tiles;
  if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool uniform = (a.pt.page_size % kBN) == 0;
  // soft cap and logit rounding share the general score path
  const bool cap = a.sm.soft_cap != 0.f || a.sm.round_logits != 0;
  static const bool force_staged = [] { const char* v = getenv("RPA_PREFILL_STAGED"); return v && *v == '1'; }();
  const bool staged = a.fp8 || force_staged;
  const dim3 g((unsigned)grid), blk(256);
  const bool ext = a.sm.xai_len > 0.f || a.sm.mask_mode != 0 || a.sm.q_scale > 0.f;
#define RPA_STAGED(F, U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_staged_kernel<F, U, C, E>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_ASYNC(U, C, E) hipLaunchKernelGGL((rpa_prefill_async_kernel<U, C, E>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_ASYNC256(U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_async_kernel<U, C, E, 256>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_PICK(M, ...)                                            \
  switch ((uniform ? 4 : 0) | (cap ? 2 : 0) | (ext ? 1 : 0)) {        \
    case 0: M(__VA_ARGS__ false, false, false); break;              \
    case 1: M(__VA_ARGS__ false, false, true); break;               \
    case 2: M(__VA_ARGS__ false, true, false); break;               \
    case 3: M(__VA_ARGS__ false, true, true); break;                \
    case 4: M(__VA_ARGS__ true, false, false); break;               \
    case 5: M(__VA_ARGS__ true, false, true); break;                \
    case 6: M(__VA_ARGS__ true, true, false); break;                \
    default: M(__VA_ARGS__ true, true, true); break;                \
  }
#define RPA_STAGED_FP8(U, C, E) RPA_STAGED(true, U, C, E)
#define RPA_STAGED_BF16(U, C, E) RPA_STAGED(false, U, C, E)
  if (a.head_dim == 256) {
    if (a.fp8) return hipErrorInvalidValue;  // 256-wide fp8 rows go through the row kernel
    RPA_PICK(RPA_ASYNC256, )
  } else if (!staged) {
    RPA_PICK(RPA_ASYNC, )
  } else if (a.fp8) {
    RPA_PICK(RPA_STAGED_FP8, )
  } else {
    RPA_PICK(RPA_STAGED_BF16, )
  }
#undef RPA_STAGED_FP8
#undef RPA_STAGED_BF16
#undef RPA_PICK
#undef RPA_STAGED
#undef RPA_ASYNC
#undef RPA_ASYNC256
  return hipGetLastError();
}

}  // namespace rpa
