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

#include "rpa_prefill_common.h"

namespace rpa {

using namespace pf;

namespace {


// ---- fp8 rows into the same LDS layout (the 256-wide heads' fp8 path) ----
// Thread tid stages a quarter of K row and V row (tid >> 2): HD / 4 bytes of e4m3 each, loaded
// two tiles ahead into registers, widened to bf16 and written one tile ahead to the chunk
// positions the asynchronous copy would have used, so the products read both caches alike.
template <int HD>
struct Fp8Stage {
  u32x4_t k[HD / 64], v[HD / 64];
};

template <bool UNIFORM>
__device__ __forceinline__ int32_t fp8_fetch_page(const TileSrc& s, int tb, int tid) {
  tb = min(tb, s.last_tok & ~(kBN - 1));
  if constexpr (UNIFORM) {
    return scalar_load_i32(s.pages + __builtin_amdgcn_readfirstlane(page_slot(s, tb)));
  } else {
    return s.pages[page_slot(s, min(tb + (tid >> 2), s.last_tok))];
  }
}

template <bool UNIFORM, int HD>
__device__ __forceinline__ void fp8_gload(Fp8Stage<HD>& st, const TileSrc& s, const KvAddr& kv, const char* kh,
                                          const char* vh, int tb, int tid, int32_t page) {
  tb = min(tb, s.last_tok & ~(kBN - 1));  // past the end: re-read the last tile
  const int64_t ro = row_offset<UNIFORM>(s, kv, tb, tb + (tid >> 2), page) + (tid & 3) * (HD / 4);
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) {
    st.k[i] = ld16(kh + ro + i * 16);
    st.v[i] = ld16(vh + ro + i * 16);
  }
}

template <int HD>
__device__ __forceinline__ void fp8_lstore(const Fp8Stage<HD>& st, char* lds_k, char* lds_v, int tid) {
  const int t = tid >> 2;
  char* kr = lds_k + t * Tile<HD>::kRowB;
  char* vr = lds_v + t * Tile<HD>::kRowB;
  const int ks = t & 15, vs = (t & 3) << 2;
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) {
    const int j = (tid & 3) * (HD / 32) + 2 * i;  // the first of the two bf16 chunks these 16 bytes widen to
    {
      const u32x2_t a = fp8x4_to_bf16x4(st.k[i][0]), b = fp8x4_to_bf16x4(st.k[i][1]);
      const u32x2_t c = fp8x4_to_bf16x4(st.k[i][2]), d = fp8x4_to_bf16x4(st.k[i][3]);
      lds_st16(kr + ((j ^ ks) << 4), u32x4_t{a[0], a[1], b[0], b[1]});
      lds_st16(kr + (((j + 1) ^ ks) << 4), u32x4_t{c[0], c[1], d[0], d[1]});
    }
    {
      const u32x2_t a = fp8x4_to_bf16x4(st.v[i][0]), b = fp8x4_to_bf16x4(st.v[i][1]);
      const u32x2_t c = fp8x4_to_bf16x4(st.v[i][2]), d = fp8x4_to_bf16x4(st.v[i][3]);
      lds_st16(vr + ((j ^ vs) << 4), u32x4_t{a[0], a[1], b[0], b[1]});
      lds_st16(vr + (((j + 1) ^ vs) << 4), u32x4_t{c[0], c[1], d[0], d[1]});
    }
  }
}

// EXT compiles in the rarely used options (temperature factor, custom mask / no mask); the
// plain causal instantiation keeps its scale in a scalar register and its mask test to one compare.
// HD = 256 doubles the rows in LDS (two 64 KiB slots), the Q^T operands and the accumulators: one
// workgroup per CU, one wave per SIMD with up to 512 registers.
// FP8: an e4m3 cache staged through registers into the same LDS layout (see above).
// HEADS4: the short-chunk tile (chunks of at most 64 tokens: a verify step, a short prompt).  A workgroup owns 32
// query positions of FOUR query heads of a kv head, one head per wave, instead of 128 positions of one head:
// such chunks then fill their tiles, and the four waves still share every K/V tile.
template <bool UNIFORM, bool CAP, bool EXT, int HD = 128, bool FP8 = false, bool HEADS4 = false>
__global__ __launch_bounds__(256, (HD == 128 ? 2 : 1)) void rpa_prefill_async_kernel(const PrefillArgs a_in, int tiles, int nseq,
                                                                                  bool by_level) {
  PrefillArgs a = a_in;  // static-shape mode: the sequences to process come from the device
  if (a.dist) {
    a.seq_begin = (a.sm.mask_mode == 1) ? 0 : scalar_load_i32(a.dist);
    a.seq_end = min(a.seq_end, scalar_load_i32(a.dist + 2));
  }
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

  static_assert(!HEADS4 || (HD == 128 && !FP8), "the short-chunk tile exists for 128-wide heads on bf16 caches");
  constexpr int BM = HEADS4 ? 32 : kBM;  // query positions per workgroup
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

  WaveRows wr;
  wr.r_lo = w.q_start + (HEADS4 ? 0 : wave * 32);
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
      for (int ks = 0; ks < T::kSteps; ++ks) qB[ks] = requantise_q(qB[ks], a.sm.q_scale, FP8);
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

  const int wg_r_hi = min(w.q_start + BM, w.q_len) - 1;
  const bool causal = !EXT || a.sm.mask_mode == 0;
  MaskCtx mc;
  mc.mode = 0;
  if constexpr (EXT) mc = make_mask_ctx(a, w, wr.row);
  int t_hi = causal ? min(w.kv_len, w.prefix + wg_r_hi + 1) : w.kv_len;  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, w.prefix + w.q_start - W_ + 1) & ~(kBN - 1);
  int split = 0;
  if (a.kv_splits > 1 && !kv_piece(a, t_lo, t_hi, split)) {  // under-filled launch, nothing left for this piece
    write_empty_partial_rows<T::kDimTiles>(a, w, wr, h, split);
    return;
  }

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
  AsyncOffsets<HD> ofs;
  AsyncPages<UNIFORM, HD> pg;
  Fp8Stage<HD> stg;     // FP8: rows of the tile after the next one
  int32_t fp8_page = 0;  // FP8: page of this thread's row in the tile loaded next
  if constexpr (FP8) {
    fp8_page = fp8_fetch_page<UNIFORM>(src, t_lo, tid);
    fp8_gload<UNIFORM, HD>(stg, src, a.kv, kh, vh, t_lo, tid, fp8_page);
    fp8_page = fp8_fetch_page<UNIFORM>(src, t_lo + kBN, tid);
    fp8_lstore<HD>(stg, lds_k0, lds_v0, tid);
    fp8_gload<UNIFORM, HD>(stg, src, a.kv, kh, vh, t_lo + kBN, tid, fp8_page);
    fp8_page = fp8_fetch_page<UNIFORM>(src, t_lo + 2 * kBN, tid);
  } else {
    ofs = make_async_offsets<HD>(a.kv, wave, lane);
    async_fetch_pages<UNIFORM, HD>(pg, src, t_lo, wave, lane);
    async_copy_tile<UNIFORM, HD>(lds_k0, lds_v0, src, a.kv, kh, vh, t_lo, wave, lane, pg, ofs);
    async_fetch_pages<UNIFORM, HD>(pg, src, t_lo + kBN, wave, lane);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the copies have landed in LDS
  }
  __syncthreads();

  // one tile: consume (lds_k, lds_v), fill (nxt_k, nxt_v) with the tile after it
  auto tile_step = [&](const char* lds_k, const char* lds_v, char* nxt_k, char* nxt_v, int tb) {
    uint64_t mask_word = 0;  // a caller's mask turned into bits by the pre-pass: one word per lane and tile
    if constexpr (EXT && HD == 128) {
      if (mc.mode == 1 && mc.bits) mask_word = mc.bits[min(tb >> 6, mc.bit_words - 1)];
    }
    if (tb + kBN < t_hi) {
      // the other slot was last read before the barrier that ended the previous tile
      if constexpr (FP8) {
        fp8_lstore<HD>(stg, nxt_k, nxt_v, tid);
        fp8_gload<UNIFORM, HD>(stg, src, a.kv, kh, vh, tb + 2 * kBN, tid, fp8_page);
        fp8_page = fp8_fetch_page<UNIFORM>(src, tb + 3 * kBN, tid);
      } else {
        async_copy_tile<UNIFORM, HD>(nxt_k, nxt_v, src, a.kv, kh, vh, tb + kBN, wave, lane, pg, ofs);
        async_fetch_pages<UNIFORM, HD>(pg, src, tb + 2 * kBN, wave, lane);
      }
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
        softmax_tile<CAP, EXT, T::kDimTiles>(S, O, m, l, sm, need_mask, tb, h, wr.qpos, W_, pB, mc, mask_word);
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
    if constexpr (!FP8) __builtin_amdgcn_s_waitcnt(0x0F70);  // the next tile has landed
    __syncthreads();
  };
  for (int tb = t_lo; tb < t_hi; tb += 2 * kBN) {
    tile_step(lds_k0, lds_v0, lds_k1, lds_v1, tb);
    if (tb + kBN >= t_hi) break;
    tile_step(lds_k1, lds_v1, lds_k0, lds_v0, tb + kBN);
  }
  if (a.kv_splits > 1) write_partial_rows<T::kDimTiles>(a, w, wr, O, l, h, m * sm.sc2, split);
  else write_rows<T::kDimTiles>(a, w, wr, O, l, h, m * sm.sc2);
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

template <bool FP8, bool UNIFORM, bool CAP, bool EXT, bool HEADS4 = false>
__global__ __launch_bounds__(256, 2) void rpa_prefill_staged_kernel(const PrefillArgs a_in, int tiles, int nseq, bool by_level) {
  PrefillArgs a = a_in;  // static-shape mode: the sequences to process come from the device
  if (a.dist) {
    a.seq_begin = (a.sm.mask_mode == 1) ? 0 : scalar_load_i32(a.dist);
    a.seq_end = min(a.seq_end, scalar_load_i32(a.dist + 2));
  }
  __shared__ __attribute__((aligned(16))) char lds_k_buf[2][kBN * kKPitch];
  __shared__ __attribute__((aligned(16))) char lds_v_buf[2][128 * kVPitch];

  constexpr int BM = HEADS4 ? 32 : kBM;  // the short-chunk tile: 32 positions x 4 heads, one head per wave
  Work w = decompose(a, tiles, nseq, by_level, BM, HEADS4 ? 4 : 1);
  if (!w.valid) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  if constexpr (HEADS4) w.head += wave;
  const int c = lane & 31, h = lane >> 5;
  const TileSrc src = make_src(a, w);
  const char* kh = a.kv.k_base + (int64_t)w.hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)w.hk * a.kv.head_stride;

  WaveRows wr;
  wr.r_lo = w.q_start + (HEADS4 ? 0 : wave * 32);
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

  const int wg_r_hi = min(w.q_start + BM, w.q_len) - 1;
  const bool causal = !EXT || a.sm.mask_mode == 0;
  MaskCtx mc;
  mc.mode = 0;
  if constexpr (EXT) mc = make_mask_ctx(a, w, wr.row);
  int t_hi = causal ? min(w.kv_len, w.prefix + wg_r_hi + 1) : w.kv_len;  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, w.prefix + w.q_start - W_ + 1) & ~(kBN - 1);
  int split = 0;
  if (a.kv_splits > 1 && !kv_piece(a, t_lo, t_hi, split)) {  // under-filled launch, nothing left for this piece
    write_empty_partial_rows<4>(a, w, wr, h, split);
    return;
  }

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
    uint64_t mask_word = 0;  // a caller's mask turned into bits by the pre-pass: one word per lane and tile
    if constexpr (EXT) {
      if (mc.mode == 1 && mc.bits) mask_word = mc.bits[min(tb >> 6, mc.bit_words - 1)];
    }
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
      softmax_tile<CAP, EXT>(S, O, m, l, sm, need_mask, tb, h, wr.qpos, W_, pB, mc, mask_word);
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
  if (a.kv_splits > 1) write_partial_rows<4>(a, w, wr, O, l, h, m * sm.sc2, split);
  else write_rows(a, w, wr, O, l, h, m * sm.sc2);
}

}  // namespace

namespace {
// ---------------------------------------------------------------- custom masks as bits
// The caller's mask is one i32 per (query token, kv token).  Read where the scores are, a wave's 32 rows are 32
// separate 256-byte runs per tile -- four times the cache lines of the K/V tile itself, per query head.  This
// pre-pass reads it once, coalesced, and leaves one bit per pair (>= 1 keeps): bit t % 64 of word t / 64 of
// row `token`, mask_pitch words per row; tokens from kv_len on read as hidden.  grid = query tokens, 4 waves,
// wave w takes words w, w + 4, ...
__device__ __forceinline__ int mask_owner_of_token(const int32_t* cu_q_lens, int num_seqs, int tok) {
  int lo = 0, hi = num_seqs;  // last i with cu_q_lens[i] <= tok (zero-length sequences are skipped)
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_q_lens[mid] <= tok) lo = mid; else hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(256) void rpa_mask_bits_kernel(const PrefillArgs a) {
  // (masked calls run every sequence through the prefill kernels; with the composition on the device the number
  // of sequences is only a bound)
  const int seq_end = a.dist ? min(a.seq_end, a.dist[2]) : a.seq_end;
  const int token = a.pt.cu_q_lens[a.seq_begin] + (int)blockIdx.x;
  if (token >= a.pt.cu_q_lens[seq_end]) return;
  const int seq = mask_owner_of_token(a.pt.cu_q_lens, seq_end, token);
  const int kv_len = a.pt.kv_lens[seq];
  const int width = a.sm.mask_rows_page_aligned ? (a.pt.cu_kv_lens[seq + 1] - a.pt.cu_kv_lens[seq]) : kv_len;
  const int32_t* row = a.sm.custom_mask + a.sm.cu_mask_lens[seq] + (int64_t)(token - a.pt.cu_q_lens[seq]) * width;
  uint64_t* out = a.mask_bits + (int64_t)token * a.mask_pitch;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int words = min((kv_len + 63) >> 6, a.mask_pitch);
  for (int k = wave; k < words; k += 4) {
    const int t = 64 * k + lane;
    const int v = (t < kv_len) ? row[t] : 0;
    const uint64_t keep = __ballot(v >= 1);
    if (lane == 0) out[k] = keep;
  }
}

hipError_t launch_mask_bits(const PrefillArgs& a, hipStream_t stream) {
  if (!a.mask_bits || a.num_tokens <= 0) return hipSuccess;
  hipLaunchKernelGGL(rpa_mask_bits_kernel, dim3((unsigned)a.num_tokens), dim3(256), 0, stream, a);
  return hipGetLastError();
}

bool takes_pipe_kernel(const PrefillArgs& a) { return prefill_shape(a).kernel == kKernelPrefillPipe; }
}  // namespace

namespace {
// The compiled flash kernels' short-chunk tile: 32 positions x 4 heads per workgroup (rows "prefill_options_short"
// and "prefill_fp8_short" of the shape table).  RPA_PREFILL_STAGED=1 (bf16 rows through the register-staged
// kernel, a testing path) has no such tile.
bool compiled_short_chunk_tile(const PrefillArgs& a) {
  if (tuning().prefill_staged == 1 && !a.fp8) return false;
  const ShapeRule& r = prefill_shape(a);
  return r.kernel != kKernelPrefillPipe && r.tile_q == 32;
}
}  // namespace

const ShapeRule& prefill_shape_of(const PrefillArgs& a) {
  // RPA_PREFILL_STAGED=1 on a bf16 cache is a testing path outside the table: the fp8 kernel's rows
  return prefill_shape(a);
}

int prefill_kv_splits(const PrefillArgs& a) {
  const int nseq = a.seq_end - a.seq_begin;
  if (takes_pipe_kernel(a)) return prefill_pipe_kv_splits(a, nseq);
  // the compiled kernels: a tile takes about 1.1 us alone on its CU (2.2 us for 256-wide heads)
  const bool heads4 = compiled_short_chunk_tile(a);
  return kv_pieces(a, nseq, heads4 ? 32 : kBM, heads4 ? 4 : 1, a.head_dim == 256 ? 2.2 : 1.1);
}

size_t prefill_split_workspace_bytes(const PrefillArgs& a, int splits) {
  return splits > 1 ? (size_t)a.num_tokens * a.Hq * splits * (a.head_dim + 2) * sizeof(float) : 0;
}

hipError_t launch_prefill(const PrefillArgs& a, hipStream_t stream) {
  const int nseq = a.seq_end - a.seq_begin;
  if (nseq <= 0 || a.max_q_len <= 0) return hipSuccess;
  if (takes_pipe_kernel(a)) {
    return launch_prefill_pipe(a, nseq, tuning().prefill_level_order != 0, stream);
  }
  const bool heads4 = compiled_short_chunk_tile(a);
  const int bm = heads4 ? 32 : kBM;
  int tiles = (a.max_q_len + bm - 1) / bm;
  // levels 0 .. ceil(max_kv_len / rows): only worth their empty workgroups when prefixes are
  // not much longer than the chunks (else every tile of a sequence costs about the same anyway)
  const bool level_order = tuning().prefill_level_order != 0;
  const int levels = a.max_kv_len > 0 ? (a.max_kv_len + bm - 1) / bm + 1 : 0;
  const bool by_level = level_order && a.sm.mask_mode == 0 && levels > tiles && levels <= 2 * tiles + 2;
  if (by_level) tiles = levels;
  const int64_t units = (int64_t)nseq * a.Hkv;
  const int64_t grid = (units >= 8 ? ((units + 7) / 8) * 8 : units) * (heads4 ? a.G / 4 : a.G) * tiles;
  if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool uniform = (a.pt.page_size % kBN) == 0;
  // soft cap and logit rounding share the general score path
  const bool cap = a.sm.soft_cap != 0.f || a.sm.round_logits != 0;
  const bool staged = a.fp8 || tuning().prefill_staged == 1;
  if (a.sm.mask_mode == 1) {
    hipError_t e = launch_mask_bits(a, stream);
    if (e != hipSuccess) return e;
  }
  const bool cut = a.kv_splits > 1;  // pieces of the K/V ranges on the second grid dimension, then the merge
  if (cut && (!a.ws_o || !a.ws_ml || a.kv_splits > 64)) return hipErrorInvalidValue;
  const dim3 g((unsigned)grid, cut ? (unsigned)a.kv_splits : 1u), blk(256);
  const bool ext = a.sm.xai_len > 0.f || a.sm.mask_mode != 0 || a.sm.q_scale > 0.f;
#define RPA_STAGED(F, U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_staged_kernel<F, U, C, E>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_STAGED_FP8_HEADS4(U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_staged_kernel<true, U, C, E, true>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_ASYNC(U, C, E) hipLaunchKernelGGL((rpa_prefill_async_kernel<U, C, E>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_ASYNC_HEADS4(U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_async_kernel<U, C, E, 128, false, true>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_ASYNC256(U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_async_kernel<U, C, E, 256>), g, blk, 0, stream, a, tiles, nseq, by_level)
#define RPA_ASYNC256_FP8(U, C, E) \
  hipLaunchKernelGGL((rpa_prefill_async_kernel<U, C, E, 256, true>), g, blk, 0, stream, a, tiles, nseq, by_level)
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
    if (a.fp8) {
      RPA_PICK(RPA_ASYNC256_FP8, )
    } else {
      RPA_PICK(RPA_ASYNC256, )
    }
  } else if (heads4 && a.fp8) {
    RPA_PICK(RPA_STAGED_FP8_HEADS4, )
  } else if (heads4) {
    RPA_PICK(RPA_ASYNC_HEADS4, )
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
#undef RPA_ASYNC_HEADS4
#undef RPA_STAGED_FP8_HEADS4
#undef RPA_ASYNC256
#undef RPA_ASYNC256_FP8
  return cut ? launch_prefill_combine(a, stream) : hipGetLastError();
}

}  // namespace rpa
