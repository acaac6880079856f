// Absorbed-MLA split-KV decode on gfx950.
//
// Every token has ONE shared latent row [kv_c (512) | k_pe (64)]; all query
// heads attend to it (scores over 576 dims, values = the first 512 dims).  A
// workgroup of 8 waves owns one (sequence, kv split) and 128 heads (wave w owns
// heads 16w..16w+15), so each latent row is fetched from HBM exactly once:
//   global -> LDS   global_load_lds_dwordx4 copies 32-token tiles (rows of 72
//                   16-byte chunks, row-major) into a 4-slot ring,
//                   three tiles ahead of the MFMAs; no staging registers
//   S^T[tok, head] = K . Q^T       36 MFMA 16x16x32 per wave and tile, A = rows
//                                  read with ds_read_b128, B = Q^T in registers
//   online softmax, P rounded to bf16 (as the reference rounds it)
//   O^T[dim, head] += V^T . P^T    32 MFMA 16x16x32; A = V^T read from the SAME
//                                  row-major rows with ds_read_b64_tr_b16
// Partials (unnormalised O, running max, sum) go to the workspace and are merged
// by rpa_mla_combine_kernel; with a single split the output is written directly.
//
// LDS layout of a tile: row r (token) at r * 1184 bytes = 74 chunks of 16 bytes, the last two
// padding.  Measured on gfx950 (256 WGs of 8 waves reading one pattern): a ds_read_b128 whose 16
// lanes of a group read the same column of 16 rows runs at the full rate (3.7 clk per wave
// instruction, like 64 contiguous chunks) when the pitch is 74 or 78 chunks and at half of it
// (7.3 clk) for 73, 75, 76, 77, 79 and 81 chunks, whatever the order of the rows; the
// transposing b64 read of 4 consecutive rows x 32 bytes is full rate (2.6 clk) at 74 chunks
// too.  So no address swizzle and no row permutation: MFMA row m of a score tile is token
// 16b + m, and every LDS address is a per-lane base plus a compile-time offset.

#include <type_traits>

#include "rpa_common.h"
#include "rpa_kernels.h"
#include "rpa_shapes.h"
#include "rpa_tuning.h"
#include "rpa_mla_pipe_loop.inc"
#include "rpa_mla_wide_loop.inc"
#include "rpa_mla_wide32_loop.inc"

namespace rpa {

// Per-workgroup timestamps of the wide balanced kernel, compiled in with -DRPA_MLA_TRACE only (build.py passes
// extra flags through): for up to four pieces per workgroup the 100 MHz clock at piece entry, first tiles and
// queries landed, tile loop entered, tile loop left, rows written.  rpa_debug_mla_trace() copies them out.
#ifdef RPA_MLA_TRACE
__device__ unsigned long long rpa_mla_trace_buf[1024][4][8];
#define RPA_MLA_STAMP(slot)                                                                              \
  do {                                                                                                   \
    if (threadIdx.x == 0 && trace_piece < 4) rpa_mla_trace_buf[blockIdx.x & 1023][trace_piece][slot] = wall_clock64(); \
  } while (0)
#else
#define RPA_MLA_STAMP(slot) do { } while (0)
#endif

namespace {

constexpr int kTok = 32;                 // tokens per tile
constexpr int kRowB = 1184;              // latent row in LDS: 576 bf16 + 32 bytes of padding
constexpr int kChunks = 74;              // 16-byte chunks per row (72 data + 2 pad)
constexpr int kUsedBlocks = 37;          // copy blocks of 64 chunks that hold a tile (32 rows x 74 chunks)
constexpr int kSlotB = kUsedBlocks * 1024;  // one ring slot
constexpr int kCopiesPerWave = 5;        // every wave issues 5 copy instructions per tile
// fp8 caches: a tile arrives as bytes in a staging area (rows of 576 bytes, no padding: 18 copy
// blocks) and is expanded to the bf16 layout above by all waves together
constexpr int kF8Chunks = 36;            // 16-byte chunks per staged row
constexpr int kF8Blocks = 18;            // copy blocks per staged tile (32 rows x 36 chunks)
constexpr int kF8StageB = kF8Blocks * 1024;
constexpr int kF8CopiesPerWave = 3;      // 8 x 3 = 24 copy instructions cover 18 blocks (the rest repeat block 0)

__device__ __forceinline__ u32x4_t lds_ld16(const char* p) { return *reinterpret_cast<const u32x4_t*>(p); }

typedef uint32_t u32x32_t __attribute__((ext_vector_type(32)));
typedef uint32_t u32x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x32_t __attribute__((ext_vector_type(32)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2_t lds_tr16(const char* p) {
  typedef __attribute__((address_space(3))) s16x4_t* lds_ptr_t;
  const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
  return __builtin_bit_cast(u32x2_t, v);
}

// The lane id behind a fence the compiler cannot see through: values derived from it are not common
// subexpressions of anything earlier, so they are worked out again where they are used instead of being
// kept in registers across code that has none to spare (the assembly loop pins 251 of a wave's 256; with
// them carried over it, 23-37 registers went to scratch memory per segment, 100 MB a launch on a
// prefill batch).  Taken from threadIdx: the same helper on v_mbcnt made the allocator spill 140.
__device__ __forceinline__ int fresh_lane() {
  int ln = (int)(threadIdx.x & 63);
  asm volatile("" : "+v"(ln));
  return ln;
}

// token (inside a tile) behind slot i = 4b + r of lane group g in the S^T result registers
__device__ __forceinline__ int tok_of(int g, int i) {
  return 16 * (i >> 2) + 4 * g + (i & 3);
}

struct Src {
  const int32_t* pages;
  // pages smaller than a tile: the wave's LDS window of this row's page ids (entry 0 = page slot win_first),
  // which the lanes look their rows' pages up in; fetched from memory per tile they would be a load the next
  // tile's copies depend on, behind which the copies in flight drain
  const int32_t* win;
  int32_t win_first;
  int32_t page_size, page_shift, last_tok;
  int64_t page_stride;  // bytes
  int32_t row_bytes;    // bytes between tokens of a page
  int32_t rope_byte;    // byte offset of k_pe inside a cached row
};

__device__ __forceinline__ int page_slot(const Src& s, int tok) {
  return s.page_shift >= 0 ? (tok >> s.page_shift) : (tok / s.page_size);
}

// A lane's 5 chunks of a tile: position p = 64*(5*wave + n) + lane; row p / 74, chunk
// column p % 74.  The pad columns copy the tile's first chunk.
// The 8 x 5 = 40 copy instructions of a tile cover 37 blocks: the last three repeat block 0
// (same source, same destination, same bytes), so every wave has the same number of copies
// in flight and the slot is exactly 37 KiB.
// CPW: copy instructions per wave and tile -- 5 with eight waves, 10 with four (wide workgroups).
template <int CPW = kCopiesPerWave>
__device__ __forceinline__ int copy_block(int wave, int n) {
  const int blk = wave * CPW + n;
  if constexpr (CPW == kCopiesPerWave) return blk < kUsedBlocks ? blk : 0;
  // wide workgroups: copy n < 9 of wave w is block w + 4 n (the assembly loop then adds a constant to one base
  // per copy), and every wave's last copy is the 37th block (the same bytes four times)
  else return n < CPW - 1 ? wave + 4 * n : kUsedBlocks - 1;
}

template <int CPW = kCopiesPerWave>
__device__ __forceinline__ void chunk_of(const Src& s, int wave, int lane, int n, int& row, int& inner) {
  const int p = copy_block<CPW>(wave, n) * 64 + lane;
  row = p / kChunks;
  int j = p - row * kChunks;
  if (j >= 72) { row = 0; j = 0; }
  inner = j < 64 ? j * 16 : s.rope_byte + (j - 64) * 16;
}

template <bool UNIFORM, int CPW = kCopiesPerWave>
__device__ __forceinline__ void copy_tile(char* slot, const Src& s, const char* cache, int tb, int wave, int lane,
                                          int page) {
  tb = min(tb, s.last_tok & ~(kTok - 1));  // past the end: re-copy the last tile
  if constexpr (UNIFORM) {
    if (tb + kTok - 1 <= s.last_tok) {
      const char* base = cache + (int64_t)page * s.page_stride +
                         (int64_t)(tb - page_slot(s, tb) * s.page_size) * s.row_bytes;  // scalar
      // chunk offsets are recomputed per tile (a dozen integer ops) rather than kept in
      // registers: the accumulators and Q^T leave no room, and a spill reload would be a
      // vector-memory load that drains the copy queue
      int ln = lane;
      asm volatile("" : "+v"(ln));  // opaque: keeps the offset arithmetic inside the loop
#pragma unroll
      for (int n = 0; n < CPW; ++n) {
        int row, inner;
        chunk_of<CPW>(s, wave, ln, n, row, inner);
        async_copy16(base + (uint32_t)(row * s.row_bytes + inner), slot + copy_block<CPW>(wave, n) * 1024);
      }
      return;
    }
  }
  // last, partial tile (rows clamped to the last valid token) or pages smaller than a tile
#pragma unroll
  for (int n = 0; n < CPW; ++n) {
    int row, inner;
    chunk_of<CPW>(s, wave, lane, n, row, inner);
    const int tok = min(tb + row, s.last_tok);
    const int ps = page_slot(s, tok);
    const int pg = UNIFORM ? page : s.win[ps - s.win_first];
    const char* src = cache + (int64_t)pg * s.page_stride + (int64_t)(tok - ps * s.page_size) * s.row_bytes + inner;
    async_copy16(src, slot + copy_block<CPW>(wave, n) * 1024);
  }
}

// fp8 caches: the same copy, of a tile of bytes into a staging area.  Position p = 64 * block + lane
// is chunk p % 36 of row p / 36; chunks 0..31 are kv_c, 32..35 k_pe.
__device__ __forceinline__ int f8_copy_block(int wave, int n) {
  const int blk = wave * kF8CopiesPerWave + n;
  return blk < kF8Blocks ? blk : 0;
}

// row and byte offset inside a cached row of the chunk that lane `lane` moves with copy n of wave `wave`
__device__ __forceinline__ void f8_chunk_of(const Src& s, int wave, int lane, int n, int& row, int& inner) {
  const int p = f8_copy_block(wave, n) * 64 + lane;
  row = p / kF8Chunks;
  const int j = p - row * kF8Chunks;
  inner = j < 32 ? j * 16 : s.rope_byte + (j - 32) * 16;
}

template <bool UNIFORM>
__device__ __forceinline__ void copy_tile_f8(char* stage, const Src& s, const char* cache, int tb, int wave, int lane,
                                             int page) {
  tb = min(tb, s.last_tok & ~(kTok - 1));
  const bool whole = UNIFORM && (tb + kTok - 1 <= s.last_tok);
  const char* base = cache + (int64_t)page * s.page_stride + (int64_t)(tb - page_slot(s, tb) * s.page_size) * s.row_bytes;
  int ln = lane;
  asm volatile("" : "+v"(ln));
#pragma unroll
  for (int n = 0; n < kF8CopiesPerWave; ++n) {
    const int blk = f8_copy_block(wave, n);
    int row, inner;
    f8_chunk_of(s, wave, ln, n, row, inner);
    if (whole) {
      async_copy16(base + (uint32_t)(row * s.row_bytes + inner), stage + blk * 1024);
    } else {  // last, partial tile (rows clamped to the last valid token) or pages smaller than a tile
      const int tok = min(tb + row, s.last_tok);
      const int ps = page_slot(s, tok);
      const int pg = UNIFORM ? page : s.win[ps - s.win_first];
      async_copy16(cache + (int64_t)pg * s.page_stride + (int64_t)(tok - ps * s.page_size) * s.row_bytes + inner,
                   stage + blk * 1024);
    }
  }
}

// e4m3 bytes of a staged tile -> bf16 rows of a ring slot (exact).  512 threads, 1152 chunks of 16
// elements: three rounds, the last one a quarter full.
__device__ __forceinline__ void expand_f8_tile(const char* stage, char* slot, int tid) {
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int p = tid + 512 * i;
    if (p < kTok * kF8Chunks) {
      const int row = p / kF8Chunks;
      const int j = p - row * kF8Chunks;
      const u32x4_t w = lds_ld16(stage + p * 16);
      u32x4_t lo, hi;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        lo[2 * d] = fp8x2_to_bf16x2(w[d], false);
        lo[2 * d + 1] = fp8x2_to_bf16x2(w[d], true);
        hi[2 * d] = fp8x2_to_bf16x2(w[2 + d], false);
        hi[2 * d + 1] = fp8x2_to_bf16x2(w[2 + d], true);
      }
      char* dst = slot + row * kRowB + j * 32;
      *reinterpret_cast<u32x4_t*>(dst) = lo;
      *reinterpret_cast<u32x4_t*>(dst + 16) = hi;
    }
  }
}

// Sequence that owns query token `row`: the last one whose first token is <= row
// (zero-length sequences are skipped).  cu_q_lens[0 .. num_seqs] is non-decreasing.
__device__ __forceinline__ int owner_of_token(const int32_t* cu_q_lens, int num_seqs, int row) {
  int lo = 0, hi = num_seqs;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (scalar_load_i32(cu_q_lens + mid) <= row) lo = mid;
    else hi = mid;
  }
  return lo;
}

// What a grid row attends to.  Sequence rows (decode batches): the one query of sequence `row`
// sees all kv_len tokens.  Token rows: query token `row` of a sequence with q_len new tokens
// sits at position kv_len - q_len + j and sees the tokens up to itself -- an absorbed-MLA
// prefill row is a decode row over a shorter prefix (mla/v1/ref.py:229-233).
struct MlaRow {
  int seq, kv_len, tq;
  bool valid;
};

__device__ __forceinline__ MlaRow mla_row(const MlaDecodeArgs& a, int row) {
  MlaRow r;
  r.valid = true;
  // static-shape mode: num_seqs is a bound, the number of sequences comes from the device
  const int num_seqs = a.dist ? min(a.num_seqs, scalar_load_i32(a.dist + 2)) : a.num_seqs;
  if (a.rows_are_tokens) {
    if (row >= scalar_load_i32(a.pt.cu_q_lens + num_seqs)) {
      r.valid = false;
      r.seq = r.kv_len = r.tq = 0;
      return r;
    }
    r.seq = owner_of_token(a.pt.cu_q_lens, num_seqs, row);
    const int q0 = scalar_load_i32(a.pt.cu_q_lens + r.seq);
    const int q_len = scalar_load_i32(a.pt.cu_q_lens + r.seq + 1) - q0;
    r.kv_len = scalar_load_i32(a.pt.kv_lens + r.seq) - q_len + (row - q0) + 1;
    r.tq = row;
  } else {
    r.seq = row;
    r.kv_len = (row < num_seqs) ? a.pt.kv_lens[row] : 0;
    r.tq = a.pt.cu_q_lens[row];
    r.valid = row < num_seqs;
  }
  return r;
}

// Where a workgroup leaves the result of one piece of work: finished bf16 rows in `out`, or
// unnormalised partial rows plus (max, sum) in workspace slot `base` + head.
struct MlaDest {
  bool final_rows;
  int64_t base;
};

// One workgroup, one row, one group of 128 heads, tokens [t_begin, t_end).  Every wave of the
// workgroup calls it with the same arguments; all LDS reads of an earlier call are behind a
// barrier when it returns.
// PIPE: the tiles of the segment that are whole and unmasked, all but the first, run inside the
// assembly loop of rpa_mla_pipe_loop.inc (same LDS ring, same copy protocol, same registers as the
// compiled step, which still does the first tile, masked tiles and the last three before a
// partial one).  Needs UNIFORM pages of a power-of-two size, no soft cap, every wave at work.
// FP8: the cache holds e4m3 bytes.  Slots 0 and 1 are the bf16 ring, slot 2 (two halves) and slot 3 three
// staging areas; a step copies the bytes of tile k + 3, multiplies tile k, and ends by expanding tile
// k + 1 between two barriers.
// DS: with at most 64 heads (a tensor-parallel share) most waves of the workgroup would have no heads, and a step
// would last as long as one wave's serial chain through the tile (36 + 32 dependent matrix instructions with
// their LDS reads) while the others only copy.  With DS = 8 / 4 / 2 (at most 16 / 32 / 64 heads) the DS waves of a
// block of 16 heads share its tile instead: wave `sub` of the block takes token half sub & 1 and k-step group
// sub >> 1 of the first product, leaves its partial scores in LDS, every wave of the block sums them and takes
// the (same) probabilities, and the second product's 32 output chunks are dealt out 32 / DS per wave.
// TG (token group): with 16 / 32 / 64 heads, the eight waves hold 8 / 4 / 2 CONSECUTIVE QUERY TOKENS of one
// sequence instead of one token's heads, `group_tokens` of them real (a chunk's tail may leave fewer): wave w
// owns token (16 w) / Hq of the group and the block of 16 heads (16 w) % Hq.  mr.tq is the group's first token,
// mr.kv_len what its LAST token sees; a wave's own token sees kv_len - (group_tokens - 1) + its place, and
// masks with that.  Tokens of one sequence follow each other in q and out, so (token, head) of the group is
// "head" 16 w + c of a 128-head row at mr.tq: every address below stays what it was.  The reference's
// kernel shares each latent tile among 16 query tokens the same way (kernels/mla/v2/kernel.py:1448-1459).
template <bool UNIFORM, bool CAP, bool PIPE = false, bool FP8 = false, int DS = 1, bool TG = false>
__device__ __forceinline__ void mla_segment(const MlaDecodeArgs& a, const MlaRow mr, int head_base, int t_lo,
                                            int t_begin, int t_end, const MlaDest dest, char* slot0, char* slot1,
                                            char* slot2, char* slot3, int group_tokens = 1) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;
  static_assert(DS == 1 || (UNIFORM && !PIPE), "shared tiles: compiled loop, whole tiles per page (LDS for the partial scores)");
  static_assert(!TG || DS == 1, "token groups: one wave per (token, block of 16 heads)");
  const int sub = wave % DS;                       // this wave's place among the DS waves of its block of heads
  // token groups: a wave past the group's last real token repeats that token's work and writes nothing
  const int tg_place = TG ? min((wave * 16) / a.Hq, group_tokens - 1) : 0;
  const bool tg_real = !TG || (wave * 16) / a.Hq < group_tokens;
  const int head0 = TG ? tg_place * a.Hq + (wave * 16) % a.Hq : head_base + (wave / DS) * 16;
  const bool wave_on = TG || head0 < a.Hq;
  // what this wave's token sees (all waves alike unless TG)
  const int kv_len_w = TG ? mr.kv_len - (group_tokens - 1) + tg_place : mr.kv_len;
  const int t_lo_w = (TG && a.sm.window > 0) ? max(0, kv_len_w - a.sm.window) : t_lo;
  const int t_lo_last = (TG && a.sm.window > 0) ? max(0, mr.kv_len - a.sm.window) : t_lo;  // the largest of the group
  constexpr int kChunksPerWave = 32 / DS;          // output chunks of 16 dims per wave
  __shared__ __attribute__((aligned(16))) float partial_scores[DS == 1 ? 1 : 8][DS == 1 ? 4 : 256];  // [wave][lane x 4]
  const int seq = mr.seq;
  const int kv_len = mr.kv_len;

  Src src;
  src.page_size = a.pt.page_size;
  src.page_shift = ((src.page_size & (src.page_size - 1)) == 0) ? (31 - __builtin_clz(src.page_size)) : -1;
  src.last_tok = kv_len - 1;
  src.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / a.pt.page_size)
                                                  : (int64_t)seq * a.pt.pages_per_seq);
  src.row_bytes = a.row_stride * (FP8 ? 1 : 2);
  src.page_stride = (int64_t)src.row_bytes * a.pt.page_size;
  src.rope_byte = a.rope_offset * (FP8 ? 1 : 2);
  src.win = nullptr;
  src.win_first = 0;
  __shared__ int32_t page_windows[UNIFORM ? 1 : 8][UNIFORM ? 1 : kWinSmallPages];  // [wave][entry]
  auto cover = [&](int tb) __attribute__((always_inline)) {  // make the wave's window hold the pages of tile tb
    if constexpr (!UNIFORM) {
      tb = min(tb, src.last_tok & ~(kTok - 1));
      if (!src.win || page_slot(src, min(tb + kTok - 1, src.last_tok)) - src.win_first >= kWinSmallPages) {
        src.win_first = __builtin_amdgcn_readfirstlane(page_slot(src, tb));
        copy_page_window<kWinSmallPages>(src.pages, page_slot(src, src.last_tok), page_windows[wave], src.win_first, lane);
        wait_all_loads();
        src.win = page_windows[wave];
      }
    }
  };
  auto page_of = [&](int tb) -> int {
    if constexpr (UNIFORM) {
      tb = min(tb, src.last_tok & ~(kTok - 1));
      return scalar_load_i32(src.pages + __builtin_amdgcn_readfirstlane(page_slot(src, tb)));
    } else {
      return 0;
    }
  };

  // ---- Q^T operands of this wave: column c = head head0 + c, k-step ks covers dims 32ks + 8g .. ----
  const int tq = mr.tq;
  u32x4_t qB[18];
  {
    const int head = TG ? head0 + c : min(head0 + c, a.Hq - 1);
    const uint16_t* qn = a.ql_nope + ((int64_t)tq * a.Hq + head) * 512 + g * 8;
    const uint16_t* qr = a.q_pe + ((int64_t)tq * a.Hq + head) * 64 + g * 8;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) qB[ks] = ld16(qn + ks * 32);
    qB[16] = ld16(qr);
    qB[17] = ld16(qr + 32);
  }

  const float scale = a.sm.sm_scale;
  const float scale2 = scale * kLog2e;
  const float cap = a.sm.soft_cap;
  const float inv_cap = (cap != 0.f) ? 1.0f / cap : 0.f;
  const float mask2 = fmaxf(a.sm.mask_value * kLog2e, -3.0e38f);

  // ---- LDS operand addresses (bytes inside a slot) ----
  // K operand of score tile b, k-step ks: row 16b + c, bytes 64ks + 16g
  const int k_off = c * kRowB + g * 16;
  // V^T operand of dim chunk j: source lane r = c points at token 4g + (r >> 2)
  // (+16 for the second half of the k-step), dims 16j + 4(r & 3)
  const int v_off = (4 * g + (c >> 2)) * kRowB + (c & 3) * 8;

  f32x4_t acc[32];
#pragma unroll
  for (int j = 0; j < 32; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // ---- pipeline: copies run three tiles ahead of the MFMAs (4-slot ring, 148 of the CU's 160 KiB:
  // 111 KiB per CU in flight, which is what HBM latency under load asks for) ----
  int pg_next = page_of(t_begin + 3 * kTok);
  auto stage_of = [&](int i) -> char* { return i == 0 ? slot2 : (i == 1 ? slot2 + kF8StageB : slot3); };
  cover(t_begin);  // (the first three tiles never span a window's 256 pages)
  if constexpr (FP8) {
    copy_tile_f8<UNIFORM>(stage_of(0), src, a.cache, t_begin, wave, lane, page_of(t_begin));
    copy_tile_f8<UNIFORM>(stage_of(1), src, a.cache, t_begin + kTok, wave, lane, page_of(t_begin + kTok));
    copy_tile_f8<UNIFORM>(stage_of(2), src, a.cache, t_begin + 2 * kTok, wave, lane, page_of(t_begin + 2 * kTok));
  } else {
    copy_tile<UNIFORM>(slot0, src, a.cache, t_begin, wave, lane, page_of(t_begin));
    copy_tile<UNIFORM>(slot1, src, a.cache, t_begin + kTok, wave, lane, page_of(t_begin + kTok));
    copy_tile<UNIFORM>(slot2, src, a.cache, t_begin + 2 * kTok, wave, lane, page_of(t_begin + 2 * kTok));
  }
  // Touch every Q^T register here: the compiler then waits for the Q loads now, instead of
  // re-checking them with s_waitcnt vmcnt(0..4) inside the loop, where such a wait would also
  // drain the copy queue.
#pragma unroll
  for (int ks = 0; ks < 18; ++ks) asm volatile("" ::"v"(qB[ks]));
  // wait for the first tile (all but the 10 newest copies), then meet
  constexpr int kAhead = 2 * (FP8 ? kF8CopiesPerWave : kCopiesPerWave);  // copies of the two tiles behind the next one
  __builtin_amdgcn_s_waitcnt(0x0F70 | kAhead);
  __syncthreads();
  auto bare_barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // expand the staged tile `from` into ring slot `to`: every wave's bytes have landed (wait + barrier
  // before), every wave's LDS writes are done before the barrier behind it
  auto expand = [&](const char* from, char* to) {
    expand_f8_tile(from, to, PIPE ? wave * 64 + fresh_lane() : tid);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0) only: the copies in flight stay in flight
    bare_barrier();
  };
  if constexpr (FP8) expand(stage_of(0), slot0);

  auto tile_step = [&](const char* cur, char* fill, int tb, const char* next_stage = nullptr, char* next_slot = nullptr) {
    // with the assembly loop in the same function every lane-dependent value is worked out here, per
    // step, rather than carried over that loop
    const int lane_t = PIPE ? fresh_lane() : lane;
    const int c_t = PIPE ? (lane_t & 15) : c, g_t = PIPE ? (lane_t >> 4) : g;
    const int k_off_t = PIPE ? (c_t * kRowB + g_t * 16) : k_off;
    const int v_off_t = PIPE ? ((4 * g_t + (c_t >> 2)) * kRowB + (c_t & 3) * 8) : v_off;
    // `fill` held tile tb - 32, which every wave finished before the last barrier
    cover(tb + 3 * kTok);
    if constexpr (FP8) copy_tile_f8<UNIFORM>(fill, src, a.cache, tb + 3 * kTok, wave, lane_t, pg_next);
    else copy_tile<UNIFORM>(fill, src, a.cache, tb + 3 * kTok, wave, lane_t, pg_next);
    pg_next = page_of(tb + 4 * kTok);
    if constexpr (DS > 1) {
      // this wave's share of the first product: one token half, one group of k-steps
      f32x4_t sp = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (wave_on) {
        const char* kp = cur + k_off_t + (sub & 1) * 16 * kRowB;
        constexpr int kGroups = DS / 2;  // 4 groups of 5, 5, 4, 4 k-steps; 2 of 9; 1 of 18
        auto chain = [&](auto lo, auto hi) __attribute__((always_inline)) {
#pragma unroll
          for (int ks = decltype(lo)::value; ks < decltype(hi)::value; ++ks) sp = mfma16(lds_ld16(kp + ks * 64), qB[ks], sp);
        };
        using std::integral_constant;
        const int kg = sub >> 1;
        if constexpr (kGroups == 4) {
          if (kg == 0) chain(integral_constant<int, 0>{}, integral_constant<int, 5>{});
          else if (kg == 1) chain(integral_constant<int, 5>{}, integral_constant<int, 10>{});
          else if (kg == 2) chain(integral_constant<int, 10>{}, integral_constant<int, 14>{});
          else chain(integral_constant<int, 14>{}, integral_constant<int, 18>{});
        } else if constexpr (kGroups == 2) {
          if (kg == 0) chain(integral_constant<int, 0>{}, integral_constant<int, 9>{});
          else chain(integral_constant<int, 9>{}, integral_constant<int, 18>{});
        } else {
          chain(integral_constant<int, 0>{}, integral_constant<int, 18>{});
        }
      }
      *reinterpret_cast<f32x4_t*>(&partial_scores[wave][lane_t * 4]) = sp;
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the partial scores are written
      bare_barrier();
    }
    if (wave_on) {
      // two independent accumulator chains (token halves), issued alternately
      f32x4_t s[2];
      s[0] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      s[1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if constexpr (DS > 1) {
        // the block's scores: the partial sums of its DS waves (wave sub' holds half sub' & 1, group sub' >> 1)
        const int w0 = (wave / DS) * DS;
#pragma unroll
        for (int u = 0; u < DS; ++u) {
          const f32x4_t part = *reinterpret_cast<const f32x4_t*>(&partial_scores[w0 + u][lane_t * 4]);
          s[u & 1] += part;
        }
      } else {
      const char* kp = cur + k_off_t;
#pragma unroll
      for (int ks = 0; ks < 18; ++ks) {
        s[0] = mfma16(lds_ld16(kp + ks * 64), qB[ks], s[0]);
        s[1] = mfma16(lds_ld16(kp + 16 * kRowB + ks * 64), qB[ks], s[1]);
        // fence the scheduler every few MFMAs: it would otherwise hoist all LDS reads of the
        // tile, run out of registers and spill (a spill reload drains the copy queue)
        if (ks % 3 == 2) __builtin_amdgcn_sched_barrier(0);
      }
      }
      float x[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float v = s[i >> 2][i & 3];
        if constexpr (CAP) v = soft_cap_f(v * scale, cap, inv_cap) * kLog2e;
        else v = v * scale2;
        x[i] = v;
      }
      if ((tb + kTok > kv_len_w) || (tb < t_lo_w)) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int tok = tb + tok_of(g_t, i);
          if (tok >= kv_len_w || tok < t_lo_w) x[i] = mask2;
        }
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
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int j = 0; j < kChunksPerWave; ++j) acc[j] = acc[j] * alpha;
      }
      // (shared tiles: this wave's chunks are sub * kChunksPerWave .. of the 32)
      const char* vp = cur + v_off_t + (DS > 1 ? sub * kChunksPerWave * 32 : 0);
#pragma unroll
      for (int j = 0; j < kChunksPerWave; ++j) {
        const char* vt = vp + j * 32;
        const u32x2_t lo = lds_tr16(vt);
        const u32x2_t hi = lds_tr16(vt + 16 * kRowB);
        acc[j] = mfma16(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, pB, acc[j]);
        if (j % 2 == 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
    // Tile tb + 32 has landed once at most the 10 copies of tiles tb + 64 and tb + 96 are outstanding.  A bare
    // s_barrier is used instead of __syncthreads(): the fence in the latter makes the compiler
    // wait for ALL outstanding copies, which would shorten the prefetch distance to one tile.
    // Every LDS read of this tile has returned (its MFMA consumed it) before the barrier, and
    // each wave has waited for its own share of the next tile, so no fence is needed.
    __builtin_amdgcn_s_waitcnt(0x0F70 | kAhead);
    bare_barrier();
    if constexpr (FP8) expand(next_stage, next_slot);  // tile tb + 32 becomes bf16 rows
  };
  // compiled step for tile k of the segment, whichever ring it uses
  auto step_at = [&](int k) {
    const int tb = t_begin + k * kTok;
    if constexpr (FP8) {
      const int k3 = k % 3;
      tile_step((k & 1) ? slot1 : slot0, stage_of(k3), tb, stage_of(k3 == 2 ? 0 : k3 + 1), (k & 1) ? slot0 : slot1);
    } else {
      const int c4 = k & 3, f4 = (k + 3) & 3;
      tile_step(c4 == 0 ? slot0 : (c4 == 1 ? slot1 : (c4 == 2 ? slot2 : slot3)),
                f4 == 0 ? slot0 : (f4 == 1 ? slot1 : (f4 == 2 ? slot2 : slot3)), tb);
    }
  };
  if constexpr (FP8 && !PIPE) {
    const int nT = (t_end - t_begin + kTok - 1) / kTok;
    for (int k = 0; k < nT; ++k) step_at(k);
  } else if constexpr (!PIPE) {
    for (int tb = t_begin; tb < t_end; tb += 4 * kTok) {
      tile_step(slot0, slot3, tb);
      if (tb + kTok >= t_end) break;
      tile_step(slot1, slot0, tb + kTok);
      if (tb + 2 * kTok >= t_end) break;
      tile_step(slot2, slot1, tb + 2 * kTok);
      if (tb + 3 * kTok >= t_end) break;
      tile_step(slot3, slot2, tb + 3 * kTok);
    }
  } else {
    const int nT = (t_end - t_begin + kTok - 1) / kTok;  // tiles of the segment
    // tiles [k0, k1) go through the assembly loop: past the first tile (which fixes the reference the
    // probabilities are taken against) and past the window's edge; the loop copies tile k + 3 without
    // clamping rows, so that one has to be a whole tile of the row
    int k0 = 1;
    // (every wave must have met a token it sees, and with it a real reference, before the loop: with token
    // groups the last token's window may open a tile later than the first one's)
    if (t_begin < t_lo_last) k0 = max(k0, TG ? (t_lo_last - t_begin) / kTok + 1 : (t_lo_last - t_begin + kTok - 1) / kTok);
    const int k1 = min(nT, (kv_len - t_begin) / kTok - 3);
    typedef __attribute__((address_space(3))) char* lds_ptr_t;
    int k = 0;
    for (int phase = 0; phase < 2; ++phase) {
      const int stop = (phase == 0 && k0 < k1) ? k0 : nT;
      for (; k < stop; ++k) step_at(k);
      if (k >= nT) break;
      // ---- tiles k .. k1 - 1 in assembly
      f32x16_t o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[i][e] = acc[4 * i + (e >> 2)][e & 3];
      u32x32_t q0, q1;
      u32x8_t q2;
#pragma unroll
      for (int e = 0; e < 32; ++e) {
        q0[e] = qB[e >> 2][e & 3];
        q1[e] = qB[8 + (e >> 2)][e & 3];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) q2[e] = qB[16 + (e >> 2)][e & 3];
      const int ln = fresh_lane();  // the lane parts below are worked out here, not carried from the top
      const int cc = ln & 15, gg = ln >> 4;
      u32x4_t ml = {__float_as_uint(m), __float_as_uint(l), (uint32_t)(cc * kRowB + gg * 16),
                    (uint32_t)((4 * gg + (cc >> 2)) * kRowB + (cc & 3) * 8)};
      u32x8_t ofs = {0, 0, 0, 0, 0, 0, 0, 0};
      if constexpr (FP8) {
#pragma unroll
        for (int n = 0; n < kF8CopiesPerWave; ++n) {
          int row, inner;
          f8_chunk_of(src, wave, ln, n, row, inner);
          ofs[n] = (uint32_t)(row * src.row_bytes + inner);
        }
        // what the expansion needs of this thread: where its chunks start in a staging area, where they go
        const int td = wave * 64 + ln;
        ofs[3] = (uint32_t)(td * 16);
#pragma unroll
        for (int i = 0; i < 3; ++i) {
          const int p = td + 512 * i;
          const int row = p / kF8Chunks;
          ofs[4 + i] = (uint32_t)(row * kRowB + (p - row * kF8Chunks) * 32);
        }
      } else {
#pragma unroll
        for (int n = 0; n < kCopiesPerWave; ++n) {
          int row, inner;
          chunk_of(src, wave, ln, n, row, inner);
          ofs[n] = (uint32_t)(row * src.row_bytes + inner);
        }
      }
      const uint32_t s0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)slot0);
      const uint32_t s1 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)slot1);
      const uint32_t s2 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)slot2);
      const uint32_t s3 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)slot3);
      const uint32_t cache_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)a.cache);
      const uint32_t cache_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)a.cache >> 32));
      const int last_tile_tok = __builtin_amdgcn_readfirstlane(src.last_tok & ~(kTok - 1));
      const uint32_t scale2_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(scale2));
#define C(n) RPA_MLA_PIPE_C_##n
      if constexpr (FP8) {
        const int wave_blk = wave * kF8CopiesPerWave * 1024;
        asm volatile(RPA_MLA_PIPE_F8_ASM
                     : "+" C(O0)(o[0]), "+" C(O1)(o[1]), "+" C(O2)(o[2]), "+" C(O3)(o[3]), "+" C(O4)(o[4]),
                       "+" C(O5)(o[5]), "+" C(O6)(o[6]), "+" C(O7)(o[7]), "+" C(ML)(ml), "+" C(OFS)(ofs),
                       [t] "+&s"(k), [pg] "+&s"(pg_next)
                     : C(Q0)(q0), C(Q1)(q1), C(Q2)(q2), [t_end] "s"(k1), [t_begin] "s"(t_begin),
                       [last_tile_tok] "s"(last_tile_tok), [row_bytes] "s"(src.row_bytes), [pshift] "s"(src.page_shift),
                       [cache_lo] "s"(cache_lo), [cache_hi] "s"(cache_hi), [pages] "s"(src.pages), [scale2] "s"(scale2_bits),
                       [wave_blk] "s"(wave_blk), [slot0] "s"(s0), [slot1] "s"(s1), [stage0] "s"(s2),
                       [stage1] "s"(s2 + (uint32_t)kF8StageB), [stage2] "s"(s3)
                     : RPA_MLA_PIPE_F8_CLOBBERS);
      } else {
        const int wave_blk = wave * kCopiesPerWave * 1024;
        asm volatile(RPA_MLA_PIPE_ASM
                     : "+" C(O0)(o[0]), "+" C(O1)(o[1]), "+" C(O2)(o[2]), "+" C(O3)(o[3]), "+" C(O4)(o[4]),
                       "+" C(O5)(o[5]), "+" C(O6)(o[6]), "+" C(O7)(o[7]), "+" C(ML)(ml), "+" C(OFS)(ofs),
                       [t] "+&s"(k), [pg] "+&s"(pg_next)
                     : C(Q0)(q0), C(Q1)(q1), C(Q2)(q2), [t_end] "s"(k1), [t_begin] "s"(t_begin),
                       [last_tile_tok] "s"(last_tile_tok), [row_bytes] "s"(src.row_bytes), [pshift] "s"(src.page_shift),
                       [cache_lo] "s"(cache_lo), [cache_hi] "s"(cache_hi), [pages] "s"(src.pages), [scale2] "s"(scale2_bits),
                       [wave_blk] "s"(wave_blk), [slot0] "s"(s0), [slot1] "s"(s1), [slot2] "s"(s2), [slot3] "s"(s3)
                     : RPA_MLA_PIPE_CLOBBERS);
      }
#undef C
      m = __uint_as_float(ml[0]);
      l = __uint_as_float(ml[1]);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[4 * i + (e >> 2)][e & 3] = o[i][e];
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // drain the copies issued past the end

  // ---- epilogue: lane (c, g) holds head head0+c, dims 16j + 4g + r in acc[j][r] ----
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  // The lane parts of the output addresses are worked out here, from values the compiler cannot
  // trace back across the tile loop: hoisted out of it they would sit in registers the loop has
  // none to spare for (they were spilled to scratch memory).
  int c_out = c, g_out = g;
  if constexpr (PIPE) {
    const int ln = fresh_lane();
    c_out = ln & 15;
    g_out = ln >> 4;
  }
  asm volatile("" : "+v"(c_out), "+v"(g_out));
  const int head = head0 + c_out;
  if (TG ? !tg_real : (!wave_on || head >= a.Hq)) return;
  const int chunk0 = DS > 1 ? sub * kChunksPerWave : 0;  // shared tiles: this wave's output chunks
  if (dest.final_rows) {
    const float inv = a.out_scale / l;
    uint16_t* op = a.out + ((int64_t)tq * a.Hq + head) * 512 + g_out * 4 + chunk0 * 16;
#pragma unroll
    for (int j = 0; j < kChunksPerWave; ++j) {
      u32x2_t w = {pack_bf16x2(acc[j][0] * inv, acc[j][1] * inv), pack_bf16x2(acc[j][2] * inv, acc[j][3] * inv)};
      *reinterpret_cast<u32x2_t*>(op + j * 16) = w;
    }
  } else {
    const int64_t slot = dest.base + head;
    // partial rows are left as bf16: the merge reads half the bytes, and the result is rounded to
    // bf16 anyway
    uint16_t* wo = a.ws_o + slot * 512 + g_out * 4 + chunk0 * 16;
#pragma unroll
    for (int j = 0; j < kChunksPerWave; ++j) {
      u32x2_t w = {pack_bf16x2(acc[j][0], acc[j][1]), pack_bf16x2(acc[j][2], acc[j][3])};
      *reinterpret_cast<u32x2_t*>(wo + j * 16) = w;
    }
    if (g_out == 0 && (DS == 1 || sub == 0)) {
      a.ws_ml[slot * 2 + 0] = m;
      a.ws_ml[slot * 2 + 1] = l;
    }
  }
}

// ---- fixed split plan: grid = (max_splits * rows, 1, head groups of 128); block = 512 threads
template <bool UNIFORM, bool CAP, bool PIPE = false, bool FP8 = false, int DS = 1>
__global__ __launch_bounds__(512, 2) void rpa_mla_decode_kernel(const MlaDecodeArgs a) {
  // three separate arrays: lets the compiler see that a copy into one slot does not alias the
  // reads of another, so it does not drain the vector-memory queue before LDS reads
  __shared__ __attribute__((aligned(1024))) char slot0[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot1[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot2[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot3[kSlotB];
  const int nsp = max(a.max_splits, 1);  // grid.x = max_splits * rows, splits fastest
  const int row_id = (int)(blockIdx.x / (unsigned)nsp);
  const int split = (int)blockIdx.x - row_id * nsp;
  const MlaRow mr = mla_row(a, row_id);
  if (!mr.valid) return;
  const int kv_len = mr.kv_len;
  if (kv_len <= 0) return;
  const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
  const int t0 = t_lo & ~(kTok - 1);
  const int t_begin = t0 + split * a.chunk;
  if (t_begin >= kv_len) return;
  const int t_end = (split == a.max_splits - 1) ? kv_len : min(kv_len, t_begin + a.chunk);
  MlaDest dest;
  dest.final_rows = a.max_splits == 1;
  dest.base = ((int64_t)row_id * a.max_splits + split) * a.Hq;
  mla_segment<UNIFORM, CAP, PIPE, FP8, DS>(a, mr, blockIdx.z * 128, t_lo, t_begin, t_end, dest, slot0, slot1, slot2, slot3);
}

// immediate of s_waitcnt vmcnt(n) (n < 64) with the other counters left alone
constexpr int vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// ---- wide workgroups: FOUR waves, each owning two blocks of 16 heads, so that every K and V^T operand read
// from LDS feeds two matrix instructions (LDS reads, not the matrix pipe, are what the eight-wave
// workgroups wait for).  256 accumulators in the accumulation registers, 144 registers of Q^T, one wave per
// SIMD.  Every tile of the segment runs inside the assembly loop of rpa_mla_wide_loop.inc (masks and the
// clamped copies of the row's last tile included); compiled code only loads the queries, starts the ring,
// takes the first tile's maxima as the reference and writes the result.  bf16 caches, pages of a
// power-of-two size >= 32, no soft cap, Hq a multiple of 128.  `ring`: the four slots, contiguous.
// M32: the loop of rpa_mla_wide32_loop.inc (32x32x16 matrix instructions, one head per lane and half: lane c of
// half h = lane / 32 owns head head0 + c and the tokens 8 (i / 4) + 4 h + i % 4 of a tile) instead of two blocks of
// 16 heads on 16x16x32 instructions.
// TG (token group, see mla_segment; 16 / 32 / 64 heads, no window): the workgroup's eight blocks of 16 heads are the
// heads of 8 / 4 / 2 consecutive query tokens of one sequence, `group_tokens` of them real.  Block hb of wave w
// is "head" 32 w + 16 hb .. of a 128-head row at mr.tq, i.e. token (32 w + 16 hb) / Hq of the group; mr.kv_len is what
// the group's LAST token sees, a block's own token sees up to group_tokens - 1 fewer, so the loop masks the
// tile before the last too and takes the second block's row end relative to the first's.
template <bool M32, bool TG = false>
__device__ __forceinline__ void mla_segment_wide(const MlaDecodeArgs& a, const MlaRow mr, int head_base, int t_lo,
                                                 int t_begin, int t_end, const MlaDest dest, char* ring,
                                                 int trace_piece = 0, int group_tokens = 1) {
  static_assert(!(M32 && TG), "token groups run on the loop of two 16-head blocks");
  (void)trace_piece;
  RPA_MLA_STAMP(0);
  constexpr int CPW = 2 * kCopiesPerWave;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = M32 ? (lane & 31) : (lane & 15), g = M32 ? (lane >> 5) : (lane >> 4);
  const int head0 = head_base + wave * 32;
  const int seq = mr.seq;
  const int kv_len = mr.kv_len;
  const int tq = mr.tq;
  // per block of 16 heads: its first head in the row at tq, whether it writes, and the length its token sees
  int blk_head[2], blk_len[2];
  bool blk_real[2];
#pragma unroll
  for (int hb = 0; hb < 2; ++hb) {
    if constexpr (TG) {
      // (16, 32 or 64 heads: shifts, and every value the same in all lanes)
      const int hq_shift = __builtin_amdgcn_readfirstlane(31 - __builtin_clz(a.Hq));
      const int h = wave * 32 + 16 * hb;
      const int place = min(h >> hq_shift, group_tokens - 1);  // a block past the group's last real token repeats that token
      blk_real[hb] = (h >> hq_shift) < group_tokens;
      blk_head[hb] = __builtin_amdgcn_readfirstlane((place << hq_shift) + (h & (a.Hq - 1)));
      blk_len[hb] = __builtin_amdgcn_readfirstlane(kv_len - (group_tokens - 1) + place);
    } else {
      blk_real[hb] = true;
      blk_head[hb] = head0 + 16 * hb;
      blk_len[hb] = kv_len;
    }
  }

  Src src;
  src.page_size = a.pt.page_size;
  src.page_shift = 31 - __builtin_clz(src.page_size);
  src.last_tok = kv_len - 1;
  src.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / a.pt.page_size)
                                                  : (int64_t)seq * a.pt.pages_per_seq);
  src.row_bytes = a.row_stride * 2;
  src.page_stride = (int64_t)src.row_bytes * a.pt.page_size;
  src.rope_byte = a.rope_offset * 2;
  auto page_of = [&](int tb) -> int {
    tb = min(tb, src.last_tok & ~(kTok - 1));
    return scalar_load_i32(src.pages + __builtin_amdgcn_readfirstlane(page_slot(src, tb)));
  };

  // ---- Q^T operands: column c of block hb = head head0 + 16 hb + c, k-step ks covers dims 32ks + 8g .. ----
  // 16x16x32: qB[hb][ks], k-step ks covers dims 32ks + 8g ..; 32x32x16: the same 36 registers of 4 as
  // qB[ks / 18][ks % 18], k-step ks covers dims 16ks + 8g .. of head head0 + c
  u32x4_t qB[2][18];
  if constexpr (M32) {
    const int head = min(head0 + c, a.Hq - 1);
    const uint16_t* qn = a.ql_nope + ((int64_t)tq * a.Hq + head) * 512 + g * 8;
    const uint16_t* qr = a.q_pe + ((int64_t)tq * a.Hq + head) * 64 + g * 8;
#pragma unroll
    for (int ks = 0; ks < 36; ++ks) qB[ks / 18][ks % 18] = ld16(ks < 32 ? qn + ks * 16 : qr + (ks - 32) * 16);
  } else {
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {
      const int head = TG ? blk_head[hb] + c : min(head0 + 16 * hb + c, a.Hq - 1);
      const uint16_t* qn = a.ql_nope + ((int64_t)tq * a.Hq + head) * 512 + g * 8;
      const uint16_t* qr = a.q_pe + ((int64_t)tq * a.Hq + head) * 64 + g * 8;
#pragma unroll
      for (int ks = 0; ks < 16; ++ks) qB[hb][ks] = ld16(qn + ks * 32);
      qB[hb][16] = ld16(qr);
      qB[hb][17] = ld16(qr + 32);
    }
  }
  const float scale2 = a.sm.sm_scale * kLog2e;

  int pg_next = page_of(t_begin + 3 * kTok);
  copy_tile<true, CPW>(ring, src, a.cache, t_begin, wave, lane, page_of(t_begin));
  copy_tile<true, CPW>(ring + kSlotB, src, a.cache, t_begin + kTok, wave, lane, page_of(t_begin + kTok));
  copy_tile<true, CPW>(ring + 2 * kSlotB, src, a.cache, t_begin + 2 * kTok, wave, lane, page_of(t_begin + 2 * kTok));
#pragma unroll
  for (int hb = 0; hb < 2; ++hb)
#pragma unroll
    for (int ks = 0; ks < 18; ++ks) asm volatile("" ::"v"(qB[hb][ks]));
  // the tiles the first step reads have landed once only the newest copies are outstanding (the generated
  // loop says how many: the same count its own end-of-step wait uses)
  static_assert(RPA_MLA_WIDE_COPIES_AHEAD == RPA_MLA_WIDE32_COPIES_AHEAD, "one prologue for both loops");
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(RPA_MLA_WIDE_COPIES_AHEAD));
  __syncthreads();
  RPA_MLA_STAMP(1);

  // ---- the reference of the probabilities: per head, the maximum of the first tile's visible scores ----
  float m_init[2];
  if constexpr (M32) {
    f32x16_t s = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const char* kp = ring + c * kRowB + g * 16;
#pragma unroll
    for (int ks = 0; ks < 36; ++ks) s = mfma32(lds_ld16(kp + ks * 32), qB[ks / 18][ks % 18], s);
    float mx = -3.0e38f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int tok = t_begin + 8 * (i >> 2) + 4 * g + (i & 3);
      if (tok < kv_len && tok >= t_lo) mx = fmaxf(mx, s[i] * scale2);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    m_init[0] = m_init[1] = mx;
  } else {
    f32x4_t s[2][2];
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) s[hb][0] = s[hb][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const char* kp = ring + c * kRowB + g * 16;
#pragma unroll
    for (int ks = 0; ks < 18; ++ks) {
      const u32x4_t k0 = lds_ld16(kp + ks * 64);
      const u32x4_t k1 = lds_ld16(kp + 16 * kRowB + ks * 64);
#pragma unroll
      for (int hb = 0; hb < 2; ++hb) {
        s[hb][0] = mfma16(k0, qB[hb][ks], s[hb][0]);
        s[hb][1] = mfma16(k1, qB[hb][ks], s[hb][1]);
      }
    }
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {
      float mx = -3.0e38f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int tok = t_begin + tok_of(g, i);
        if (tok < blk_len[hb] && tok >= t_lo) mx = fmaxf(mx, s[hb][i >> 2][i & 3] * scale2);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      m_init[hb] = mx;
    }
  }

  // ---- the loop ----
  typedef __attribute__((address_space(3))) char* lds_ptr_t;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)ring);
  const int nT = (t_end - t_begin + kTok - 1) / kTok;
  f32x32_t o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 32; ++e) o[i][e] = 0.f;
  u32x32_t q0, q1, q2, q3;
  u32x16_t q4;
#pragma unroll
  for (int e = 0; e < 32; ++e) {
    q0[e] = qB[0][e >> 2][e & 3];
    q1[e] = qB[0][8 + (e >> 2)][e & 3];
    q3[e] = qB[1][6 + (e >> 2)][e & 3];           // registers 96 .. 127 = block 1, operands 6 .. 13
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) q2[e] = qB[0][16 + (e >> 2)][e & 3];                 // registers 64 .. 71
#pragma unroll
  for (int e = 8; e < 32; ++e) q2[e] = qB[1][(e - 8) >> 2][(e - 8) & 3];            // registers 72 .. 95 = block 1, operands 0 .. 5
#pragma unroll
  for (int e = 0; e < 16; ++e) q4[e] = qB[1][14 + (e >> 2)][e & 3];                // registers 128 .. 143
  const int ln = fresh_lane();  // lane parts are worked out here, not carried from the top
  u32x8_t ml;
  if constexpr (M32) {
    // K operand: row c, bytes 32ks + 16g.  V^T operand of (dim block d, k-step kk): the lane points at token
    // 16kk + 4g + (r >> 2) (+ 8 for the second read), dims 32d + 16 (b & 1) + 8 ((r & 3) >> 1) + 4 (r & 1), with
    // r = lane & 15, b = lane >> 4 (what the transposing read hands to lane dim = lane % 32)
    const int cc = ln & 31, gg = ln >> 5, r16 = ln & 15, b16 = ln >> 4;
    const int v_in = ((b16 & 1) << 5) + (((r16 & 3) >> 1) << 4) + ((r16 & 1) << 3);
    ml = u32x8_t{__float_as_uint(m_init[0]), 0u, lds_base + (uint32_t)(cc * kRowB + gg * 16),
                 lds_base + (uint32_t)((4 * gg + (r16 >> 2)) * kRowB + v_in), (uint32_t)(t_lo - t_begin - 4 * gg),
                 (uint32_t)(kv_len - t_begin - 4 * gg), 0u, 0u};
  } else {
    const int cc = ln & 15, gg = ln >> 4;
    ml = u32x8_t{__float_as_uint(m_init[0]), 0u, __float_as_uint(m_init[1]), 0u,
                 lds_base + (uint32_t)(cc * kRowB + gg * 16),
                 lds_base + (uint32_t)((4 * gg + (cc >> 2)) * kRowB + (cc & 3) * 8),
                 (uint32_t)(t_lo - t_begin - 4 * gg), (uint32_t)(blk_len[0] - t_begin - 4 * gg)};
  }
  const int hi_step = blk_len[1] - blk_len[0];
  const int mask_early = TG ? 1 : 0;
  u32x16_t ofs, ofsl;
#pragma unroll
  for (int n = 0; n < 16; ++n) ofs[n] = ofsl[n] = 0;
  const int last_row = src.last_tok & (kTok - 1);  // last valid row of the row's last tile
#pragma unroll
  for (int n = 0; n < CPW; ++n) {
    int row, inner;
    chunk_of<CPW>(src, wave, ln, n, row, inner);
    ofs[n] = (uint32_t)(row * src.row_bytes + inner);
    ofsl[n] = (uint32_t)(min(row, last_row) * src.row_bytes + inner);
  }
  const uint32_t cache_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)a.cache);
  const uint32_t cache_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)a.cache >> 32));
  const int last_tile_tok = __builtin_amdgcn_readfirstlane(src.last_tok & ~(kTok - 1));
  const uint32_t scale2_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(scale2));
  const int wave_blk = wave * 1024;  // the wave's first copy block inside a slot (see copy_block)
  // `t` and `pg` change inside the block while the inputs are still being read: early-clobber, or the compiler
  // may give an input that happens to hold the same value on entry (the LDS base, 0, and t = 0) the same register
  int k = 0;
  RPA_MLA_STAMP(2);
  // both loops bind their operands to the same registers
#define C(n) RPA_MLA_WIDE_C_##n
#define RPA_WIDE_OPERANDS                                                                                              \
  : "+" C(O0)(o[0]), "+" C(O1)(o[1]), "+" C(O2)(o[2]), "+" C(O3)(o[3]), "+" C(O4)(o[4]), "+" C(O5)(o[5]),                \
    "+" C(O6)(o[6]), "+" C(O7)(o[7]), "+" C(ML)(ml), "+" C(OFS)(ofs), [t] "+&s"(k), [pg] "+&s"(pg_next)                 \
  : C(Q0)(q0), C(Q1)(q1), C(Q2)(q2), C(Q3)(q3), C(Q4)(q4), C(OFSL)(ofsl), [t_end] "s"(nT), [t_begin] "s"(t_begin),     \
    [last_tile_tok] "s"(last_tile_tok), [row_bytes] "s"(src.row_bytes), [pshift] "s"(src.page_shift),                  \
    [cache_lo] "s"(cache_lo), [cache_hi] "s"(cache_hi), [pages] "s"(src.pages), [scale2] "s"(scale2_bits),             \
    [wave_blk] "s"(wave_blk), [slot0] "s"(lds_base), [hi_step] "s"(hi_step), [mask_early] "s"(mask_early)
  if constexpr (M32) {
    asm volatile(RPA_MLA_WIDE32_ASM RPA_WIDE_OPERANDS : RPA_MLA_WIDE32_CLOBBERS);
  } else {
    asm volatile(RPA_MLA_WIDE_ASM RPA_WIDE_OPERANDS : RPA_MLA_WIDE_CLOBBERS);
  }
#undef RPA_WIDE_OPERANDS
#undef C
  __builtin_amdgcn_s_waitcnt(0x0F70);  // drain the copies issued past the end
  RPA_MLA_STAMP(3);

  // ---- epilogue ----
  const int lo_ = fresh_lane();
  if constexpr (M32) {
    // lane (c, h) holds head head0 + c, dims 32d + 8q + 4h + r in accumulator 16d + 4q + r
    const int c_out = lo_ & 31, h_out = lo_ >> 5;
    const float m = __uint_as_float(ml[0]);
    float l = __uint_as_float(ml[1]);
    l += __shfl_xor(l, 32);
    const int head = head0 + c_out;
    if (head < a.Hq) {
      const float inv = dest.final_rows ? a.out_scale / l : 1.0f;
      uint16_t* op = dest.final_rows ? a.out + ((int64_t)tq * a.Hq + head) * 512 + h_out * 4
                                     : a.ws_o + (dest.base + head) * 512 + h_out * 4;
#pragma unroll
      for (int d = 0; d < 16; ++d)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int e = (16 * d + 4 * q) & 31, i = d >> 1;
          u32x2_t w = {pack_bf16x2(o[i][e] * inv, o[i][e + 1] * inv), pack_bf16x2(o[i][e + 2] * inv, o[i][e + 3] * inv)};
          *reinterpret_cast<u32x2_t*>(op + 32 * d + 8 * q) = w;
        }
      if (!dest.final_rows && h_out == 0) {
        a.ws_ml[(dest.base + head) * 2 + 0] = m;
        a.ws_ml[(dest.base + head) * 2 + 1] = l;
      }
    }
  } else {
  // lane (c, g) holds head head0 + 16 hb + c, dims 16j + 4g + r in accumulator 128 hb + 4 j + r
  const int c_out = lo_ & 15, g_out = lo_ >> 4;
#pragma unroll
  for (int hb = 0; hb < 2; ++hb) {
    const float m = __uint_as_float(ml[2 * hb]);
    float l = __uint_as_float(ml[2 * hb + 1]);
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    const int head = blk_head[hb] + c_out;
    if (TG ? !blk_real[hb] : head >= a.Hq) continue;
    if (dest.final_rows) {
      const float inv = a.out_scale / l;
      uint16_t* op = a.out + ((int64_t)tq * a.Hq + head) * 512 + g_out * 4;
#pragma unroll
      for (int j = 0; j < 32; ++j) {
        const int e = (4 * j) & 31, i = 4 * hb + (j >> 3);
        u32x2_t w = {pack_bf16x2(o[i][e] * inv, o[i][e + 1] * inv), pack_bf16x2(o[i][e + 2] * inv, o[i][e + 3] * inv)};
        *reinterpret_cast<u32x2_t*>(op + j * 16) = w;
      }
    } else {
      const int64_t slot = dest.base + head;
      uint16_t* wo = a.ws_o + slot * 512 + g_out * 4;
#pragma unroll
      for (int j = 0; j < 32; ++j) {
        const int e = (4 * j) & 31, i = 4 * hb + (j >> 3);
        u32x2_t w = {pack_bf16x2(o[i][e], o[i][e + 1]), pack_bf16x2(o[i][e + 2], o[i][e + 3])};
        *reinterpret_cast<u32x2_t*>(wo + j * 16) = w;
      }
      if (g_out == 0) {
        a.ws_ml[slot * 2 + 0] = m;
        a.ws_ml[slot * 2 + 1] = l;
      }
    }
  }
  }
  // every wave has left the loop behind its last barrier; the next segment's first copies overwrite slots
  // 0 .. 2, whose last readers (this segment's last steps) may still be running in another wave
  __syncthreads();
  RPA_MLA_STAMP(4);
#ifdef RPA_MLA_TRACE
  if (threadIdx.x == 0 && trace_piece < 4) {
    rpa_mla_trace_buf[blockIdx.x & 1023][trace_piece][5] = (unsigned long long)((t_end - t_begin + kTok - 1) / kTok);
    rpa_mla_trace_buf[blockIdx.x & 1023][trace_piece][6] = (unsigned long long)dest.final_rows;
  }
#endif
}

// ---- token groups (see mla_segment, TG): 16 / 32 / 64 heads, every query token a row, whole rows (no pieces).
// grid = windows of 128 / Hq consecutive query tokens of the call.  A window that lies inside one sequence is one
// group; one that spans a border between sequences (the end of a chunk, decode rows of one token each) runs one
// group per sequence, one after the other.
template <bool PIPE, bool FP8>
__global__ __launch_bounds__(512, 2) void rpa_mla_token_group_kernel(const MlaDecodeArgs a) {
  __shared__ __attribute__((aligned(1024))) char slot0[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot1[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot2[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot3[kSlotB];
  const int num_seqs = a.dist ? min(a.num_seqs, scalar_load_i32(a.dist + 2)) : a.num_seqs;
  const int total = min(a.num_rows, scalar_load_i32(a.pt.cu_q_lens + num_seqs));
  const int per = 128 / a.Hq;
  int t = (int)blockIdx.x * per;
  if (t >= total) return;
  const int t_stop = min(t + per, total);
  int seq = owner_of_token(a.pt.cu_q_lens, num_seqs, t);
  while (t < t_stop) {
    // (everything here is the same in every lane; said so explicitly, the assembly loop takes scalars)
    seq = __builtin_amdgcn_readfirstlane(seq);
    t = __builtin_amdgcn_readfirstlane(t);
    const int q0 = scalar_load_i32(a.pt.cu_q_lens + seq);
    const int q1 = scalar_load_i32(a.pt.cu_q_lens + seq + 1);
    if (q1 <= t) {  // (a sequence without tokens)
      ++seq;
      continue;
    }
    const int n = __builtin_amdgcn_readfirstlane(min(t_stop, q1) - t);  // tokens of this sequence in the window
    MlaRow mr;
    mr.seq = seq;
    mr.tq = t;
    mr.valid = true;
    // what the group's last token sees
    mr.kv_len = __builtin_amdgcn_readfirstlane(scalar_load_i32(a.pt.kv_lens + seq) - (q1 - q0) + (t + n - 1 - q0) + 1);
    const int first_len = mr.kv_len - (n - 1);
    if (mr.kv_len > 0 && first_len > 0) {
      const int t_lo = (a.sm.window > 0) ? max(0, first_len - a.sm.window) : 0;
      MlaDest dest;
      dest.final_rows = true;
      dest.base = 0;
      mla_segment<true, false, PIPE, FP8, 1, true>(a, mr, 0, t_lo, t_lo & ~(kTok - 1), mr.kv_len, dest, slot0, slot1, slot2,
                                                   slot3, n);
    }
    t += n;
    if (t >= q1) ++seq;
  }
}

// ---- token groups on wide workgroups (see mla_segment_wide, TG): bf16 latents, no window.  Same grid and the same
// walk over a window of 128 / Hq query tokens as rpa_mla_token_group_kernel.
__global__ __launch_bounds__(256, 1) void rpa_mla_token_group_wide_kernel(const MlaDecodeArgs a) {
  __shared__ __attribute__((aligned(1024))) char ring[4 * kSlotB];
  const int num_seqs = a.dist ? min(a.num_seqs, scalar_load_i32(a.dist + 2)) : a.num_seqs;
  const int total = min(a.num_rows, scalar_load_i32(a.pt.cu_q_lens + num_seqs));
  const int per = 128 / a.Hq;
  int t = (int)blockIdx.x * per;
  if (t >= total) return;
  const int t_stop = min(t + per, total);
  int seq = owner_of_token(a.pt.cu_q_lens, num_seqs, t);
  while (t < t_stop) {
    seq = __builtin_amdgcn_readfirstlane(seq);
    t = __builtin_amdgcn_readfirstlane(t);
    const int q0 = scalar_load_i32(a.pt.cu_q_lens + seq);
    const int q1 = scalar_load_i32(a.pt.cu_q_lens + seq + 1);
    if (q1 <= t) {  // (a sequence without tokens)
      ++seq;
      continue;
    }
    const int n = __builtin_amdgcn_readfirstlane(min(t_stop, q1) - t);  // tokens of this sequence in the window
    MlaRow mr;
    mr.seq = seq;
    mr.tq = t;
    mr.valid = true;
    mr.kv_len = __builtin_amdgcn_readfirstlane(scalar_load_i32(a.pt.kv_lens + seq) - (q1 - q0) + (t + n - 1 - q0) + 1);
    if (mr.kv_len > 0 && mr.kv_len - (n - 1) > 0) {
      MlaDest dest;
      dest.final_rows = true;
      dest.base = 0;
      mla_segment_wide<false, true>(a, mr, 0, 0, 0, mr.kv_len, dest, ring, 0, n);
    }
    t += n;
    if (t >= q1) ++seq;
  }
}

// ---- fixed split plan, wide workgroups: grid = (max_splits * rows, 1, head groups of 128); block = 256 threads
template <bool M32>
__global__ __launch_bounds__(256, 1) void rpa_mla_decode_wide_kernel(const MlaDecodeArgs a) {
  __shared__ __attribute__((aligned(1024))) char ring[4 * kSlotB];
  const int nsp = max(a.max_splits, 1);  // grid.x = max_splits * rows, splits fastest
  const int row_id = (int)(blockIdx.x / (unsigned)nsp);
  const int split = (int)blockIdx.x - row_id * nsp;
  const MlaRow mr = mla_row(a, row_id);
  if (!mr.valid) return;
  const int kv_len = mr.kv_len;
  if (kv_len <= 0) return;
  const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
  const int t0 = t_lo & ~(kTok - 1);
  const int t_begin = t0 + split * a.chunk;
  if (t_begin >= kv_len) return;
  const int t_end = (split == a.max_splits - 1) ? kv_len : min(kv_len, t_begin + a.chunk);
  MlaDest dest;
  dest.final_rows = a.max_splits == 1;
  dest.base = ((int64_t)row_id * a.max_splits + split) * a.Hq;
  mla_segment_wide<M32>(a, mr, blockIdx.z * 128, t_lo, t_begin, t_end, dest, ring);
}

// ---- balanced plan (one row per sequence): the 32-token tiles of the whole batch, sequence by
// sequence and inside a sequence head group by head group, are dealt evenly to the workgroups;
// workgroup j takes tiles [j * pw, (j + 1) * pw).  Pieces that are whole rows are finished in
// place, cut ones (at most the first and the last of a workgroup) leave partial rows in the
// workspace slots 2j and 2j + 1 (128 heads each).
//
// Starting a piece is not free: 147 KB of queries and the first tiles have to arrive and the
// piece before it has to be written out -- 17 us on the DeepSeek-V3 batch, five tiles' worth, and
// a workgroup with three pieces finished 37 us after one with a single piece.  So the line the
// workgroups share is padded: every (row, head group) is preceded by `piece_pad` tiles that hold
// no work.  A workgroup that runs into a new row spends that much of its share on the way, which
// is what the switch costs it; one that starts in the middle of a row, like most, pays nothing
// extra -- every workgroup has one start of its own anyway.
__device__ __forceinline__ int mla_tiles(int kv_len, int window) {
  if (kv_len <= 0) return 0;
  const int t_lo = (window > 0) ? max(0, kv_len - window) : 0;
  return (kv_len - (t_lo & ~(kTok - 1)) + kTok - 1) / kTok;
}

// extent of a (row, head group) on the padded line
__device__ __forceinline__ int mla_extent(const MlaDecodeArgs& a, int kv_len) {
  const int nt = mla_tiles(kv_len, a.sm.window);
  return nt > 0 ? nt + a.piece_pad : 0;
}

__device__ __forceinline__ int mla_tiles_per_wg(const MlaDecodeArgs& a, int total) {
  const int even = (total + a.num_wgs - 1) / a.num_wgs;  // the grid has exactly num_wgs workgroups
  return max(a.forced_tiles_per_wg > 0 ? a.forced_tiles_per_wg : a.min_tiles_per_wg, even);
}

// `segment(mr, head_base, t_lo, t_begin, t_end, dest)` runs one piece on the workgroup's LDS ring.
template <class Segment>
__device__ __forceinline__ void mla_balanced_body(const MlaDecodeArgs& a, Segment segment) {
  const int lane = threadIdx.x & 63;
  const int wg = blockIdx.x;
  const int units = (a.Hq + 127) / 128;
#ifdef RPA_MLA_TRACE
  if (threadIdx.x == 0) rpa_mla_trace_buf[blockIdx.x & 1023][0][7] = wall_clock64();  // kernel entry
#endif
  // prefix sums of tiles over the sequences: every wave scans (the result is wave-uniform)
  int total = 0, seq = -1, seq_first = 0;
  {
    // first pass: total; second pass (below) locates this workgroup's first tile
    for (int s0 = 0; s0 < a.num_rows; s0 += 64) {
      const int s = s0 + lane;
      int nt = (s < a.num_rows) ? mla_extent(a, a.pt.kv_lens[s]) : 0;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) nt += __shfl_xor(nt, off);
      total += nt;
    }
    total = __builtin_amdgcn_readfirstlane(total) * units;
  }
  const int pw = mla_tiles_per_wg(a, total);
  if (wg == 0 && threadIdx.x < 64) {
    int base = 0;
    for (int s0 = 0; s0 < a.num_rows; s0 += 64) {
      const int s = s0 + lane;
      const int nt = (s < a.num_rows) ? mla_extent(a, a.pt.kv_lens[s]) : 0;
      int incl = nt;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int n = __shfl_up(incl, off);
        if (lane >= off) incl += n;
      }
      if (s < a.num_rows) a.cu_tiles[s + 1] = base + incl;
      base += __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
    }
    if (lane == 0) a.cu_tiles[0] = 0;
  }
  if ((int64_t)wg * pw >= total) return;
  int x = wg * pw;
  const int x_end = min(total, x + pw);
  {
    int base = 0;
    for (int s0 = 0; s0 < a.num_rows && seq < 0; s0 += 64) {
      const int s = s0 + lane;
      const int nt = (s < a.num_rows) ? mla_extent(a, a.pt.kv_lens[s]) : 0;
      int incl = nt;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int n = __shfl_up(incl, off);
        if (lane >= off) incl += n;
      }
      const uint64_t hit = __builtin_amdgcn_ballot_w64((base + incl) * units > x);
      if (hit != 0) {
        const int first = __builtin_ctzll(hit);
        seq = s0 + first;
        seq_first = __builtin_amdgcn_readfirstlane((base + __shfl(incl - nt, first)) * units);
      } else {
        base += __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
      }
    }
    seq = __builtin_amdgcn_readfirstlane(seq);
  }
  int kv_len = scalar_load_i32(a.pt.kv_lens + seq);
  int nt = mla_tiles(kv_len, a.sm.window);
  const int pad = a.piece_pad;
  bool first_piece = true;
  int piece_no = 0;  // (only the optional timestamps use it)
  while (x < x_end) {
    const int r = x - seq_first;  // position inside the row's padded extents
    const int unit = r / (nt + pad);
    int off = r - unit * (nt + pad);
    if (off < pad) {  // the padding in front of this (row, head group): no work there
      x += pad - off;
      off = pad;
      if (x >= x_end) break;
    }
    const int tile = off - pad;
    const int take = min(nt - tile, x_end - x);
    const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
    const int t0 = t_lo & ~(kTok - 1);
    MlaRow mr;
    mr.seq = seq;
    mr.kv_len = kv_len;
    mr.tq = scalar_load_i32(a.pt.cu_q_lens + seq);
    mr.valid = true;
    MlaDest dest;
    dest.final_rows = (tile == 0) && (take == nt);
    dest.base = ((int64_t)wg * 2 + (first_piece ? 0 : 1)) * 128 - unit * 128;  // + head
    first_piece = false;
    segment(mr, unit * 128, t_lo, t0 + tile * kTok, min(kv_len, t0 + (tile + take) * kTok), dest, piece_no++);
    x += take;
    if (x < x_end && tile + take == nt && unit == units - 1) {
      seq_first += (nt + pad) * units;
      do {
        ++seq;
        kv_len = scalar_load_i32(a.pt.kv_lens + seq);
        nt = mla_tiles(kv_len, a.sm.window);
      } while (nt == 0);
    }
  }
}


template <bool UNIFORM, bool CAP, bool PIPE = false, bool FP8 = false, int DS = 1>
__global__ __launch_bounds__(512, 2) void rpa_mla_balanced_kernel(const MlaDecodeArgs a) {
  __shared__ __attribute__((aligned(1024))) char slot0[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot1[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot2[kSlotB];
  __shared__ __attribute__((aligned(1024))) char slot3[kSlotB];
  mla_balanced_body(a, [&](const MlaRow& mr, int head_base, int t_lo, int t_begin, int t_end, const MlaDest& dest, int)
                        __attribute__((always_inline)) {
    mla_segment<UNIFORM, CAP, PIPE, FP8, DS>(a, mr, head_base, t_lo, t_begin, t_end, dest, slot0, slot1, slot2, slot3);
  });
}

// the same plan on wide workgroups (four waves of 32 heads)
template <bool M32>
__global__ __launch_bounds__(256, 1) void rpa_mla_balanced_wide_kernel(const MlaDecodeArgs a) {
  __shared__ __attribute__((aligned(1024))) char ring[4 * kSlotB];
  mla_balanced_body(a, [&](const MlaRow& mr, int head_base, int t_lo, int t_begin, int t_end, const MlaDest& dest,
                           int piece) __attribute__((always_inline)) {
    mla_segment_wide<M32>(a, mr, head_base, t_lo, t_begin, t_end, dest, ring, piece);
  });
}

// Merge the n partial rows of one (row, head): one wave, 8 dims (16 bytes) per lane.  Partials are taken eight at
// a time with every load of a group (references, sums, rows) requested before any is used -- one
// round trip to memory per group instead of one per partial -- and groups are chained like tiles of
// an online softmax.  Places of a group past the last partial load nothing.
constexpr int kMergeThreads = 64;
template <typename SlotOf>
__device__ __forceinline__ void mla_merge(const MlaDecodeArgs& a, int n, SlotOf slot_of, int head, int tq) {
  const int d = threadIdx.x * 8;
  float mstar = -INFINITY, den = 0.f;
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = 0.f;
  for (int j0 = 0; j0 < n; j0 += 8) {
    float mj[8], lj[8];
    u32x4_t pr[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      mj[u] = -INFINITY;
      lj[u] = 0.f;
      pr[u] = u32x4_t{0u, 0u, 0u, 0u};
      if (j0 + u < n) {  // (the same in every lane)
        const int64_t slot = slot_of(j0 + u);
        mj[u] = a.ws_ml[slot * 2];
        lj[u] = a.ws_ml[slot * 2 + 1];
        pr[u] = ld16(a.ws_o + slot * 512 + d);
      }
    }
    float mnew = mstar;
#pragma unroll
    for (int u = 0; u < 8; ++u) mnew = fmaxf(mnew, mj[u]);
    const float keep = fast_exp2(mstar - mnew);  // 0 for the first group
    den *= keep;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] *= keep;
    mstar = mnew;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float w = (j0 + u < n) ? fast_exp2(mj[u] - mstar) : 0.f;
      den += lj[u] * w;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        o[2 * e] += bf16_lo_to_f32(pr[u][e]) * w;
        o[2 * e + 1] += bf16_hi_to_f32(pr[u][e]) * w;
      }
    }
  }
  const float inv = a.out_scale / den;
  const u32x4_t w = {pack_bf16x2(o[0] * inv, o[1] * inv), pack_bf16x2(o[2] * inv, o[3] * inv),
                     pack_bf16x2(o[4] * inv, o[5] * inv), pack_bf16x2(o[6] * inv, o[7] * inv)};
  st16(a.out + ((int64_t)tq * a.Hq + head) * 512 + d, w);
}

// Merge of the balanced plan.  grid = (Hq * rows); block = kMergeThreads.
__global__ __launch_bounds__(kMergeThreads) void rpa_mla_combine_balanced_kernel(const MlaDecodeArgs a) {
  const int seq = (int)(blockIdx.x / (unsigned)a.Hq);  // grid.x = Hq * rows, heads fastest
  const int head = (int)blockIdx.x - seq * a.Hq;
  const int nt = mla_tiles(a.pt.kv_lens[seq], a.sm.window);
  if (nt == 0) return;
  const int units = (a.Hq + 127) / 128;
  const int total = a.cu_tiles[a.num_rows] * units;
  const int pw = mla_tiles_per_wg(a, total);
  const int unit = head >> 7;
  // the row's head group on the padded line: `piece_pad` empty tiles, then its nt tiles
  const int extent_first = a.cu_tiles[seq] * units + unit * (nt + a.piece_pad);
  const int first_tile = extent_first + a.piece_pad;
  const int w_first = first_tile / pw, w_last = (first_tile + nt - 1) / pw;
  if (w_first == w_last) return;  // one workgroup covered the row and wrote the finished output
  auto slot_of = [&](int wj) -> int64_t {
    // slot 0 holds a workgroup's first piece: this one iff its share starts inside this extent
    // (padding included); a share that starts before it holds the last tile of the extent before
    const int part = ((int64_t)wj * pw >= extent_first) ? 0 : 1;
    return ((int64_t)wj * 2 + part) * 128 + (head & 127);
  };
  const int tq = scalar_load_i32(a.pt.cu_q_lens + seq);
  mla_merge(a, w_last - w_first + 1, [&](int j) { return slot_of(w_first + j); }, head, tq);
}

// grid = (Hq * rows); block = kMergeThreads.
__global__ __launch_bounds__(kMergeThreads) void rpa_mla_combine_kernel(const MlaDecodeArgs a) {
  const int row_id = (int)(blockIdx.x / (unsigned)a.Hq);  // grid.x = Hq * rows, heads fastest
  const int head = (int)blockIdx.x - row_id * a.Hq;
  const MlaRow mr = mla_row(a, row_id);
  if (!mr.valid || mr.kv_len <= 0) return;
  const int kv_len = mr.kv_len;
  const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
  const int t0 = t_lo & ~(kTok - 1);
  const int n = min(a.max_splits, (kv_len - t0 + a.chunk - 1) / a.chunk);
  if (n <= 0) return;
  const int64_t base = ((int64_t)row_id * a.max_splits) * a.Hq + head;
  mla_merge(a, n, [&](int jj) { return base + (int64_t)jj * a.Hq; }, head, mr.tq);
}

// New latent rows into the paged cache (mla/v1/ref.py:56-105): token j of sequence i goes to
// position kv_len_i - q_len_i + j; kv_c to elements [0, 512), k_pe to [rope_offset, +64).
// grid = tokens; block = 128 threads of which 72 move 16 bytes each.
__global__ __launch_bounds__(128) void rpa_mla_kv_write_kernel(const MlaWriteArgs a) {
  const int tok = blockIdx.x;
  const int num_seqs = a.dist ? min(a.num_seqs, scalar_load_i32(a.dist + 2)) : a.num_seqs;
  if (tok >= scalar_load_i32(a.pt.cu_q_lens + num_seqs)) return;
  const int seq = owner_of_token(a.pt.cu_q_lens, num_seqs, tok);
  const int q0 = scalar_load_i32(a.pt.cu_q_lens + seq);
  const int q_len = scalar_load_i32(a.pt.cu_q_lens + seq + 1) - q0;
  const int pos = scalar_load_i32(a.pt.kv_lens + seq) - q_len + (tok - q0);
  if (pos < 0) return;
  const int P = a.pt.page_size;
  const int32_t* pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / P)
                                                              : (int64_t)seq * a.pt.pages_per_seq);
  const int page = pages[pos / P];
  const int es = a.fp8 ? 1 : 2;  // bytes per element
  char* row = a.cache + ((int64_t)page * P + (pos % P)) * a.row_stride * es;
  const int t = threadIdx.x;
  const int nc = 32 * es;  // 16-byte chunks of kv_c; k_pe has an eighth of that
  if (t < nc) st16(row + t * 16, ld16(a.new_kv_c + ((int64_t)tok * 512 * es + t * 16)));
  else if (t < nc + 4 * es)
    st16(row + a.rope_offset * es + (t - nc) * 16, ld16(a.new_k_pe + ((int64_t)tok * 64 * es + (t - nc) * 16)));
}

}  // namespace

hipError_t launch_mla_kv_write(const MlaWriteArgs& a, hipStream_t stream) {
  if (a.num_tokens <= 0 || a.num_seqs <= 0) return hipSuccess;
  hipLaunchKernelGGL(rpa_mla_kv_write_kernel, dim3(a.num_tokens), dim3(128), 0, stream, a);
  return hipGetLastError();
}

ShapeKey mla_shape_key(const MlaDecodeArgs& a) {
  const int P = a.pt.page_size;
  ShapeKey k = {};
  k.stage = kStageMla;
  k.kv_bits = a.fp8 ? 8 : 16;
  k.head_dim = 576;
  k.heads = a.Hq;
  k.options = (a.sm.soft_cap != 0.f ? kOptSoftCap : 0u) | ((P % kTok) != 0 ? kOptOddPages : 0u) |
              ((P & (P - 1)) != 0 ? kOptNotPow2Pages : 0u) |
              ((int64_t)a.row_stride * 2 * P >= (int64_t(1) << 32) ? kOptWidePages : 0u);
  return k;
}

unsigned mla_shape_skip(const Tuning& tune) {
  return (tune.mla_pipe == 0 ? (1u << kKernelMlaWide) | (1u << kKernelMlaPipe) : 0u) |
         (tune.mla_wide == 0 ? (1u << kKernelMlaWide) : 0u) | (tune.mla_shared_tiles == 0 ? (1u << kKernelMlaShared) : 0u);
}

// Prefill / mixed rows with few heads: a workgroup holds 128 / Hq consecutive query tokens of a sequence over
// shared tiles instead of one token whose heads leave most of it idle (rows_are_tokens, whole rows, a head count
// that divides 128, whole tiles in pages, no soft cap; RPA_MLA_TOKEN_GROUPS=0 keeps one token per workgroup).
// Decode batches (one token per sequence) have nothing to group and keep the shared tiles.
// 0: no groups; 1: eight waves of one block of 16 heads (compiled tile loop); 2: the same around the assembly
// steady state; 3: four waves of two blocks on the wide loop (every operand fragment feeds two matrix
// instructions: bf16 latents, power-of-two pages, no window).
int mla_token_group_mode(const MlaDecodeArgs& a, const Tuning& tune, const ShapeRule& shape) {
  if (shape.kernel != kKernelMlaShared || !a.rows_are_tokens || a.max_splits > 1 || a.balanced ||
      tune.mla_token_groups == 0 || (128 % a.Hq) != 0 || a.Hq < 16 || a.num_rows < 4 * a.num_seqs)
    return 0;
  const int P = a.pt.page_size;
  const bool pipe_ok = tune.mla_pipe != 0 && (P & (P - 1)) == 0 && (int64_t)a.row_stride * 2 * P < (int64_t(1) << 32);
  if (!pipe_ok) return 1;
  if (!a.fp8 && a.sm.window <= 0 && tune.mla_wide != 0 && tune.mla_wide != 32) return 3;
  return 2;
}

hipError_t launch_mla_decode(const MlaDecodeArgs& a, hipStream_t stream) {
  if (a.num_rows <= 0) return hipSuccess;
  const int head_groups = (a.Hq + 127) / 128;
  if ((int64_t)a.max_splits * a.num_rows > 0x7fffffffLL || (int64_t)a.Hq * a.num_rows > 0x7fffffffLL)
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)max(a.max_splits, 1) * (unsigned)a.num_rows, 1, head_groups), block(512);
  const bool uniform = (a.pt.page_size % kTok) == 0;
  const bool cap = a.sm.soft_cap != 0.f;
  // the kernel family by shape (rpa_shapes.h): wide workgroups and the assembly tile loops need whole tiles inside
  // power-of-two pages, no soft cap and head counts in multiples of 128; with at most 64 heads (a tensor-parallel
  // share) the waves of a workgroup share each tile of a block of 16 heads; everything else runs the compiled
  // loop.  RPA_MLA_PIPE=0, RPA_MLA_WIDE=0 and RPA_MLA_SHARED_TILES=0 take a family out of the selection.
  const Tuning& tune = tuning();
  const ShapeRule& shape = select_shape(mla_shape_key(a), mla_shape_skip(tune));
  const bool pipe = shape.kernel == kKernelMlaWide || shape.kernel == kKernelMlaPipe;
  const int ds = shape.kernel == kKernelMlaShared ? shape.share : 1;
  if (const int tg = mla_token_group_mode(a, tune, shape)) {
    const bool pipe_ok = tg >= 2;
    const int per = 128 / a.Hq;
    const dim3 tg_grid((unsigned)((a.num_rows + per - 1) / per));
    if (tg == 3) {
      hipLaunchKernelGGL(rpa_mla_token_group_wide_kernel, tg_grid, dim3(256), 0, stream, a);
      return hipGetLastError();
    }
    if (a.fp8) {
      if (pipe_ok) hipLaunchKernelGGL((rpa_mla_token_group_kernel<true, true>), tg_grid, block, 0, stream, a);
      else hipLaunchKernelGGL((rpa_mla_token_group_kernel<false, true>), tg_grid, block, 0, stream, a);
    } else {
      if (pipe_ok) hipLaunchKernelGGL((rpa_mla_token_group_kernel<true, false>), tg_grid, block, 0, stream, a);
      else hipLaunchKernelGGL((rpa_mla_token_group_kernel<false, false>), tg_grid, block, 0, stream, a);
    }
    return hipGetLastError();
  }
  if (ds != 1) {
#define RPA_MLA_DS(KERNEL, GRID, F8)                                                                                  \
  do {                                                                                                                \
    if (ds == 8) hipLaunchKernelGGL((KERNEL<true, false, false, F8, 8>), GRID, block, 0, stream, a);                 \
    else if (ds == 4) hipLaunchKernelGGL((KERNEL<true, false, false, F8, 4>), GRID, block, 0, stream, a);            \
    else hipLaunchKernelGGL((KERNEL<true, false, false, F8, 2>), GRID, block, 0, stream, a);                         \
  } while (0)
    if (a.balanced) {
      const dim3 bgrid(a.num_wgs);
      if (a.fp8) RPA_MLA_DS(rpa_mla_balanced_kernel, bgrid, true);
      else RPA_MLA_DS(rpa_mla_balanced_kernel, bgrid, false);
      hipError_t eb = hipGetLastError();
      if (eb != hipSuccess) return eb;
      hipLaunchKernelGGL(rpa_mla_combine_balanced_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
      return hipGetLastError();
    }
    if (a.fp8) RPA_MLA_DS(rpa_mla_decode_kernel, grid, true);
    else RPA_MLA_DS(rpa_mla_decode_kernel, grid, false);
#undef RPA_MLA_DS
    hipError_t es = hipGetLastError();
    if (es != hipSuccess) return es;
    if (a.max_splits > 1) {
      hipLaunchKernelGGL(rpa_mla_combine_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
      es = hipGetLastError();
    }
    return es;
  }
  if (a.fp8) {  // e4m3 caches
    if (a.balanced) {
      const dim3 bgrid(a.num_wgs);
      if (pipe) {
        hipLaunchKernelGGL((rpa_mla_balanced_kernel<true, false, true, true>), bgrid, block, 0, stream, a);
      } else if (uniform) {
        if (cap) hipLaunchKernelGGL((rpa_mla_balanced_kernel<true, true, false, true>), bgrid, block, 0, stream, a);
        else hipLaunchKernelGGL((rpa_mla_balanced_kernel<true, false, false, true>), bgrid, block, 0, stream, a);
      } else {
        if (cap) hipLaunchKernelGGL((rpa_mla_balanced_kernel<false, true, false, true>), bgrid, block, 0, stream, a);
        else hipLaunchKernelGGL((rpa_mla_balanced_kernel<false, false, false, true>), bgrid, block, 0, stream, a);
      }
      hipError_t eb = hipGetLastError();
      if (eb != hipSuccess) return eb;
      hipLaunchKernelGGL(rpa_mla_combine_balanced_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
      return hipGetLastError();
    }
    if (pipe) {
      hipLaunchKernelGGL((rpa_mla_decode_kernel<true, false, true, true>), grid, block, 0, stream, a);
    } else if (uniform) {
      if (cap) hipLaunchKernelGGL((rpa_mla_decode_kernel<true, true, false, true>), grid, block, 0, stream, a);
      else hipLaunchKernelGGL((rpa_mla_decode_kernel<true, false, false, true>), grid, block, 0, stream, a);
    } else {
      if (cap) hipLaunchKernelGGL((rpa_mla_decode_kernel<false, true, false, true>), grid, block, 0, stream, a);
      else hipLaunchKernelGGL((rpa_mla_decode_kernel<false, false, false, true>), grid, block, 0, stream, a);
    }
    hipError_t ef = hipGetLastError();
    if (ef != hipSuccess) return ef;
    if (a.max_splits > 1) {
      hipLaunchKernelGGL(rpa_mla_combine_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
      ef = hipGetLastError();
    }
    return ef;
  }
  // wide workgroups (four waves of 32 heads) wherever the assembly loop applies; RPA_MLA_WIDE=0 keeps the
  // eight-wave kernels
  const bool wide = shape.kernel == kKernelMlaWide;
  // RPA_MLA_WIDE=32: the wide loop on 32x32x16 matrix instructions (one head per lane and half).  Half the matrix
  // instructions, and 8 % faster than the default loop when neither reads its operands -- but its 32-row LDS
  // reads collide on the 1184-byte row pitch that suits the 16-row reads (7 % slower as a whole): opt-in until
  // it has a row layout of its own
  const bool m32 = tune.mla_wide == 32;
  if (wide && a.balanced) {
    if (m32) hipLaunchKernelGGL(rpa_mla_balanced_wide_kernel<true>, dim3(a.num_wgs), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(rpa_mla_balanced_wide_kernel<false>, dim3(a.num_wgs), dim3(256), 0, stream, a);
    hipError_t eb = hipGetLastError();
    if (eb != hipSuccess) return eb;
    hipLaunchKernelGGL(rpa_mla_combine_balanced_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
    return hipGetLastError();
  }
  if (wide) {
    if (m32) hipLaunchKernelGGL(rpa_mla_decode_wide_kernel<true>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(rpa_mla_decode_wide_kernel<false>, grid, dim3(256), 0, stream, a);
    hipError_t ew = hipGetLastError();
    if (ew != hipSuccess) return ew;
    if (a.max_splits > 1) {
      hipLaunchKernelGGL(rpa_mla_combine_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
      ew = hipGetLastError();
    }
    return ew;
  }
  if (a.balanced) {
    const dim3 bgrid(a.num_wgs);
    if (pipe) {
      hipLaunchKernelGGL((rpa_mla_balanced_kernel<true, false, true>), bgrid, block, 0, stream, a);
    } else if (uniform) {
      if (cap) hipLaunchKernelGGL((rpa_mla_balanced_kernel<true, true>), bgrid, block, 0, stream, a);
      else hipLaunchKernelGGL((rpa_mla_balanced_kernel<true, false>), bgrid, block, 0, stream, a);
    } else {
      if (cap) hipLaunchKernelGGL((rpa_mla_balanced_kernel<false, true>), bgrid, block, 0, stream, a);
      else hipLaunchKernelGGL((rpa_mla_balanced_kernel<false, false>), bgrid, block, 0, stream, a);
    }
    hipError_t eb = hipGetLastError();
    if (eb != hipSuccess) return eb;
    hipLaunchKernelGGL(rpa_mla_combine_balanced_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
    return hipGetLastError();
  }
  if (pipe) {
    hipLaunchKernelGGL((rpa_mla_decode_kernel<true, false, true>), grid, block, 0, stream, a);
  } else if (uniform) {
    if (cap) hipLaunchKernelGGL((rpa_mla_decode_kernel<true, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((rpa_mla_decode_kernel<true, false>), grid, block, 0, stream, a);
  } else {
    if (cap) hipLaunchKernelGGL((rpa_mla_decode_kernel<false, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((rpa_mla_decode_kernel<false, false>), grid, block, 0, stream, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (a.max_splits > 1) {
    hipLaunchKernelGGL(rpa_mla_combine_kernel, dim3((unsigned)a.Hq * (unsigned)a.num_rows), dim3(kMergeThreads), 0, stream, a);
    e = hipGetLastError();
  }
  return e;
}

}  // namespace rpa

#ifdef RPA_MLA_TRACE
extern "C" __attribute__((visibility("default"))) int rpa_debug_mla_trace(void* host, size_t bytes) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(rpa::rpa_mla_trace_buf), std::min(bytes, sizeof(rpa::rpa_mla_trace_buf)));
}
#endif
