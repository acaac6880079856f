// Flash-style prefill / mixed kernel for ragged paged attention on gfx950.
//
// One workgroup (4 waves) owns a tile of 128 query positions of one query head
// of one sequence; wave w owns 32 of them.  KV is walked in tiles of 64 tokens
// gathered through the page table:
//   global -> registers -> LDS   K tile  [64 tok][128 dims]  (row pitch 272 B)
//                                V tile  transposed [128 dims][64 tok] (pitch 144 B)
//   S^T[tok, q]  = K . Q^T        v_mfma_f32_32x32x16_bf16, A = K rows from LDS,
//                                 B = Q^T held in registers for the whole loop
//   online softmax per query column (in-lane over tokens + one lane swap)
//   O^T[dim, q] += V^T . P^T      A = V^T rows from LDS, B = P^T straight from
//                                 the S^T result registers
// The S^T result layout (lane = query, registers = tokens) is the B operand
// layout of the second product provided the 16 tokens of a k-step are ordered
// 16kk + 8*(i/4) + 4h + i%4; the V loader writes its transposed rows in exactly
// that order (register transpose with v_perm_b32 while staging), so no data
// crosses lanes between the two products.
//
// Workgroup ids are remapped so that everything that reads one kv head of one
// sequence runs on the same XCD (same L2) while the ragged sequences are spread
// evenly over the 8 XCDs: hardware deals workgroup n to XCD n % 8.

#include "rpa_common.h"
#include "rpa_kernels.h"

namespace rpa {

namespace {

constexpr int kBM = 128;      // query rows per workgroup
constexpr int kBN = 64;       // kv tokens per tile
constexpr int kKPitch = 272;  // bytes per K row in LDS (256 + 16 pad: conflict-free b128 reads)
constexpr int kVPitch = 144;  // bytes per V^T row in LDS (128 + 16 pad)

__device__ __forceinline__ u32x4_t lds_ld16(const char* p) { return *reinterpret_cast<const u32x4_t*>(p); }
__device__ __forceinline__ void lds_st16(char* p, u32x4_t v) { *reinterpret_cast<u32x4_t*>(p) = v; }

// token (inside a 64-token tile) that lands at LDS position 8*tg + i of a V^T row
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

// Page ids a thread needs for one tile, fetched one tile ahead of the rows themselves so
// that the dependent chain "page id -> row address -> row" is never exposed.
//   UNIFORM (page_size % 64 == 0): the whole tile lies in one page, one id.
//   otherwise: the K loader needs 1 id, a V loader thread up to 8 (one per token it stages).
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
  if constexpr (UNIFORM) {
    pg.id[0] = __builtin_amdgcn_readfirstlane(s.pages[page_slot(s, min(tb, s.last_tok))]);
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

__device__ __forceinline__ int64_t row_offset(const TileSrc& s, const KvAddr& kv, int tok, int page) {
  tok = min(tok, s.last_tok);
  return (int64_t)page * kv.page_stride + (int64_t)(tok - page_slot(s, tok) * s.page_size) * kv.tok_stride;
}

// Threads 0..127 stage K (one half row each), threads 128..255 stage V (8 tokens x 8 dims each).
template <bool FP8, bool UNIFORM>
__device__ __forceinline__ void tile_gload(Stage<FP8>& st, const TileSrc& s, const KvAddr& kv, const char* kh,
                                           const char* vh, int tb, int tid, const PageIds<UNIFORM>& pg) {
  if (tid < 128) {
    const int tl = tid >> 1, half = tid & 1;
    const char* p = kh + row_offset(s, kv, tb + tl, pg.id[0]) + half * (FP8 ? 64 : 128);
#pragma unroll
    for (int i = 0; i < (FP8 ? 4 : 8); ++i) st.r[i] = ld16(p + i * 16);
  } else {
    const int u = tid - 128;
    const int tg = u & 7, dc = u >> 3;
    if constexpr (FP8) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const u32x2_t w = ld8(vh + row_offset(s, kv, tb + vt_token(tg, i), pg.id[UNIFORM ? 0 : i]) + dc * 8);
        st.r[i >> 1][(i & 1) * 2 + 0] = w[0];
        st.r[i >> 1][(i & 1) * 2 + 1] = w[1];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        st.r[i] = ld16(vh + row_offset(s, kv, tb + vt_token(tg, i), pg.id[UNIFORM ? 0 : i]) + dc * 16);
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

template <bool FP8, bool UNIFORM, bool CAP>
__global__ __launch_bounds__(256, 2) void rpa_prefill_flash_kernel(const PrefillArgs a, int tiles, int nseq) {
  // two tile buffers: tile t+1 is written while tile t is read, one barrier per tile
  __shared__ __attribute__((aligned(16))) char lds_k_buf[2][kBN * kKPitch];
  __shared__ __attribute__((aligned(16))) char lds_v_buf[2][128 * kVPitch];

  // ---- work decomposition ----
  // A unit is one (sequence, kv head): its G query heads and all their query tiles read the
  // same K/V, so a unit stays on one XCD (one L2).  Hardware deals workgroup n to XCD n % 8;
  // XCD x owns units x, x+8, ...: units of one sequence cost the same, so the XCDs stay
  // balanced whatever the ragged lengths are.  Inside an XCD, late (long, causal) query
  // tiles of every unit are issued first and the G heads of a unit sit next to each other.
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
  if (u >= units || tile_rev >= tiles) return;
  const int qt = tiles - 1 - tile_rev;
  const int si = u / a.Hkv;
  const int hk = u - si * a.Hkv;
  const int head = hk * a.G + gi;
  const int seq = a.seq_begin + si;
  const int qg0 = a.pt.cu_q_lens[seq];
  const int q_len = a.pt.cu_q_lens[seq + 1] - qg0;
  const int q_start = qt * kBM;
  if (q_start >= q_len) return;
  const int kv_len = a.pt.kv_lens[seq];
  const int prefix = kv_len - q_len;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5;

  TileSrc src;
  src.page_size = a.pt.page_size;
  src.page_shift = ((src.page_size & (src.page_size - 1)) == 0) ? (31 - __builtin_clz(src.page_size)) : -1;
  src.last_tok = kv_len - 1;
  src.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / a.pt.page_size)
                                                  : (int64_t)seq * a.pt.pages_per_seq);
  const char* kh = a.kv.k_base + (int64_t)hk * a.kv.head_stride;
  const char* vh = a.kv.v_base + (int64_t)hk * a.kv.head_stride;

  // ---- this wave's query rows ----
  const int r_lo = q_start + wave * 32;
  const int r_hi = min(r_lo + 31, q_len - 1);
  const bool wave_active = r_lo < q_len;
  const int row = r_lo + c;
  const int qpos = prefix + row;  // position of this lane's query inside the sequence
  const int W_ = a.sm.window;

  u32x4_t qB[8];
  {
    const int rr = min(row, q_len - 1);
    const uint16_t* qp = a.q + ((int64_t)(qg0 + rr) * a.Hq + head) * 128 + h * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qB[ks] = ld16(qp + ks * 16);
  }

  const float ksc = a.k_scale ? a.k_scale[hk] : 1.0f;
  const float scale = a.sm.sm_scale * ksc;
  const float scale2 = scale * kLog2e;
  const float cap = a.sm.soft_cap;
  const float inv_cap = (cap != 0.f) ? 1.0f / cap : 0.f;
  const float mask2 = fmaxf(a.sm.mask_value * kLog2e, -3.0e38f);

  f32x16_t O[4];
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) O[d][v] = 0.f;
  float m = -INFINITY, l = 0.f;

  // ---- kv tile range of the workgroup ----
  const int wg_r_hi = min(q_start + kBM, q_len) - 1;
  const int t_hi = min(kv_len, prefix + wg_r_hi + 1);  // exclusive
  int t_lo = 0;
  if (W_ > 0) t_lo = max(0, prefix + q_start - W_ + 1) & ~(kBN - 1);

  // ---- pipeline: page ids run two tiles ahead, rows one tile ahead (in registers), LDS one
  // tile ahead of the MFMAs.  Loads past the last tile re-read the last valid token.
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

    // visible to this wave?  causal: some token <= last row's position; window: some token
    // newer than the first row's horizon
    const bool vis = wave_active && (tb <= prefix + r_hi) && (W_ <= 0 || tb + kBN - 1 > prefix + r_lo - W_);
    if (vis) {
    const bool need_mask = (tb + kBN - 1 > prefix + r_lo) || (W_ > 0 && tb <= prefix + r_hi - W_);

    f32x16_t S[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int v = 0; v < 16; ++v) S[mt][v] = 0.f;
      const char* kp = lds_k + (mt * 32 + c) * kKPitch + h * 16;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) S[mt] = mfma32(lds_ld16(kp + ks * 32), qB[ks], S[mt]);
    }
    // scores -> log2 units
    if constexpr (CAP) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v) S[mt][v] = soft_cap_f(S[mt][v] * scale, cap, inv_cap) * kLog2e;
    } else {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v) S[mt][v] *= scale2;
    }
    uint32_t mbits = 0;  // bit (mt*16+v) set => masked
    if (need_mask) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int tok = tb + mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
          const bool masked = (tok > qpos) || (W_ > 0 && tok <= qpos - W_);
          if (masked) {
            S[mt][v] = mask2;
            mbits |= 1u << (mt * 16 + v);
          }
        }
    }
    float mx = S[0][0];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, S[mt][v]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2(m - m_new);
    float ps = 0.f;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float p = fast_exp2(S[mt][v] - m_new);
        if (need_mask && ((mbits >> (mt * 16 + v)) & 1u)) p = 0.f;
        S[mt][v] = p;
        ps += p;
      }
    l = l * alpha + ps;
    m = m_new;
    // the running max rarely moves once a few tiles are in: rescale only if some lane needs it
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) O[d][v] *= alpha;
    }
    u32x4_t pB[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
        pB[mt][kk] = u32x4_t{pack_bf16x2(S[mt][8 * kk + 0], S[mt][8 * kk + 1]),
                             pack_bf16x2(S[mt][8 * kk + 2], S[mt][8 * kk + 3]),
                             pack_bf16x2(S[mt][8 * kk + 4], S[mt][8 * kk + 5]),
                             pack_bf16x2(S[mt][8 * kk + 6], S[mt][8 * kk + 7])};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const char* vp = lds_v + (d * 32 + c) * kVPitch + h * 16;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
          O[d] = mfma32(lds_ld16(vp + (mt * 32 + kk * 16) * 2), pB[mt][kk], O[d]);
    }
    }  // vis
    __syncthreads();
  }

  // ---- epilogue: lane (c, h) holds query row c, dims 32d + 8*(v/4) + 4h + v%4 ----
  l += __shfl_xor(l, 32);
  if (!wave_active || row >= q_len) return;
  const float vs = a.v_scale ? a.v_scale[hk] : 1.0f;
  const float inv = vs / l;
  uint16_t* op = a.out + ((int64_t)(qg0 + row) * a.Hq + head) * 128 + 4 * h;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      u32x2_t w = {pack_bf16x2(O[d][4 * vq + 0] * inv, O[d][4 * vq + 1] * inv),
                   pack_bf16x2(O[d][4 * vq + 2] * inv, O[d][4 * vq + 3] * inv)};
      *reinterpret_cast<u32x2_t*>(op + d * 32 + vq * 8) = w;
    }
}

}  // namespace

hipError_t launch_prefill(const PrefillArgs& a, hipStream_t stream) {
  const int nseq = a.seq_end - a.seq_begin;
  if (nseq <= 0 || a.max_q_len <= 0) return hipSuccess;
  const int tiles = (a.max_q_len + kBM - 1) / kBM;
  const int64_t units = (int64_t)nseq * a.Hkv;
  const int64_t grid = (units >= 8 ? ((units + 7) / 8) * 8 : units) * a.G * tiles;
  if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool uniform = (a.pt.page_size % kBN) == 0;
  const bool cap = a.sm.soft_cap != 0.f;
  const dim3 g((unsigned)grid), blk(256);
#define RPA_PREFILL_LAUNCH(F, U, C) \
  hipLaunchKernelGGL((rpa_prefill_flash_kernel<F, U, C>), g, blk, 0, stream, a, tiles, nseq)
  switch ((a.fp8 ? 4 : 0) | (uniform ? 2 : 0) | (cap ? 1 : 0)) {
    case 0: RPA_PREFILL_LAUNCH(false, false, false); break;
    case 1: RPA_PREFILL_LAUNCH(false, false, true); break;
    case 2: RPA_PREFILL_LAUNCH(false, true, false); break;
    case 3: RPA_PREFILL_LAUNCH(false, true, true); break;
    case 4: RPA_PREFILL_LAUNCH(true, false, false); break;
    case 5: RPA_PREFILL_LAUNCH(true, false, true); break;
    case 6: RPA_PREFILL_LAUNCH(true, true, false); break;
    default: RPA_PREFILL_LAUNCH(true, true, true); break;
  }
#undef RPA_PREFILL_LAUNCH
  return hipGetLastError();
}

}  // namespace rpa
