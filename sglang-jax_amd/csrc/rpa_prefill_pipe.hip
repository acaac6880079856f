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
// the pair of iterations (2t-1, 2t): it reads K tile t and V tile t-1, so the two-slot rings of
// the unpipelined kernel suffice (V lags K by one tile) and there is still one barrier per tile.
//
// The running maximum is checked after the fact: the exponentials of half i use the maximum known
// before it; the half's own maximum is taken by the vector pipe next to them, and only if it
// exceeds the stale one by more than 2^kMaxSlack is the half redone (its scores are still in
// registers) and the accumulators rescaled.  Halves that touch the causal diagonal or a window
// edge, the first and the last steps run the same pipeline through a general iteration with
// masking and run-time flags.

#include "rpa_prefill_common.h"

namespace rpa {

using namespace pf;

namespace {

constexpr int kRowB = 256;               // bytes of one K or V row of a head
constexpr int kTileB = kBN * kRowB;      // 16 KiB
constexpr int kHalfB = 32 * kRowB;       // byte distance between the halves of a tile

struct PipeState {
  f32x16_t O[4];
  float m, l;
  float sc2;
};

// one matrix copy (K or V rows of a tile) global -> LDS: 4 instructions per wave
template <bool IS_V>
__device__ __forceinline__ void copy_rows(char* lds, const TileSrc& s, const KvAddr& kv, const char* head, int tb,
                                          int wave, int lane, int page, const AsyncOffsets<128>& ofs) {
  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  tb = min(tb, s.last_tok & ~(kBN - 1));
  if (tb + kBN - 1 <= s.last_tok) {
    const int64_t base = (int64_t)page * kv.page_stride + (int64_t)(tb - page_slot(s, tb) * s.page_size) * kv.tok_stride;
    const char* b = head + base;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int blk = wave * 4 + n;
      __builtin_amdgcn_global_load_lds((gptr_t)(b + (IS_V ? ofs.v[n] : ofs.k[n])), (lptr_t)(lds + blk * 1024), 16, 0, 0);
    }
    return;
  }
  const int cp = lane & 15;
#pragma unroll
  for (int n = 0; n < 4; ++n) {
    const int blk = wave * 4 + n;
    const int t = blk * 4 + (lane >> 4);
    const int64_t ro = row_offset<true>(s, kv, tb, tb + t, page);
    const int j = IS_V ? (cp ^ ((t & 3) << 2)) : (cp ^ (t & 15));
    __builtin_amdgcn_global_load_lds((gptr_t)(head + ro + j * 16), (lptr_t)(lds + blk * 1024), 16, 0, 0);
  }
}

__device__ __forceinline__ int scalar_page(const TileSrc& s, int tb) {
  tb = min(tb, s.last_tok & ~(kBN - 1));
  return scalar_load_i32(s.pages + __builtin_amdgcn_readfirstlane(page_slot(s, tb)));
}

// first product of one 32-token half: one chain of 8 MFMAs
__device__ __forceinline__ f32x16_t qk_half(const char* lds_k_half, const int (&koff)[8], const u32x4_t (&qB)[8]) {
  f32x16_t S = mfma32(lds_ld16(lds_k_half + koff[0]), qB[0], kZero16);
#pragma unroll
  for (int ks = 1; ks < 8; ++ks) S = mfma32(lds_ld16(lds_k_half + koff[ks]), qB[ks], S);
  return S;
}

// second product of one 32-token half: four chains of 2 MFMAs
__device__ __forceinline__ void pv_half(f32x16_t (&O)[4], const char* lds_v_half, const int (&voff)[4],
                                        const u32x4_t (&P)[2]) {
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const char* vt = lds_v_half + voff[d] + kk * 16 * kRowB;
      const u32x2_t lo = lds_tr16(vt);
      const u32x2_t hi = lds_tr16(vt + 8 * kRowB);
      O[d] = mfma32(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, P[kk], O[d]);
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

// raise the running maximum to cover mx and rescale what has been accumulated
__device__ __forceinline__ void raise_max(PipeState& st, float mx) {
  const float m_new = fmaxf(st.m, mx);
  const float alpha = fast_exp2((st.m - m_new) * st.sc2);
  st.m = m_new;
  st.l *= alpha;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) st.O[d][v] *= alpha;
}

// softmax of a half with the maximum taken first (first half of a row, masked halves)
__device__ __forceinline__ void softmax_half_general(f32x16_t& S, PipeState& st, bool need_mask, int tb, int h, int qpos,
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
  if (__builtin_amdgcn_ballot_w64((mx - st.m) * st.sc2 > kMaxSlack) != 0) raise_max(st, mx);
  st.l += exp_pack(S, st.sc2, -st.m * st.sc2, P);
}

template <bool WIN>
__global__ __launch_bounds__(256, 2) void rpa_prefill_pipe_kernel(const PrefillArgs a, int tiles, int nseq, bool by_level) {
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
  const int W_ = WIN ? a.sm.window : 0;

  u32x4_t qB[8];
  {
    const int rr = min(wr.row, w.q_len - 1);
    const uint16_t* qp = a.q + ((int64_t)(w.qg0 + rr) * a.Hq + w.head) * 128 + h * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qB[ks] = ld16(qp + ks * 16);
  }
  PipeState st;
  st.sc2 = a.sm.sm_scale * (a.k_scale ? a.k_scale[w.hk] : 1.0f) * kLog2e;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) st.O[d][v] = 0.f;
  st.m = kMaxFloor;
  st.l = 0.f;

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

  // operand offsets inside a tile (see rpa_prefill_async_kernel)
  const int k_row = c * kRowB;
  const int k_swz = (h ^ (c & 15)) << 4;
  const int r16 = lane & 15, b16 = lane >> 4;
  const int v_row = (4 * h + (r16 >> 2)) * kRowB;
  const int v_in = ((b16 & 1) << 5) + (((r16 & 3) >> 1) << 4) + ((r16 & 1) << 3);
  const int v_swz = (r16 >> 2) << 6;
  int koff[8], voff[4];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    koff[ks] = k_row + ((ks * 32) ^ k_swz);
    asm volatile("" : "+v"(koff[ks]));
  }
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    voff[d] = v_row + v_in + ((d * 64) ^ v_swz);
    asm volatile("" : "+v"(voff[d]));
  }

  const AsyncOffsets<128> ofs = make_async_offsets<128>(a.kv, wave, lane);
  int pg_a = scalar_page(src, t_lo);         // page of tile t
  copy_rows<false>(lds_k0, src, a.kv, kh, t_lo, wave, lane, pg_a, ofs);
  int pg_b = scalar_page(src, t_lo + kBN);   // page of tile t + 1
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  // pipeline registers: scores of half i in S[i & 1], its probabilities in P[i & 1]
  f32x16_t S0 = kZero16, S1 = kZero16;
  u32x4_t P0[2] = {}, P1[2] = {};

  // iteration i of the general kind: Sn <- scores of half i + 1, Pc <- softmax of Sc (half i), O += P(i - 1) V
  auto general_iter = [&](int i, f32x16_t& Sc, f32x16_t& Sn, u32x4_t (&Pc)[2], const u32x4_t (&Pp)[2],
                          const char* lds_k_half, const char* lds_v_half) __attribute__((always_inline)) {
    if (i + 1 < n_w) Sn = qk_half(lds_k_half, koff, qB);
    if (i >= 1 && i - 1 < n_w) pv_half(st.O, lds_v_half, voff, Pp);
    if (i >= 0 && i < n_w) {
      const bool need_mask = i < i_f0 || i >= i_f1;
      softmax_half_general(Sc, st, need_mask, t_lo + 32 * i, h, wr.qpos, W_, Pc);
    }
  };

  // iteration i of the fast kind: no mask, every part present, maximum checked afterwards.  The
  // source order is the intended issue order (one matrix instruction, then the vector work of one
  // score pair); the group barriers at the end pin it.
  auto fast_iter = [&](f32x16_t& Sc, f32x16_t& Sn, u32x4_t (&Pc)[2], const u32x4_t (&Pp)[2], const char* lds_k_half,
                       const char* lds_v_half) __attribute__((always_inline)) {
    const float neg_m = -st.m * st.sc2;
    const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
    float ps0 = 0.f, ps1 = 0.f;
    float mx = Sc[0];
    uint32_t w[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      // first product, k-step k
      Sn = mfma32(lds_ld16(lds_k_half + koff[k]), qB[k], k == 0 ? kZero16 : Sn);
      // second product: k-step k / 4 of dim tile k % 4
      {
        const char* vt = lds_v_half + voff[k & 3] + (k >> 2) * 16 * kRowB;
        const u32x2_t lo = lds_tr16(vt);
        const u32x2_t hi = lds_tr16(vt + 8 * kRowB);
        st.O[k & 3] = mfma32(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, Pp[k >> 2], st.O[k & 3]);
      }
      // softmax of score pair k
      const float p0 = fast_exp2(__builtin_fmaf(Sc[2 * k], st.sc2, neg_m));
      const float p1 = fast_exp2(__builtin_fmaf(Sc[2 * k + 1], st.sc2, neg_m));
      w[k] = pack_bf16x2(p0, p1);
      if (k & 1) ps1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[k]), ones, ps1, false);
      else ps0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w[k]), ones, ps0, false);
      mx = k == 0 ? __builtin_fmaxf(mx, Sc[1]) : __builtin_fmaxf(__builtin_fmaxf(mx, Sc[2 * k]), Sc[2 * k + 1]);
    }
    Pc[0] = u32x4_t{w[0], w[1], w[2], w[3]};
    Pc[1] = u32x4_t{w[4], w[5], w[6], w[7]};
    mx = swap_max(mx);
    float ps = ps0 + ps1;
    // the probabilities are final here in all but rare cases: keep them from being sunk behind the branch
    asm volatile("" : "+v"(Pc[0]), "+v"(Pc[1]), "+v"(ps));
    const bool raise = __builtin_amdgcn_ballot_w64((mx - st.m) * st.sc2 > kMaxSlack) != 0;
#define RPA_PIPE_GROUP(LDS_A, LDS_B)                                                        \
  __builtin_amdgcn_sched_group_barrier(0x100, LDS_A, 0); /* LDS reads run ahead */          \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     /* MFMA of the first product */    \
  __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);                                        \
  __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);                                        \
  __builtin_amdgcn_sched_group_barrier(0x100, LDS_B, 0);                                    \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     /* MFMA of the second product */   \
  __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);                                        \
  __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
    RPA_PIPE_GROUP(6, 3)
    RPA_PIPE_GROUP(3, 3)
    RPA_PIPE_GROUP(3, 3)
    RPA_PIPE_GROUP(3, 0)
    RPA_PIPE_GROUP(0, 0)
    RPA_PIPE_GROUP(0, 0)
    RPA_PIPE_GROUP(0, 0)
    RPA_PIPE_GROUP(0, 0)
#undef RPA_PIPE_GROUP
    if (raise) {
      asm volatile("" ::: "memory");  // keep the rescale out of the common path
      raise_max(st, mx);
      st.l += exp_pack(Sc, st.sc2, -st.m * st.sc2, Pc);
    } else {
      st.l += ps;
    }
  };

  // step t: iterations 2t - 1 and 2t; reads K tile t from (ck) and V tile t - 1 from (cv), fills the
  // other K slot with tile t + 1 and the other V slot with tile t
  auto step = [&](int t, const char* ck, const char* cv, char* fk, char* fv) __attribute__((always_inline)) {
    if (t + 1 < nT) copy_rows<false>(fk, src, a.kv, kh, t_lo + (t + 1) * kBN, wave, lane, pg_b, ofs);
    if (t < nT) copy_rows<true>(fv, src, a.kv, vh, t_lo + t * kBN, wave, lane, pg_a, ofs);
    pg_a = pg_b;
    if (t + 2 < nT) pg_b = scalar_page(src, t_lo + (t + 2) * kBN);
    const int i = 2 * t - 1;
    if (i >= max(i_f0, 1) && i + 1 < i_f1) {
      fast_iter(S1, S0, P1, P0, ck, cv);
      fast_iter(S0, S1, P0, P1, ck + kHalfB, cv + kHalfB);
    } else {
      general_iter(i, S1, S0, P1, P0, ck, cv);
      general_iter(i + 1, S0, S1, P0, P1, ck + kHalfB, cv + kHalfB);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  };

  for (int t = 0; t <= nT; t += 2) {
    step(t, lds_k0, lds_v1, lds_k1, lds_v0);
    if (t + 1 > nT) break;
    step(t + 1, lds_k1, lds_v0, lds_k0, lds_v1);
  }
  write_rows<4>(a, w, wr, st.O, st.l, h, st.m * st.sc2);
}

}  // namespace

bool prefill_pipe_applies(const PrefillArgs& a) {
  return !a.fp8 && a.head_dim == 128 && (a.pt.page_size % kBN) == 0 && a.sm.mask_mode == 0 && a.sm.soft_cap == 0.f &&
         a.sm.round_logits == 0 && !(a.sm.xai_len > 0.f) && !(a.sm.q_scale > 0.f);
}

hipError_t launch_prefill_pipe(const PrefillArgs& a, int tiles, int nseq, bool by_level, unsigned grid, hipStream_t stream) {
  const dim3 g(grid), blk(256);
  if (a.sm.window > 0) hipLaunchKernelGGL((rpa_prefill_pipe_kernel<true>), g, blk, 0, stream, a, tiles, nseq, by_level);
  else hipLaunchKernelGGL((rpa_prefill_pipe_kernel<false>), g, blk, 0, stream, a, tiles, nseq, by_level);
  return hipGetLastError();
}

}  // namespace rpa
