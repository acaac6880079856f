// Absorbed-MLA split-KV decode on gfx950.
//
// Every token has ONE shared latent row [kv_c (512) | k_pe (64)]; all query
// heads attend to it (scores over 576 dims, values = the first 512 dims).  A
// workgroup of 8 waves owns one (sequence, kv split) and ALL heads in groups of
// 128 (wave w owns 16 heads), so the latent rows are fetched from HBM once:
//   global -> registers -> LDS      K tile [32 tok][576]        (pitch 1168 B)
//   LDS -> registers -> LDS         V^T tile [512 dims][32 tok] (pitch 80 B),
//                                   register transpose with v_perm_b32
//   S^T[tok, head] = K . Q^T        36 MFMA 16x16x32 per wave and tile
//   online softmax, P rounded to bf16 (as the reference rounds it)
//   O^T[dim, head] += V^T . P^T     32 MFMA 16x16x32 per wave and tile
// Partials (unnormalised O, running max, sum) go to the workspace and are merged
// by rpa_mla_combine_kernel; with a single split the output is written directly.

#include "rpa_common.h"
#include "rpa_kernels.h"

namespace rpa {

namespace {

constexpr int kTok = 32;         // tokens per tile
constexpr int kRowB = 1152;      // compact latent row bytes (576 bf16)
constexpr int kKPitch = 1168;    // LDS pitch of a K row
constexpr int kVPitch = 80;      // LDS pitch of a V^T row (32 tok * 2 B + 16)
constexpr int kPieces = kTok * 72;  // 16-byte pieces per tile

__device__ __forceinline__ u32x4_t lds_ld16(const char* p) { return *reinterpret_cast<const u32x4_t*>(p); }
__device__ __forceinline__ void lds_st16(char* p, u32x4_t v) { *reinterpret_cast<u32x4_t*>(p) = v; }

__device__ __forceinline__ int tok_slot(int g, int i) {
  return (i < 4) ? (g * 4 + i) : (16 + g * 4 + (i - 4));
}

struct Src {
  const int32_t* pages;
  int32_t page_size, page_shift, last_tok;
  int64_t page_stride;  // bytes
  int32_t row_bytes;    // bytes between tokens of a page
  int32_t rope_byte;    // byte offset of k_pe inside a cached row
};

__device__ __forceinline__ u32x4_t load_piece(const Src& s, const char* cache, int tb, int idx) {
  const int tl = idx / 72, piece = idx - tl * 72;
  const int tok = min(tb + tl, s.last_tok);
  const int slot = s.page_shift >= 0 ? (tok >> s.page_shift) : (tok / s.page_size);
  const int page = s.pages[slot];
  const int inner = piece < 64 ? piece * 16 : s.rope_byte + (piece - 64) * 16;
  return ld16(cache + (int64_t)page * s.page_stride + (int64_t)(tok - slot * s.page_size) * s.row_bytes + inner);
}

// grid = (max_splits, rows, head groups of 128); block = 512 threads.
__global__ __launch_bounds__(512, 2) void rpa_mla_decode_kernel(const MlaDecodeArgs a) {
  __shared__ __attribute__((aligned(16))) char lds_k[kTok * kKPitch];
  __shared__ __attribute__((aligned(16))) char lds_v[512 * kVPitch];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int seq = blockIdx.y, split = blockIdx.x;
  const int head0 = blockIdx.z * 128 + wave * 16;
  const bool wave_on = head0 < a.Hq;

  const int kv_len = a.pt.kv_lens[seq];
  const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
  const int t0 = t_lo & ~(kTok - 1);
  const int t_begin = t0 + split * a.chunk;
  if (t_begin >= kv_len) return;
  const int t_end = (split == a.max_splits - 1) ? kv_len : min(kv_len, t_begin + a.chunk);

  Src src;
  src.page_size = a.pt.page_size;
  src.page_shift = ((src.page_size & (src.page_size - 1)) == 0) ? (31 - __builtin_clz(src.page_size)) : -1;
  src.last_tok = kv_len - 1;
  src.pages = a.pt.page_indices + (a.pt.cu_kv_lens ? (a.pt.cu_kv_lens[seq] / a.pt.page_size)
                                                  : (int64_t)seq * a.pt.pages_per_seq);
  src.row_bytes = a.row_stride * 2;
  src.page_stride = (int64_t)src.row_bytes * a.pt.page_size;
  src.rope_byte = a.rope_offset * 2;

  // ---- Q^T operands of this wave: column c = head head0 + c, k-step ks covers dims 32ks + 8g .. ----
  const int tq = a.pt.cu_q_lens[seq];
  u32x4_t qB[18];
  {
    const int head = min(head0 + c, a.Hq - 1);
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

  f32x4_t acc[32];
#pragma unroll
  for (int j = 0; j < 32; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  u32x4_t stg[5];
#pragma unroll
  for (int r = 0; r < 5; ++r) {
    const int idx = tid + r * 512;
    if (idx < kPieces) stg[r] = load_piece(src, a.cache, t_begin, idx);
  }

  for (int tb = t_begin; tb < t_end; tb += kTok) {
    __syncthreads();  // previous tile fully consumed
#pragma unroll
    for (int r = 0; r < 5; ++r) {
      const int idx = tid + r * 512;
      if (idx < kPieces) {
        const int tl = idx / 72, piece = idx - tl * 72;
        lds_st16(lds_k + tl * kKPitch + piece * 16, stg[r]);
      }
    }
    __syncthreads();
    if (tb + kTok < t_end) {
#pragma unroll
      for (int r = 0; r < 5; ++r) {
        const int idx = tid + r * 512;
        if (idx < kPieces) stg[r] = load_piece(src, a.cache, tb + kTok, idx);
      }
    }
    // ---- transpose the value part: thread (tg, dc) turns 8 tokens x 8 dims into 8 dims x 8 tokens ----
    if (tid < 256) {
      const int tg = tid & 3, dc = tid >> 2;
      // two passes of 4 tokens keep only 16 staging registers live
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        u32x4_t v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = lds_ld16(lds_k + tok_slot(tg, half * 4 + i) * kKPitch + dc * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
          const int jj = j >> 1;
          const u32x2_t w = {__builtin_amdgcn_perm(v[1][jj], v[0][jj], sel), __builtin_amdgcn_perm(v[3][jj], v[2][jj], sel)};
          *reinterpret_cast<u32x2_t*>(lds_v + (dc * 8 + j) * kVPitch + tg * 16 + half * 8) = w;
        }
      }
    }
    __syncthreads();
    if (!wave_on) continue;

    f32x4_t s[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      s[b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const char* kp = lds_k + (b * 16 + c) * kKPitch + g * 16;
#pragma unroll
      for (int ks = 0; ks < 18; ++ks) s[b] = mfma16(lds_ld16(kp + ks * 64), qB[ks], s[b]);
    }
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = s[i >> 2][i & 3];
      if (cap != 0.f) v = soft_cap_f(v * scale, cap, inv_cap) * kLog2e;
      else v = v * scale2;
      x[i] = v;
    }
    if ((tb + kTok > kv_len) || (tb < t_lo)) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int tok = tb + tok_slot(g, i);
        if (tok >= kv_len || tok < t_lo) x[i] = mask2;
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
    const char* vp = lds_v + c * kVPitch + g * 16;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      acc[j] = acc[j] * alpha;
      acc[j] = mfma16(lds_ld16(vp + j * 16 * kVPitch), pB, acc[j]);
    }
  }

  // ---- epilogue: lane (c, g) holds head head0+c, dims 16j + 4g + r in acc[j][r] ----
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  const int head = head0 + c;
  if (!wave_on || head >= a.Hq) return;
  if (a.max_splits == 1) {
    const float inv = 1.0f / l;
    uint16_t* op = a.out + ((int64_t)tq * a.Hq + head) * 512 + g * 4;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      u32x2_t w = {pack_bf16x2(acc[j][0] * inv, acc[j][1] * inv), pack_bf16x2(acc[j][2] * inv, acc[j][3] * inv)};
      *reinterpret_cast<u32x2_t*>(op + j * 16) = w;
    }
  } else {
    const int64_t slot = ((int64_t)seq * a.max_splits + split) * a.Hq + head;
    float* wo = a.ws_o + slot * 512 + g * 4;
#pragma unroll
    for (int j = 0; j < 32; ++j) *reinterpret_cast<f32x4_t*>(wo + j * 16) = acc[j];
    if (g == 0) {
      a.ws_ml[slot * 2 + 0] = m;
      a.ws_ml[slot * 2 + 1] = l;
    }
  }
}

// grid = (Hq, rows); block = 128 threads, 4 dims each.
__global__ __launch_bounds__(128) void rpa_mla_combine_kernel(const MlaDecodeArgs a) {
  const int head = blockIdx.x, seq = blockIdx.y;
  const int kv_len = a.pt.kv_lens[seq];
  const int t_lo = (a.sm.window > 0) ? max(0, kv_len - a.sm.window) : 0;
  const int t0 = t_lo & ~(kTok - 1);
  const int n = min(a.max_splits, (kv_len - t0 + a.chunk - 1) / a.chunk);
  if (n <= 0) return;
  const int64_t base = ((int64_t)seq * a.max_splits) * a.Hq + head;
  float mstar = -INFINITY;
  for (int j = 0; j < n; ++j) mstar = fmaxf(mstar, a.ws_ml[(base + (int64_t)j * a.Hq) * 2]);
  float den = 0.f;
  f32x4_t o = {0.f, 0.f, 0.f, 0.f};
  const int d = threadIdx.x * 4;
  for (int j = 0; j < n; ++j) {
    const int64_t slot = base + (int64_t)j * a.Hq;
    const float w = fast_exp2(a.ws_ml[slot * 2] - mstar);
    den += a.ws_ml[slot * 2 + 1] * w;
    o += *reinterpret_cast<const f32x4_t*>(a.ws_o + slot * 512 + d) * w;
  }
  const float inv = 1.0f / den;
  const int tq = a.pt.cu_q_lens[seq];
  u32x2_t w = {pack_bf16x2(o[0] * inv, o[1] * inv), pack_bf16x2(o[2] * inv, o[3] * inv)};
  *reinterpret_cast<u32x2_t*>(a.out + ((int64_t)tq * a.Hq + head) * 512 + d) = w;
}

}  // namespace

hipError_t launch_mla_decode(const MlaDecodeArgs& a, hipStream_t stream) {
  if (a.num_rows <= 0) return hipSuccess;
  const int head_groups = (a.Hq + 127) / 128;
  hipLaunchKernelGGL(rpa_mla_decode_kernel, dim3(a.max_splits, a.num_rows, head_groups), dim3(512), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (a.max_splits > 1) {
    hipLaunchKernelGGL(rpa_mla_combine_kernel, dim3(a.Hq, a.num_rows), dim3(128), 0, stream, a);
    e = hipGetLastError();
  }
  return e;
}

}  // namespace rpa
