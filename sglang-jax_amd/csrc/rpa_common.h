// Shared device helpers for the gfx950 ragged paged attention kernels.
//
// Wavefront = 64 lanes.  Matrix work uses the CDNA4 bf16 MFMA instructions
//   v_mfma_f32_16x16x32_bf16 : A[16x32] B[32x16] -> C[16x16] f32
//   v_mfma_f32_32x32x16_bf16 : A[32x16] B[16x32] -> C[32x32] f32
// with the operand layouts (lane l, c = l % 16, g = l / 16):
//   16x16x32  A: row c, k = 8g..8g+7     B: col c, k = 8g..8g+7
//             C: col c, rows 4g..4g+3 in the 4 result registers
//   32x32x16  (c = l % 32, h = l / 32)
//             A: row c, k = 8h..8h+7     B: col c, k = 8h..8h+7
//             C: col c, rows 8*(v/4) + 4h + (v%4) in result register v = 0..15
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rpa {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kDefaultMaskValue = -0.7f * 3.4028234663852886e38f;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2_t f = {lo, hi};
  bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
  return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ float bf16_lo_to_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi_to_f32(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

__device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// cap * tanh(x / cap) = cap - 2 cap / (e^(2x/cap) + 1), written so that +-inf arguments give +-cap: one
// multiply, v_exp_f32, one add, v_rcp_f32 (1 ulp; an IEEE division here is ten instructions per score), one fma.
__device__ __forceinline__ float soft_cap_f(float x, float cap, float inv_cap) {
  const float e = fast_exp2(x * (2.0f * kLog2e * inv_cap));
  return __builtin_fmaf(__builtin_amdgcn_rcpf(e + 1.0f), -2.0f * cap, cap);
}

// Temperature factor of a query at position qpos (ragged_paged_attention_v3.py:171-177):
// log2(qpos) / log2(T) beyond position T, 1 before.
__device__ __forceinline__ float xai_factor(int qpos, float xai_len) {
  if (!(xai_len > 0.f)) return 1.0f;
  return ((float)qpos > xai_len) ? __log2f((float)qpos) / __log2f(xai_len) : 1.0f;
}

__device__ __forceinline__ float bf16_round(float x) { return bf16_lo_to_f32(pack_bf16x2(x, 0.f)); }

__device__ __forceinline__ float f16_round(float x) { return (float)(_Float16)x; }

// a logit rounded to the softmax dtype: 1 = bf16, 2 = f16 (0, no rounding, is handled by the callers)
__device__ __forceinline__ float round_logit(float x, int mode) { return mode == 1 ? bf16_round(x) : f16_round(x); }

// the sink logit of a query head, rounded like the other logits when rounding is on
__device__ __forceinline__ float sink_logit(const float* sink, int round_logits, int head) {
  const float s = sink[head];
  return round_logits ? round_logit(s, round_logits) : s;
}

// Queries divided by q_scale and rounded to the cache's element type
// (ragged_paged_attention_v3.py:463-470: the quotient is a bf16 array, clipped to the fp8
// range and cast when the cache holds fp8).  Eight bf16 values in, eight out.
__device__ __forceinline__ u32x4_t requantise_q(u32x4_t q, float q_scale, bool to_fp8) {
  u32x4_t r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float lo = bf16_round(bf16_lo_to_f32(q[i]) / q_scale);
    float hi = bf16_round(bf16_hi_to_f32(q[i]) / q_scale);
    if (to_fp8) {
      lo = fminf(fmaxf(lo, -448.0f), 448.0f);
      hi = fminf(fmaxf(hi, -448.0f), 448.0f);
      const uint32_t b = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, 0, false);
      const f32x2_t f = __builtin_amdgcn_cvt_pk_f32_fp8(b, false);
      lo = f[0];
      hi = f[1];
    }
    r[i] = pack_bf16x2(lo, hi);
  }
  return r;
}

// Softmax denominator with an attention sink: given the running maximum m2 (log2 units), the
// sum l of 2^(x - m2) and a sink logit (natural units), returns the factor that turns the
// unnormalised output into out = sum p v / (sum p + e^sink)
// (ragged_paged_attention_v3.py:185-196: the sink is a logit column dropped after softmax).
__device__ __forceinline__ float sink_inverse(float m2, float l, float sink) {
  const float s2 = sink * kLog2e;
  const float mm = fmaxf(m2, s2);
  const float w = __builtin_amdgcn_exp2f(m2 - mm);
  return w / (l * w + __builtin_amdgcn_exp2f(s2 - mm));
}

// Load a 32-bit word through the scalar data cache.  `p` must be wave-uniform and point at
// memory nobody writes during the kernel (page tables, lengths).  A scalar load is counted by
// lgkmcnt, not vmcnt, so waiting for it never drains the vector-memory queue.
__device__ __forceinline__ int32_t scalar_load_i32(const int32_t* p) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(a));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(a >> 32));
  typedef const __attribute__((address_space(4))) int32_t* const_ptr_t;
  return *reinterpret_cast<const_ptr_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Asynchronous 16-byte copy global -> LDS (global_load_lds_dwordx4): lane l's 16 bytes land at
// lds_base + 16*l; the data never touches a VGPR and completion is counted by vmcnt.  Issued as
// inline assembly so that the compiler does not model it as an LDS store: it would otherwise
// wait for ALL outstanding copies (vmcnt(0)) in front of every LDS read it cannot disambiguate,
// which destroys a multi-tile prefetch.  The caller waits with s_waitcnt vmcnt(n) itself.
__device__ __forceinline__ void async_copy16(const void* gsrc, const void* lds_base_uniform) {
  typedef const __attribute__((address_space(3))) char* lds_ptr_t;
  const uint32_t m0v = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)lds_base_uniform));
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(gsrc) : "memory", "m0");
}

// 16-byte global loads / stores.
__device__ __forceinline__ u32x4_t ld16(const void* p) { return *reinterpret_cast<const u32x4_t*>(p); }
__device__ __forceinline__ u32x2_t ld8(const void* p) { return *reinterpret_cast<const u32x2_t*>(p); }
__device__ __forceinline__ void st16(void* p, u32x4_t v) { *reinterpret_cast<u32x4_t*>(p) = v; }

// Two fp8-e4m3 bytes (low or high half of `w`) -> two f32.
__device__ __forceinline__ f32x2_t fp8x2_to_f32(uint32_t w, bool hi) {
  return hi ? __builtin_amdgcn_cvt_pk_f32_fp8(w, true) : __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
}

// Two fp8-e4m3 bytes (low or high half of `w`) -> two bf16 in one dword, one instruction
// (v_cvt_scalef32_pk_bf16_fp8 with scale 1; exact: e4m3 fits bf16).
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t w, bool hi) {
  const bf16x2_t r = hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)
                        : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
  return __builtin_bit_cast(uint32_t, r);
}

// Four fp8-e4m3 bytes -> four bf16 packed in two dwords (exact: e4m3 fits bf16).
__device__ __forceinline__ u32x2_t fp8x4_to_bf16x4(uint32_t w) {
  return u32x2_t{fp8x2_to_bf16x2(w, false), fp8x2_to_bf16x2(w, true)};
}

// A window of consecutive page ids of a row, copied asynchronously into a wave's own LDS slice
// (global_load_lds_dword, no register in between): 64 ids per copy instruction, entry i = page slot
// first_slot + i, clamped to the row's last page.  The copy is issued as inline assembly and its completion
// is the caller's business: loads complete in order, so it has landed once any load issued after it has been
// waited for.
constexpr int kWinSmallPages = 256;  // entries of a window when pages are smaller than a block

template <int ENTRIES>
__device__ __forceinline__ void copy_page_window(const int32_t* row_pages, int last_slot, int32_t* lds, int first_slot,
                                                 int lane) {
  typedef const __attribute__((address_space(3))) char* lds_ptr_t;
  const uint32_t base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)lds));
#pragma unroll
  for (int k = 0; k < ENTRIES / 64; ++k) {
    const int32_t* src = row_pages + min(first_slot + 64 * k + lane, last_slot);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(base + 256u * k), "v"(src) : "memory", "m0");
  }
}

__device__ __forceinline__ void wait_all_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

}  // namespace rpa
