// Launch shapes by call shape: ONE table, first match wins.
//
// The reference keys its tile sizes (bq, bkv, bq_csz, bkv_csz) on (q dtype, kv dtype, heads, head dim, page
// size, token bucket, window, case) in a table of measured optima, falling back to a heuristic
// (kernels/ragged_paged_attention/tuned_block_sizes_v3.py:2163-2229; ragged_paged_attention_v3.py:1490-1638).
// The choices that exist on this GPU are different ones -- which kernel family, how many query positions and
// query heads a workgroup owns, how many waves walk neighbouring heads together, how many waves stay resident --
// and this table is their one home: every launcher selects its row here, rpa_describe_plan() prints it, and
// the RPA_* switches (rpa_tuning.h) only override a row's fields to repeat the measurements behind it.
// What varies continuously with the lengths of a batch (how many pieces a row or a K/V range is cut into) is
// computed from the row's fields by the planners in rpa_capi.hip (plan_splits, the balanced plans) and
// kv_pieces() (rpa_prefill_common.h).
#pragma once

#include <stdint.h>

namespace rpa {

enum ShapeStage : int { kStageDecode = 0, kStagePrefill = 1, kStageMla = 2 };

enum ShapeOption : unsigned {
  kOptSoftCap = 1u << 0,      // soft cap or logits rounded to the softmax dtype (the general score path)
  kOptMaskOther = 1u << 1,    // custom mask or no mask
  kOptTemperature = 1u << 2,  // xai temperature
  kOptQScale = 1u << 3,       // quantised queries
  kOptOddPages = 1u << 4,     // pages that do not hold whole K/V tiles of the stage (64 tokens; MLA: 32)
  kOptWidePages = 1u << 5,    // a page of 4 GiB or more (the assembly loops do 32-bit page arithmetic)
  kOptNotPow2Pages = 1u << 6, // page size that is no power of two (the assembly loops shift and mask)
};

enum ShapeKernel : int {
  kKernelDecode,          // rpa_decode_splitkv_kernel / rpa_decode_balanced_kernel (the plan picks)
  kKernelRows256,         // rpa_rows256_kernel
  kKernelPrefillPipe,     // rpa_prefill_pipe_kernel (assembly steady state)
  kKernelPrefillAsync,    // rpa_prefill_async_kernel (compiled, global -> LDS copies)
  kKernelPrefillStaged,   // rpa_prefill_staged_kernel (rows through registers: fp8 caches)
  kKernelMlaWide,         // rpa_mla_*_wide_kernel: four waves x 32 heads, every tile in the assembly loop
  kKernelMlaPipe,         // rpa_mla_*_kernel, eight waves x 16 heads, assembly steady state
  kKernelMlaShared,       // rpa_mla_*_kernel, the waves of a block of 16 heads share each tile
  kKernelMlaCompiled,     // rpa_mla_*_kernel, compiled tile loop
};

struct ShapeKey {
  ShapeStage stage;
  int kv_bits;       // 16 or 8
  int head_dim;      // 128 or 256; 576 for the absorbed-MLA latent row
  int heads;         // decode / prefill: query heads per kv head; MLA: query heads
  int max_q_len;     // prefill: bound on a chunk's length (<= 0: unknown, taken as long)
  int64_t kv_bytes;  // decode: bytes the rows will stream as far as the host knows
  unsigned options;  // ShapeOption bits
};

struct ShapeRule {
  const char* name;
  // ---- key ranges (0 = any)
  ShapeStage stage;
  int kv_bits;
  int head_dim;
  int heads_lo, heads_hi;  // inclusive
  int heads_multiple;
  int q_hi;                // matches max_q_len in [1, q_hi]
  int64_t bytes_lo;        // matches kv_bytes >= bytes_lo
  unsigned forbid;         // options the row cannot run
  // ---- the choice
  ShapeKernel kernel;
  int tile_q;              // query positions per workgroup (decode, MLA: 1 row)
  int tile_heads;          // query heads per workgroup (of one kv head; MLA: of the 128-head group)
  int tile_kv;             // K/V tokens per step
  int waves_per_wg;        // decode: neighbouring kv heads walked together; others: waves of a workgroup
  int resident_x8;         // decode: resident waves per CU in eighths (28 = 3.5); MLA: workgroups per CU x 8
  int share;               // MLA shared tiles: waves that share a block of 16 heads
  int piece_pad;           // MLA balanced plan: what starting one more row costs a workgroup, in 32-token tiles
  const char* why;         // the measurement behind the row
};

constexpr unsigned kOptAsmPages = kOptOddPages | kOptWidePages | kOptNotPow2Pages;
constexpr unsigned kOptPlainOnly = kOptSoftCap | kOptMaskOther | kOptTemperature | kOptQScale | kOptAsmPages;

// clang-format off
constexpr ShapeRule kShapeRules[] = {
  // ---------------- decode rows (HBM bound: bytes in flight and launch overhead decide)
  {"decode_256", kStageDecode, 0, 256, 0, 0, 0, 0, 0, 0,
   kKernelRows256, 1, 16, 32, 1, 64, 1, 0, "one wave per (token, kv head, 16 query heads); 5.9-6.15 TB/s on long rows"},
  {"decode_fp8_stream", kStageDecode, 8, 128, 0, 0, 0, 0, 32ll << 20, 0,
   kKernelDecode, 1, 16, 32, 4, 32, 1, 0, "non-temporal loads: one wave per SIMD; C4 768 waves 226.7 us, 1024 208.7, 1536 245.9, 2048 213.3 (plain loads: 1024 254, 2048 238.5)"},
  {"decode_fp8_small", kStageDecode, 8, 128, 0, 0, 0, 0, 0, 0,
   kKernelDecode, 1, 16, 32, 2, 64, 1, 0, "latency bound: few waves spread over more CUs"},
  {"decode_bf16_stream", kStageDecode, 16, 128, 0, 0, 0, 0, 32ll << 20, 0,
   kKernelDecode, 1, 16, 32, 4, 32, 1, 0, "non-temporal loads: one wave per SIMD; C2 / C3 768 waves 96.3 / 354.8 us, 896 90.5 / 326.2, 1024 89.3 / 316.0, 1280 117 / 431, 2048 95.1 / 332.1 (plain loads: 896 104.1 / 356)"},
  {"decode_bf16_small", kStageDecode, 16, 128, 0, 0, 0, 0, 0, 0,
   kKernelDecode, 1, 16, 32, 2, 28, 1, 0, "C1 14.0 us with two waves per workgroup against 15.9 with four"},
  // ---------------- prefill / mixed rows (MFMA bound)
  {"prefill_pipe_short", kStagePrefill, 16, 128, 0, 0, 4, 64, 0, kOptPlainOnly,
   kKernelPrefillPipe, 32, 4, 64, 4, 16, 1, 0, "chunks of <= 64 tokens fill a 32 x 4-head tile: 64 x 16 tokens on 4 k prefixes 362 -> 196 us"},
  {"prefill_pipe", kStagePrefill, 16, 128, 0, 0, 0, 0, 0, kOptPlainOnly,
   kKernelPrefillPipe, 128, 1, 64, 4, 16, 1, 0, "assembly steady state: C2 295 -> 236 us"},
  {"prefill_256_fp8", kStagePrefill, 8, 256, 0, 0, 0, 0, 0, 0,
   kKernelPrefillAsync, 128, 1, 64, 4, 8, 1, 0, "e4m3 rows widened on their way into the bf16 LDS tiles: 582-639 TFLOP/s"},
  {"prefill_256", kStagePrefill, 16, 256, 0, 0, 0, 0, 0, 0,
   kKernelPrefillAsync, 128, 1, 64, 4, 8, 1, 0, "two 64 KiB ring slots, one workgroup per CU: 666-725 TFLOP/s"},
  {"prefill_fp8_short", kStagePrefill, 8, 128, 0, 0, 4, 64, 0, 0,
   kKernelPrefillStaged, 32, 4, 64, 4, 16, 1, 0, "short-chunk tile of the register-staged kernel"},
  {"prefill_fp8", kStagePrefill, 8, 128, 0, 0, 0, 0, 0, 0,
   kKernelPrefillStaged, 128, 1, 64, 4, 16, 1, 0, "rows dequantised once per tile on their way to LDS"},
  {"prefill_options_short", kStagePrefill, 16, 128, 0, 0, 4, 64, 0, 0,
   kKernelPrefillAsync, 32, 4, 64, 4, 16, 1, 0, "masked / capped verify steps: 16 draft tokens on 4 k prefixes 2329 -> 261 us with the bit mask"},
  {"prefill_options", kStagePrefill, 16, 128, 0, 0, 0, 0, 0, 0,
   kKernelPrefillAsync, 128, 1, 64, 4, 16, 1, 0, "compiled flash kernel: every option"},
  // ---------------- absorbed MLA (near the ridge: LDS operand reads and piece starts decide)
  {"mla_wide", kStageMla, 16, 576, 128, 0, 128, 0, 0, kOptSoftCap | kOptAsmPages,
   kKernelMlaWide, 1, 128, 32, 4, 8, 1, 12, "every operand fragment feeds two matrix instructions: C5 226 -> 205 us, prefill chunks 48 -> 55 % of peak; a row switch costs 22 us = 12 tiles (C5 197 -> 191 us against 5)"},
  {"mla_pipe", kStageMla, 0, 576, 128, 0, 128, 0, 0, kOptSoftCap | kOptAsmPages,
   kKernelMlaPipe, 1, 128, 32, 8, 8, 1, 12, "e4m3 latents (bytes staged and expanded once per tile) and RPA_MLA_WIDE=0"},
  {"mla_shared_16", kStageMla, 0, 576, 1, 16, 0, 0, 0, kOptSoftCap | kOptOddPages,
   kKernelMlaShared, 1, 16, 32, 8, 8, 8, 8, "a tensor-parallel share of the heads: 64 rows x 8192 tokens 146 -> 120 us"},
  {"mla_shared_32", kStageMla, 0, 576, 17, 32, 0, 0, 0, kOptSoftCap | kOptOddPages,
   kKernelMlaShared, 1, 32, 32, 8, 8, 4, 8, "144 -> 126 us"},
  {"mla_shared_64", kStageMla, 0, 576, 33, 64, 0, 0, 0, kOptSoftCap | kOptOddPages,
   kKernelMlaShared, 1, 64, 32, 8, 8, 2, 8, "159 -> 147 us"},
  {"mla_compiled", kStageMla, 0, 576, 0, 0, 0, 0, 0, 0,
   kKernelMlaCompiled, 1, 128, 32, 8, 8, 1, 5, "soft cap, pages under 32 tokens, head counts that are no multiple of 128"},
};
// clang-format on

constexpr int kNumShapeRules = sizeof(kShapeRules) / sizeof(kShapeRules[0]);

inline bool shape_rule_matches(const ShapeRule& r, const ShapeKey& k) {
  if (r.stage != k.stage) return false;
  if (r.kv_bits && r.kv_bits != k.kv_bits) return false;
  if (r.head_dim && r.head_dim != k.head_dim) return false;
  if (r.heads_lo && k.heads < r.heads_lo) return false;
  if (r.heads_hi && k.heads > r.heads_hi) return false;
  if (r.heads_multiple && (k.heads % r.heads_multiple) != 0) return false;
  if (r.q_hi && !(k.max_q_len >= 1 && k.max_q_len <= r.q_hi)) return false;
  if (k.kv_bytes < r.bytes_lo) return false;
  if (r.forbid & k.options) return false;
  return true;
}

// `skip`: kernel families switched off by the caller (bit n = ShapeKernel n), the RPA_* overrides
inline const ShapeRule& select_shape(const ShapeKey& k, unsigned skip = 0) {
  for (int i = 0; i < kNumShapeRules; ++i)
    if (!(skip & (1u << kShapeRules[i].kernel)) && shape_rule_matches(kShapeRules[i], k)) return kShapeRules[i];
  // every stage ends in a row with the fewest conditions: the last row of the key's stage
  for (int i = kNumShapeRules - 1; i > 0; --i)
    if (kShapeRules[i].stage == k.stage) return kShapeRules[i];
  return kShapeRules[0];
}

}  // namespace rpa
