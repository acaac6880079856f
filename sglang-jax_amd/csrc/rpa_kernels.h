// Host-visible launch interface between the C ABI (rpa_capi.hip) and the
// kernel translation units.  Plain structs of device pointers and integers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rpa_shapes.h"
#include "rpa_tuning.h"

namespace rpa {

// How K and V rows of one (page, token, kv head) are addressed, in bytes.
//   fused  [pages, P, 2*Hkv, D]: v_base = k_base + D*esize, head_stride = 2*D*esize
//   split  k_pages / v_pages [pages, P, Hkv, D]: head_stride = D*esize
struct KvAddr {
  const char* k_base;
  const char* v_base;
  int64_t page_stride;
  int32_t tok_stride;
  int32_t head_stride;
};

struct PageTable {
  const int32_t* kv_lens;
  const int32_t* page_indices;
  const int32_t* cu_q_lens;
  const int32_t* cu_kv_lens;  // nullptr => padded table, row stride pages_per_seq
  int32_t pages_per_seq;
  int32_t page_size;
};

struct SoftmaxOpts {
  float sm_scale;
  float soft_cap;    // 0 => off
  float mask_value;  // finite, negative
  int32_t window;    // 0 => off
  const float* sink;  // f32[Hq] extra logit per query head that only enters the denominator, or nullptr
  float xai_len;      // > 0: logits of a query at position p > xai_len are multiplied by log2(p)/log2(xai_len)
  // prefill kernels only: 0 causal, 1 custom mask, 2 no mask
  int32_t mask_mode;
  int32_t mask_rows_page_aligned;
  const int32_t* custom_mask;
  const int32_t* cu_mask_lens;
  int32_t round_logits;  // masked logits and the sink are rounded before the softmax: 1 to bf16, 2 to f16
  float q_scale;         // > 0: queries are divided by it and rounded to the cache's element type; 0 => off
};

struct DecodeArgs {
  const uint16_t* q;  // bf16 [T, Hq, D]
  uint16_t* out;      // bf16 [T, Hq, D]
  KvAddr kv;
  PageTable pt;
  SoftmaxOpts sm;
  const float* k_scale;  // f32[Hkv] or nullptr
  const float* v_scale;
  float* ws_o;   // [num_rows, max_splits, Hq, D] unnormalised partial outputs
  float* ws_ml;  // [num_rows, max_splits, Hq, 2]  (running max in log2 units, sum)
  int32_t num_rows;  // decode sequences
  int32_t Hq, Hkv, G;
  int32_t chunk;       // fixed plan: kv tokens per split (multiple of 32)
  int32_t max_splits;  // fixed plan: grid.x
  int32_t fp8;
  // balanced plan: every wave takes the same number of 32-token blocks of the whole batch;
  // ws_o / ws_ml hold 2 * num_wgs * waves_per_wg groups of 16 rows
  int32_t balanced;
  int32_t num_wgs;       // workgroups of the balanced grid
  int32_t waves_per_wg;  // neighbouring kv heads walked together
  int32_t min_blocks_per_wave;
  int32_t forced_blocks_per_wave;  // > 0: tests pin the partition
  int32_t* cu_blocks;              // [num_rows + 1] prefix sum of 32-token blocks, written by the kernel
  // balanced plan, merge inside the kernel: one arrival word per (row, unit, wave of the
  // workgroup), [generation : 48 | arrivals : 16]; nullptr => a second launch merges
  unsigned long long* merge_counters;
  unsigned long long generation;  // of this call; a word of another generation counts as zero
  // device i32[3] (decode_end, prefill_end, num_seqs) or nullptr: when given, num_rows is only a bound
  // and the rows to process are [0, min(num_rows, dist[0]))
  const int32_t* dist;
};

struct PrefillArgs {
  const uint16_t* q;
  uint16_t* out;
  KvAddr kv;
  PageTable pt;
  SoftmaxOpts sm;
  const float* k_scale;
  const float* v_scale;
  int32_t seq_begin, seq_end;  // sequences [seq_begin, seq_end)
  int32_t Hq, Hkv, G;
  int32_t max_q_len;
  int32_t max_kv_len;  // host bound on kv_len of these sequences, 0 = unknown
  int32_t fp8;
  int32_t head_dim;  // 128, or 256 (bf16 cache only)
  // device i32[3] or nullptr: when given, seq_end is only a bound and the sequences to process are
  // [dist[0], min(seq_end, dist[2])) (custom-mask calls: [0, ...))
  const int32_t* dist;
  // K/V range of every workgroup cut into kv_splits pieces (pipelined kernel, launches that would leave most
  // of the GPU idle; 0 or 1 = whole ranges): partial rows f32 [token][Hq][piece][128] in ws_o, their
  // (reference, sum) pairs in ws_ml, merged by a second launch over num_tokens x Hq rows
  int32_t kv_splits;
  int32_t num_tokens;  // bound on the query tokens of the call (rows of q)
  float* ws_o;
  float* ws_ml;
  // Custom masks: one bit per (query token, kv token), mask_pitch 64-bit words per token row, written by
  // rpa_mask_bits_kernel in front of the attention kernels; nullptr: the kernels read the caller's i32 words
  uint64_t* mask_bits;
  int32_t mask_pitch;
};

struct GatherArgs {
  KvAddr kv;
  PageTable pt;
  int32_t seq;
  int32_t row_bytes;  // Hkv * D * esize of one gathered K (or V) row
  int32_t Hkv;
  int32_t head_bytes;  // D * esize
  void* k_out;
  void* v_out;
  int32_t max_tokens;
};

struct KvWriteArgs {
  KvAddr kv;  // bases are written through
  PageTable pt;
  const char* keys;    // [T, Hkv, D] cache dtype
  const char* values;
  int32_t num_seqs;
  int32_t Hkv;
  int32_t head_bytes;
  int32_t num_tokens;
  const int32_t* dist;  // device i32[3] or nullptr: when given, num_seqs is only a bound on dist[2]
};

struct MlaDecodeArgs {
  const uint16_t* ql_nope;  // [T, Hq, lkv]
  const uint16_t* q_pe;     // [T, Hq, rope]
  uint16_t* out;            // [T, Hq, lkv]
  const char* cache;        // [pages, P, row_stride] bf16 or e4m3
  PageTable pt;
  SoftmaxOpts sm;
  uint16_t* ws_o;  // [T, max_splits, Hq, lkv] unnormalised partial outputs, bf16
  float* ws_ml;    // [T, max_splits, Hq, 2] (reference in log2 units, sum)
  int32_t num_rows;     // grid rows: sequences (rows_are_tokens == 0) or query tokens
  int32_t num_seqs;
  int32_t rows_are_tokens;  // 1: row r is query token r of whatever sequence owns it (any q_len)
  int32_t Hq;
  int32_t row_stride;   // elements
  int32_t rope_offset;  // elements
  int32_t chunk;
  int32_t max_splits;
  // balanced plan (sequence rows only): the workgroups share the 32-token tiles of the batch
  // evenly; ws_o / ws_ml hold 2 * num_wgs groups of 128 heads
  int32_t balanced;
  int32_t num_wgs;
  int32_t min_tiles_per_wg;
  int32_t forced_tiles_per_wg;
  int32_t piece_pad;  // balanced plan: what starting one more (row, head group) costs a workgroup, in tiles
  int32_t* cu_tiles;  // [num_rows + 1] prefix sum of tiles, written by the kernel
  float out_scale;    // finished rows are multiplied by it (v_scale; 1 when off)
  const int32_t* dist;  // device i32[3] or nullptr: when given, num_seqs is only a bound on dist[2]
  int32_t fp8;          // cache rows are e4m3 bytes (row_stride / rope_offset stay in elements)
};

struct MlaWriteArgs {
  char* cache;              // [pages, P, row_stride] bf16
  PageTable pt;
  const char* new_kv_c;  // [T, 512] in the cache's element type
  const char* new_k_pe;  // [T, 64]
  int32_t fp8;
  int32_t num_tokens;
  int32_t num_seqs;
  int32_t row_stride;
  int32_t rope_offset;
  const int32_t* dist;  // device i32[3] or nullptr: when given, num_seqs is only a bound on dist[2]
};

hipError_t launch_decode(const DecodeArgs& a, hipStream_t stream);
hipError_t launch_prefill(const PrefillArgs& a, hipStream_t stream);
// How many pieces launch_prefill would cut the K/V ranges into if it had the workspace (1 = no cut), and the
// bytes of workspace that takes.
int prefill_kv_splits(const PrefillArgs& a);
size_t prefill_split_workspace_bytes(const PrefillArgs& a, int splits);
hipError_t launch_gather(const GatherArgs& a, hipStream_t stream);
// head_dim 256: every query token of sequences [seq_begin, seq_end) as a row of its own; at most
// max_token_rows tokens (a host bound) are covered.  With a.dist set, seq_end is a bound and dist_role says
// which partition the kernel takes from the device: 1 = decode rows, 2 = everything behind them
hipError_t launch_rows256(const DecodeArgs& a, int seq_begin, int seq_end, int max_token_rows, int dist_role,
                          hipStream_t stream);
hipError_t launch_kv_write(const KvWriteArgs& a, hipStream_t stream);
hipError_t launch_mla_decode(const MlaDecodeArgs& a, hipStream_t stream);
// The rows of the shape table (rpa_shapes.h) these launchers select for a call, RPA_* overrides applied.
const ShapeRule& prefill_shape_of(const PrefillArgs& a);
ShapeKey mla_shape_key(const MlaDecodeArgs& a);
unsigned mla_shape_skip(const Tuning& tune);
// how query tokens of a chunk share a workgroup (0: they do not; 1, 2: eight waves; 3: wide workgroups)
int mla_token_group_mode(const MlaDecodeArgs& a, const Tuning& tune, const ShapeRule& shape);
hipError_t launch_mla_kv_write(const MlaWriteArgs& a, hipStream_t stream);

}  // namespace rpa
