// The RPA_* environment switches, read into one struct.  tuning() costs a walk over the pointers of
// `environ` per call (tens of nanoseconds): the strings are parsed again only when that walk shows the
// environment has changed since this thread last looked, so a host that never touches its environment
// pays for no getenv on the serving path, and tests and experiments can still flip a switch between
// two calls.  Defaults are the measured optima of the shape-keyed selection in rpa_capi.hip; the
// switches exist to force a path (tests compare paths) and to repeat the measurements behind the
// defaults.
#pragma once

namespace rpa {

struct Tuning {
  // ---- decode (rpa_decode.hip)
  int decode_min_chunk = 64;        // RPA_DECODE_MIN_CHUNK       smallest piece of a row, tokens
  int decode_balanced = 1;          // RPA_DECODE_BALANCED        0: fixed split plan on ragged batches too
  int decode_waves_per_wg = 0;      // RPA_DECODE_WAVES_PER_WG    0: by the batch's bytes (2 or 4)
  int decode_wave_capacity = 0;     // RPA_DECODE_WAVE_CAPACITY   0: by the cache's element size
  int decode_merge_in_kernel = 0;   // RPA_DECODE_MERGE_IN_KERNEL 1: one launch, merge behind arrival counters
  // ---- prefill (rpa_prefill.hip, rpa_prefill_pipe.hip)
  int mask_bits = 1;                // RPA_MASK_BITS              0: kernels read the caller's i32 mask words
  int prefill_rows256 = 0;          // RPA_PREFILL_ROWS256        1: 256-wide chunks through the row kernel
  int prefill_staged = 0;           // RPA_PREFILL_STAGED         1: bf16 caches through the register-staged kernel
  int prefill_pipe = 1;             // RPA_PREFILL_PIPE           0: no assembly loop, compiled flash kernel
  int prefill_pipe_tile = 0;        // RPA_PREFILL_PIPE_TILE      0: by max_q_len; 32 | 128 force a tile
  int prefill_level_order = 1;      // RPA_PREFILL_LEVEL_ORDER    0: query tiles in sequence order
  int prefill_pipe_nq = 0;          // RPA_PREFILL_PIPE_NQ        2: 64 query rows per wave
  float prefill_pipe_limit = 0.f;   // RPA_PREFILL_PIPE_LIMIT     0: the kernel's own row-sum limit
  int prefill_pipe_masked = 1;      // RPA_PREFILL_PIPE_MASKED    0: the steps on the causal diagonal through compiled code
  int prefill_splits = -1;          // RPA_PREFILL_SPLITS         -1: cost model; 0 | 1 never; n forces n pieces
  // ---- absorbed MLA (rpa_mla.hip)
  int mla_min_chunk = 256;          // RPA_MLA_MIN_CHUNK
  int mla_wg_capacity = 0;          // RPA_MLA_WG_CAPACITY        0: one workgroup per CU
  int mla_balanced = 1;             // RPA_MLA_BALANCED
  int mla_piece_pad = -1;           // RPA_MLA_PIECE_PAD          -1: the shape table's; tiles a workgroup pays for starting another row
  int mla_pipe = 1;                 // RPA_MLA_PIPE               0: compiled tile loop
  int mla_shared_tiles = 1;         // RPA_MLA_SHARED_TILES       0: one wave per block of 16 heads, always
  int mla_wide = 1;                 // RPA_MLA_WIDE               0: eight-wave kernels; 32: wide loop on 32x32x16
  int mla_token_groups = 1;         // RPA_MLA_TOKEN_GROUPS       0: prefill rows with few heads one token per workgroup
};

const Tuning& tuning();

}  // namespace rpa
