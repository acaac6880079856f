/*
 * rpa.h -- C ABI of the MI355X (gfx950) ragged paged attention library.
 *
 * The reference project (sglang-jax) has no native FFI on this path: its
 * operator boundary is a jitted Python callable.  Each entry point below names
 * the reference callable it stands in for (paths relative to the reference
 * checkout, python/sgl_jax/srt/...).  A jax.ffi custom call, a ctypes stub or
 * any other host binds exactly these symbols.
 *
 * Conventions
 *   - every pointer marked "device" is caller-owned device memory; the library
 *     never allocates or frees device memory and never synchronises a stream;
 *   - every launch is enqueued on the hipStream_t passed as `stream` (NULL is
 *     the legacy default stream), so calls are graph-capturable;
 *   - functions return RPA_OK (0) or a negative RpaStatus; rpa_last_error()
 *     returns a thread-local, human readable description of the last failure;
 *   - metadata (kv_lens, page_indices, cu_q_lens, cu_kv_lens) is read on the
 *     device only.  Host copies can be checked with rpa_validate_host().
 */
#ifndef RPA_MI355_H_
#define RPA_MI355_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RPA_VERSION 100 /* 0.1.0 */

/* The entry points below are the library's ONLY dynamic symbols: it is built with hidden default
 * visibility, so nothing else of it can collide with, or be interposed by, a host process. */
#if defined(__GNUC__) || defined(__clang__)
#define RPA_API __attribute__((visibility("default")))
#else
#define RPA_API
#endif

typedef enum RpaStatus {
  RPA_OK = 0,
  RPA_EINVAL_SHAPE = -1,
  RPA_EINVAL_DTYPE = -2,
  RPA_EINVAL_HEADS = -3,
  RPA_EINVAL_PAGE_RANGE = -4,
  RPA_EINVAL_QLEN_GT_KVLEN = -5,
  RPA_EINVAL_WINDOW = -6,
  RPA_EINVAL_SOFTCAP = -7,
  RPA_EINVAL_WORKSPACE = -8,
  RPA_EHIP = -9,
  RPA_EINVAL_DISTRIBUTION = -10,
  RPA_EUNSUPPORTED = -11,
  RPA_EINVAL_NULL = -12
} RpaStatus;

typedef enum RpaKvDtype {
  RPA_KV_BF16 = 0,
  RPA_KV_FP8_E4M3 = 1 /* OCP e4m3fn, max 448 */
} RpaKvDtype;

typedef enum RpaSoftmaxDtype {
  RPA_SOFTMAX_F32 = 0,
  RPA_SOFTMAX_BF16 = 1,
  RPA_SOFTMAX_F16 = 2
} RpaSoftmaxDtype;

typedef enum RpaMaskMode {
  RPA_MASK_CAUSAL = 0, /* query j of a sequence sees tokens <= kv_len - q_len + j */
  RPA_MASK_CUSTOM = 1, /* causal = 0 with custom_mask (speculative tree verification) */
  RPA_MASK_NONE = 2    /* causal = 0 without a mask: every query sees all kv_len tokens */
} RpaMaskMode;

typedef enum RpaLayout {
  /* one buffer [pages, P, 2*Hkv, D], heads stored K0,V0,K1,V1,...
   * (mem_cache/memory_pool.py:56-91, 580-588) */
  RPA_LAYOUT_FUSED = 0,
  /* two buffers k_pages, v_pages [pages, P, Hkv, D]
   * (kernels/ragged_paged_attention/ragged_paged_attention_v3.py:96-97) */
  RPA_LAYOUT_SPLIT = 1
} RpaLayout;

/*
 * One ragged paged attention call.  Field meanings follow the arguments of
 * ragged_paged_attention (ragged_paged_attention_v3.py:1667-1700) and of
 * ref_ragged_paged_attention (same file, :94-114).
 */
typedef struct RpaParams {
  /* ---- device buffers ---- */
  const void* q;              /* bf16 [T, Hq, D] */
  void* out;                  /* bf16 [T, Hq, D]; rows >= cu_q_lens[num_seqs] untouched */
  const void* kv_cache;       /* FUSED: the cache; SPLIT: k_pages */
  const void* v_pages;        /* SPLIT only, else NULL */
  const int32_t* kv_lens;     /* i32[S]  (kv length INCLUDING the new q tokens) */
  const int32_t* page_indices;/* i32 flat (cu_kv_lens != NULL) or [S, pages_per_seq] */
  const int32_t* cu_q_lens;   /* i32[S+1] */
  const int32_t* cu_kv_lens;  /* i32[S+1] cumulative page-aligned kv lens; NULL => padded 2-D table */
  const float* k_scale;       /* f32[Hkv] dequantisation scale of K, or NULL (= 1) */
  const float* v_scale;       /* f32[Hkv] or NULL */
  void* workspace;            /* partial rows of cut K/V ranges; >= rpa_workspace_bytes() */
  size_t workspace_bytes;
  /* ---- static shape ---- */
  int32_t num_tokens;         /* T */
  int32_t num_seqs;           /* S = distribution[2]: sequences to process */
  int32_t num_q_heads;        /* Hq */
  int32_t num_kv_heads;       /* Hkv, Hq % Hkv == 0 */
  int32_t head_dim;           /* D: 128 or 256.  Narrower heads (64, 80, 96, 192 ...) run zero-padded to the next
                               * multiple of 128 exactly as in the reference (rpa_v3:1187-1241 pads the queries,
                               * memory_pool.py:70 stores aligned rows); the caller pads, as the host mirror does */
  int32_t page_size;          /* P */
  int32_t total_pages;
  int32_t pages_per_seq;      /* row stride of the padded table (cu_kv_lens == NULL) */
  int32_t layout;             /* RpaLayout */
  int32_t kv_dtype;           /* RpaKvDtype */
  /* ---- batch composition: distribution = (decode_end, prefill_end, num_seqs)
   *      (ragged_paged_attention_v3.py:82-91); sequences [0, decode_end) have
   *      q_len == 1, the rest any q_len >= 1 ---- */
  int32_t decode_end;
  /* ---- host-side bounds used only to size grids (never to index memory) ---- */
  int32_t max_kv_len;         /* upper bound of kv_lens[0:num_seqs]; 0 => pages_per_seq*P or total_pages*P */
  int32_t max_q_len;          /* upper bound of q_len over [decode_end, num_seqs); 0 => T.  A promise: rows of a
                                 longer sequence past the bound are not computed */
  int32_t num_splits;         /* decode split-KV count per sequence; 0 => automatic */
  /* ---- options ---- */
  int32_t sliding_window;     /* 0 => off */
  float sm_scale;             /* the pipelined prefill kernel (bf16 cache, 128-wide heads, causal, no option)
                                 multiplies the bf16 queries by sm_scale * log2(e) and rounds them to bf16 once,
                                 where the reference scales the f32 scores (:149): element-wise inside the
                                 reference's rtol = atol = 2e-2, and at most 1.5e-2 of a row's norm on rows whose
                                 weight sits on one or two keys (1e-2 for every other path) */
  float soft_cap;             /* 0 => off */
  float mask_value;           /* 0 => default -0.7 * FLT_MAX */
  /* sum of kv_lens over the decode rows (host-side, balances the split plan); 0 => unknown */
  int64_t sum_decode_kv_len;
  /* ---- further options of ref_ragged_paged_attention (ragged_paged_attention_v3.py:103-113) ---- */
  const float* attention_sink;  /* device f32[Hq]: one extra logit per query head that enters only the
                                   softmax denominator (:185-196), or NULL */
  const int32_t* custom_mask;   /* device i32, flat: sequence i, query row j, token t at
                                   cu_mask_lens[i] + j * row_width_i + t; >= 1 keeps, < 1 masks (:154-163).
                                   Read only when mask_mode == RPA_MASK_CUSTOM */
  const int32_t* cu_mask_lens;  /* device i32[S+1]: cumulative q_len_i * row_width_i (:123-129, 1801-1806) */
  float xai_temperature_len;    /* > 0: logits of a query at position p > len are multiplied by
                                   log2(p) / log2(len) (:171-177); 0 => off.  With soft_cap set as well
                                   the factor multiplies the capped logit, the order of
                                   ref_ragged_paged_attention (:166-177); the reference's TPU kernel
                                   multiplies first and caps after (:481-486), so the reference's two
                                   paths differ from each other when both options are on */
  int32_t mask_mode;            /* RpaMaskMode */
  int32_t mask_rows_page_aligned; /* custom mask row_width_i: 0 => kv_len_i, 1 => kv_len_i rounded up to
                                   pages (cu_kv_lens delta; mask_aligned_to_cu_kv, :1791-1806) */
  int32_t softmax_dtype;        /* RpaSoftmaxDtype: the masked logits (and the sink) are rounded to this type
                                   before the softmax (:181-186, kernel :522-523); maxima, exponentials and
                                   sums stay f32 */
  float q_scale;                /* > 0: queries are divided by it and rounded to the cache's element type
                                   (fp8 saturating at +-448) before the first product, the logits multiplied
                                   by it (kernel :463-478); 0 => off */
  /* ---- static-shape mode: the batch composition read on the device ----
   * Device i32[3] (decode_end, prefill_end, num_seqs) as ragged_paged_attention takes it
   * (ragged_paged_attention_v3.py:1676, dispatch :2060-2090), or NULL.  When given, the host fields
   * decode_end and sum_decode_kv_len are ignored and num_seqs is only the static bound S (the length of
   * kv_lens): grids are sized from T, S and the page-table bound, every workgroup reads the
   * composition itself and the ones with nothing to do leave at once, so one compiled call serves
   * every batch of a bucket and nothing is read back to the host.  128- and 256-wide heads alike.
   * Neither mode limits the sequences or tokens of a call beyond int32: rows are folded onto the first
   * grid dimension. */
  const int32_t* distribution;
} RpaParams;

/*
 * Absorbed-MLA decode (mla_ragged_paged_attention, kernels/mla/v2/kernel.py:1338-1370;
 * oracle ref_mla_ragged_paged_attention, kernels/mla/v1/ref.py:108-248).
 * One shared latent row per token: [kv_c (lkv_dim) | k_pe (rope_dim)], rows of
 * `row_stride` elements (576 compact, 640 in the reference's 128-aligned layout
 * with rope at element offset `rope_offset`).
 */
typedef struct RpaMlaParams {
  const void* ql_nope;        /* bf16 [T, Hq, lkv_dim] */
  const void* q_pe;           /* bf16 [T, Hq, rope_dim] */
  void* out;                  /* bf16 [T, Hq, lkv_dim] */
  const void* cache_kv;       /* bf16 (or fp8-e4m3, see cache_dtype) [pages, P, row_stride] */
  const int32_t* kv_lens;
  const int32_t* page_indices;
  const int32_t* cu_q_lens;
  const int32_t* cu_kv_lens;  /* NULL => padded table with pages_per_seq stride */
  void* workspace;
  size_t workspace_bytes;
  int32_t num_tokens;
  int32_t num_seqs;           /* rpa_mla_decode: all must be decode rows (q_len == 1) */
  int32_t num_q_heads;
  int32_t lkv_dim;            /* 512 */
  int32_t rope_dim;           /* 64 */
  int32_t row_stride;         /* elements per cached token row */
  int32_t rope_offset;        /* element offset of k_pe inside a row */
  int32_t page_size;
  int32_t total_pages;
  int32_t pages_per_seq;
  int32_t max_kv_len;
  int32_t num_splits;         /* 0 => automatic */
  int32_t sliding_window;     /* 0 => off */
  float sm_scale;
  float soft_cap;             /* 0 => off */
  float mask_value;           /* 0 => default */
  int64_t sum_kv_len;         /* sum of kv_lens (host-side, balances the split plan); 0 => unknown */
  /* Scalar scales of kernels/mla/v2/kernel.py:1354-1356 (used at :372-375, :408-409; oracle
   * kernels/mla/v1/ref.py:223-226, 241-242): logits are multiplied by k_scale and q_scale next to
   * sm_scale, the output by v_scale.  0 => off. */
  float q_scale;
  float k_scale;
  float v_scale;
  /* Static-shape mode (see RpaParams.distribution): device i32[3] or NULL.  When given, num_seqs is
   * the static bound and rpa_mla_attention / rpa_mla_kv_write read distribution[2] on the device;
   * rpa_mla_decode (decode rows known on the host) does not take it. */
  const int32_t* distribution;
  /* Element type of cache_kv (and of the rows rpa_mla_kv_write takes): RPA_KV_BF16 (0, the default) or
   * RPA_KV_FP8_E4M3 -- latent rows of one byte per element, expanded to bf16 on their way through
   * LDS; k_scale / v_scale above are their dequantisation scales (kernels/mla/v1/ref.py:223-226,
   * 241-242).  row_stride and rope_offset stay in elements (multiples of 16 for fp8). */
  int32_t cache_dtype;
  int32_t reserved0;
} RpaMlaParams;

/* Library version (RPA_VERSION of the build). */
RPA_API int rpa_version(void);

/* Thread-local description of the last error returned on this thread. */
RPA_API const char* rpa_last_error(void);

/*
 * Static contract check: static_validate_inputs,
 * ragged_paged_attention_v3.py:1314-1439 (3-D q, Hq % Hkv == 0,
 * sliding_window > 0, soft_cap != 0, ...).  Called by every entry point.
 */
RPA_API int rpa_validate(const RpaParams* p);

/*
 * Value check on HOST copies of the metadata: dynamic_validate_inputs,
 * ragged_paged_attention_v3.py:1442-1487 (0 < q_len <= kv_len, page count and
 * page index ranges, distribution ordering).  Pointers are host memory.
 */
RPA_API int rpa_validate_host(const RpaParams* p, const int32_t* kv_lens, const int32_t* page_indices,
                      int64_t num_page_indices, const int32_t* cu_q_lens,
                      const int32_t* cu_kv_lens, const int32_t* distribution);

/*
 * Bytes of workspace for `p`: what the decode rows' split-KV plan needs (rpa_decode fails without
 * it), or, if larger, the room that lets a prefill launch which would leave most of the GPU idle
 * (one long prompt on a few heads, a verify step on a long context) cut its K/V ranges into pieces
 * and merge them, and that holds a custom mask as one bit per (query token, kv token); rpa_prefill uses
 * that room when it is there and otherwise runs whole ranges and reads the mask's i32 words (slower,
 * same results to the tolerance of the path).
 */
RPA_API size_t rpa_workspace_bytes(const RpaParams* p);
RPA_API size_t rpa_mla_workspace_bytes(const RpaMlaParams* p);

/*
 * Page-table gather of one sequence (the indexing expression
 * k_pages[page_indices[i]].reshape(-1, Hkv, D)[:kv_len] of
 * ragged_paged_attention_v3.py:138-139).  Copies, bit for bit, the K rows and
 * V rows of sequence `seq` into k_out / v_out [kv_len, Hkv, D] (kv dtype).
 */
RPA_API int rpa_gather_pages(const RpaParams* p, int32_t seq, void* k_out, void* v_out,
                     int32_t max_tokens, void* stream);

/*
 * Decode rows [0, decode_end): split-KV pass + combine pass.  Stands in for the
 * DECODE pallas_call of ragged_paged_attention_v3.py:2065-2072.
 */
RPA_API int rpa_decode(const RpaParams* p, void* stream);

/*
 * Prefill / mixed rows [decode_end, num_seqs): flash-style MFMA kernel.  Stands
 * in for the PREFILL and MIXED pallas_calls, ragged_paged_attention_v3.py:2074-2090.
 */
RPA_API int rpa_prefill(const RpaParams* p, void* stream);

/*
 * Whole call: dispatch by distribution exactly as
 * ragged_paged_attention_v3.py:2060-2090 does (decode rows, then the rest).
 */
RPA_API int rpa_attention(const RpaParams* p, void* stream);

/*
 * Which launch shape a call would take, as text: the row of the library's shape table (kernel family, query
 * positions x query heads x K/V tokens per workgroup, waves walked together, resident waves), the split plan
 * of the decode rows and the workspace behind it.  The counterpart of the reference's get_tuned_block_sizes /
 * get_default_block_sizes, which answer the same question for its tile table
 * (kernels/ragged_paged_attention/tuned_block_sizes_v3.py:2163-2229, ragged_paged_attention_v3.py:1490-1638).
 * Host arithmetic only (no launch, no device read).  Writes at most len - 1 characters plus a NUL into buf and
 * returns the length of the whole text (as snprintf does), or a negative RpaStatus.
 */
RPA_API int rpa_describe_plan(const RpaParams* p, char* buf, size_t len);

/*
 * rpa_attention for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it).  No counterpart in the reference, where XLA owns
 * every buffer.  Same arguments and results as rpa_attention, except that p->workspace and
 * p->workspace_bytes are ignored: the split-KV workspace is an array the library holds itself on
 * every GPU, rpa_noalloc_max_workspace_bytes() (40 MiB) long.  A batch whose decode rows need more
 * than that is refused with RPA_EINVAL_WORKSPACE; a prefill launch that would cut its K/V ranges
 * does so only if its partial rows fit the array (otherwise it runs whole ranges: the same rows to
 * the tolerance of the path, not bit for bit).  The call allocates and frees nothing.  All
 * calls on one GPU share the array: calls that overlap on one GPU (two streams, a graph replay next
 * to eager work) race on it; order them on one stream.
 */
RPA_API size_t rpa_noalloc_max_workspace_bytes(void);
RPA_API int rpa_attention_noalloc(const RpaParams* p, void* stream);

/*
 * Scatter the new K/V rows of every sequence into the paged cache: the fused
 * cache update of ragged_paged_attention_v3.py:670-719 / the standalone
 * kv_cache_update of kernels/update_kv_cache/update_kv_cache.py:120.  Token j of
 * sequence i goes to position kv_len_i - q_len_i + j.  keys/values are
 * [T, Hkv, D] in the cache dtype.
 */
RPA_API int rpa_kv_write(const RpaParams* p, const void* keys, const void* values, void* stream);

/* Absorbed-MLA decode, see RpaMlaParams: every sequence contributes exactly one query token. */
RPA_API int rpa_mla_decode(const RpaMlaParams* p, void* stream);

/*
 * Absorbed-MLA attention for any batch composition (decode, prefill chunks, mixed): the three
 * launches of mla_ragged_paged_attention (kernels/mla/v2/kernel.py:1338-1744) in one.  Query
 * token j of a sequence with q_len new tokens attends to the cache tokens 0 .. kv_len - q_len + j.
 * Workspace: rpa_mla_attention_workspace_bytes(); max_kv_len / sum_kv_len bound, resp. sum, the
 * per-token visible lengths.
 */
RPA_API size_t rpa_mla_attention_workspace_bytes(const RpaMlaParams* p);
RPA_API int rpa_mla_attention(const RpaMlaParams* p, void* stream);

/* rpa_describe_plan for the absorbed-MLA entry points: token_rows = 0 describes rpa_mla_decode, 1 rpa_mla_attention. */
RPA_API int rpa_mla_describe_plan(const RpaMlaParams* p, int token_rows, char* buf, size_t len);

/*
 * Write the new latent rows into the paged cache: update_kv_cache of kernels/mla/v1/ref.py:56-105
 * (the fused cache update of kernels/mla/v2/kernel.py).  new_kv_c bf16 [T, lkv_dim], new_k_pe bf16
 * [T, rope_dim]; token j of sequence i goes to position kv_len_i - q_len_i + j.
 */
RPA_API int rpa_mla_kv_write(const RpaMlaParams* p, const void* new_kv_c, const void* new_k_pe, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RPA_MI355_H_ */
