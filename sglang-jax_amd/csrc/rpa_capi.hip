// C ABI of the library (declared in include/rpa.h): argument checking,
// grid sizing from the host-side bounds, and dispatch to the kernel launchers.
// No device allocation, no synchronisation, no host reads of device memory.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/rpa.h"
#include "rpa_kernels.h"
#include "rpa_tuning.h"

extern char** environ;

namespace rpa {

// One parse of the RPA_* switches per change of the environment (per thread): see rpa_tuning.h.
const Tuning& tuning() {
  thread_local Tuning t;
  thread_local uint64_t seen = 0;
  thread_local bool valid = false;
  // setenv() never edits a string in place: a changed variable is a changed pointer in environ
  uint64_t h = 1469598103934665603ull;
  for (char** e = environ; e && *e; ++e) h = (h ^ reinterpret_cast<uintptr_t>(*e)) * 1099511628211ull;
  if (valid && h == seen) return t;
  t = Tuning();
  auto geti = [](const char* name, int& dst) {
    const char* v = getenv(name);
    if (v && *v) dst = atoi(v);
  };
  geti("RPA_DECODE_MIN_CHUNK", t.decode_min_chunk);
  geti("RPA_DECODE_BALANCED", t.decode_balanced);
  geti("RPA_DECODE_WAVES_PER_WG", t.decode_waves_per_wg);
  geti("RPA_DECODE_WAVE_CAPACITY", t.decode_wave_capacity);
  geti("RPA_DECODE_MERGE_IN_KERNEL", t.decode_merge_in_kernel);
  geti("RPA_MASK_BITS", t.mask_bits);
  geti("RPA_PREFILL_ROWS256", t.prefill_rows256);
  geti("RPA_PREFILL_STAGED", t.prefill_staged);
  geti("RPA_PREFILL_PIPE", t.prefill_pipe);
  geti("RPA_PREFILL_PIPE_TILE", t.prefill_pipe_tile);
  geti("RPA_PREFILL_LEVEL_ORDER", t.prefill_level_order);
  geti("RPA_PREFILL_PIPE_NQ", t.prefill_pipe_nq);
  geti("RPA_PREFILL_PIPE_MASKED", t.prefill_pipe_masked);
  geti("RPA_PREFILL_SPLITS", t.prefill_splits);
  geti("RPA_MLA_MIN_CHUNK", t.mla_min_chunk);
  geti("RPA_MLA_WG_CAPACITY", t.mla_wg_capacity);
  geti("RPA_MLA_BALANCED", t.mla_balanced);
  geti("RPA_MLA_PIECE_PAD", t.mla_piece_pad);
  geti("RPA_MLA_PIPE", t.mla_pipe);
  geti("RPA_MLA_SHARED_TILES", t.mla_shared_tiles);
  geti("RPA_MLA_WIDE", t.mla_wide);
  geti("RPA_MLA_TOKEN_GROUPS", t.mla_token_groups);
  if (const char* v = getenv("RPA_PREFILL_PIPE_LIMIT")) {
    if (*v) t.prefill_pipe_limit = (float)atof(v);
  }
  seen = h;
  valid = true;
  return t;
}

}  // namespace rpa

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

constexpr float kDefaultMask = -0.7f * 3.4028234663852886e38f;

int esize_of(int kv_dtype) { return kv_dtype == RPA_KV_FP8_E4M3 ? 1 : 2; }

rpa::KvAddr kv_addr(const RpaParams* p) {
  rpa::KvAddr kv;
  const int es = esize_of(p->kv_dtype);
  const int64_t D = p->head_dim, H = p->num_kv_heads, P = p->page_size;
  kv.k_base = static_cast<const char*>(p->kv_cache);
  if (p->layout == RPA_LAYOUT_FUSED) {
    kv.v_base = kv.k_base + D * es;
    kv.head_stride = (int32_t)(2 * D * es);
    kv.tok_stride = (int32_t)(2 * H * D * es);
  } else {
    kv.v_base = static_cast<const char*>(p->v_pages);
    kv.head_stride = (int32_t)(D * es);
    kv.tok_stride = (int32_t)(H * D * es);
  }
  kv.page_stride = (int64_t)kv.tok_stride * P;
  return kv;
}

rpa::PageTable page_table(const RpaParams* p) {
  rpa::PageTable pt;
  pt.kv_lens = p->kv_lens;
  pt.page_indices = p->page_indices;
  pt.cu_q_lens = p->cu_q_lens;
  pt.cu_kv_lens = p->cu_kv_lens;
  pt.pages_per_seq = p->pages_per_seq;
  pt.page_size = p->page_size;
  return pt;
}

rpa::SoftmaxOpts softmax_opts(float sm_scale, float soft_cap, float mask_value, int window) {
  rpa::SoftmaxOpts s;
  s.sm_scale = sm_scale;
  s.soft_cap = soft_cap;
  s.mask_value = (mask_value == 0.0f) ? kDefaultMask : mask_value;
  s.window = window;
  s.sink = nullptr;
  s.xai_len = 0.f;
  s.mask_mode = RPA_MASK_CAUSAL;
  s.mask_rows_page_aligned = 0;
  s.custom_mask = nullptr;
  s.cu_mask_lens = nullptr;
  s.round_logits = 0;
  s.q_scale = 0.f;
  return s;
}

rpa::SoftmaxOpts softmax_opts(const RpaParams* p) {
  rpa::SoftmaxOpts s = softmax_opts(p->sm_scale, p->soft_cap, p->mask_value, p->sliding_window);
  s.sink = p->attention_sink;
  s.xai_len = p->xai_temperature_len;
  s.mask_mode = p->mask_mode;
  s.mask_rows_page_aligned = p->mask_rows_page_aligned;
  s.custom_mask = p->custom_mask;
  s.cu_mask_lens = p->cu_mask_lens;
  s.round_logits = p->softmax_dtype == RPA_SOFTMAX_BF16 ? 1 : (p->softmax_dtype == RPA_SOFTMAX_F16 ? 2 : 0);
  s.q_scale = p->q_scale;
  return s;
}

int64_t kv_len_bound(int max_kv_len, int pages_per_seq, int page_size, int total_pages, bool ragged) {
  if (max_kv_len > 0) return max_kv_len;
  if (!ragged && pages_per_seq > 0) return (int64_t)pages_per_seq * page_size;
  return (int64_t)total_pages * page_size;
}

// Split-KV plan.  A split is one wave job per (row, kv head); `units` such jobs exist
// per split index and `work` is their total length in tokens.  The decode kernels hold
// `capacity` waves at once (8 per CU); measured on MI355X, one full round of equally long
// jobs beats both fewer, longer jobs (idle CUs) and many short ones (per-job prologue,
// partial write and a longer combine), so the chunk is sized to fill one round.
struct SplitPlan {
  int chunk;
  int splits;
};

int wave_capacity() {
  static const int cap = [] {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    return cus * 8;
  }();
  return cap;
}

SplitPlan plan_splits(int64_t max_len, int window, int64_t units, int64_t work, int forced, int min_chunk,
                      int capacity) {
  int64_t eff = max_len;
  if (window > 0 && eff > (int64_t)window + 31) eff = (int64_t)window + 31;
  if (eff < 1) eff = 1;
  if (units < 1) units = 1;
  const bool uniform = (work <= 0 || work >= units * eff);  // every row as long as the bound (or unknown)
  if (uniform) work = units * eff;
  int64_t chunk;
  if (forced > 0) {
    chunk = (eff + forced - 1) / forced;
  } else {
    // Every row wastes about half a job on its remainder.  With ragged rows the jobs differ
    // in length and the dispatcher does not fill CUs evenly, so a plan that uses every slot
    // spills into a second, nearly empty round: aim at 85 % of the slots (measured optimum
    // on the mixed Llama-3-8B batch: 82-88 %).
    const int64_t room = (uniform ? (int64_t)capacity : (int64_t)capacity * 17 / 20) - units / 2;
    chunk = room > 0 ? (work + room - 1) / room : eff;
    if (chunk < min_chunk) chunk = min_chunk;
    if (chunk > eff) chunk = eff;
    // equal-length rows: spread the remainder over all splits instead of one short job
    if (uniform) chunk = (eff + (eff + chunk - 1) / chunk - 1) / ((eff + chunk - 1) / chunk);
  }
  chunk = (chunk + 31) / 32 * 32;
  if (chunk < 32) chunk = 32;
  int64_t splits = (eff + chunk - 1) / chunk;
  if (splits < 1) splits = 1;
  SplitPlan sp;
  sp.chunk = (int)chunk;
  sp.splits = (int)splits;
  return sp;
}

int decode_wave_capacity(const RpaParams* p);

SplitPlan decode_plan(const RpaParams* p) {
  const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                     p->cu_kv_lens != nullptr);
  const int G = p->num_q_heads / p->num_kv_heads;
  const int64_t per_row = (int64_t)p->num_kv_heads * ((G + 15) / 16);
  const int64_t units = (int64_t)p->decode_end * per_row;
  int64_t work = p->sum_decode_kv_len > 0 ? p->sum_decode_kv_len * per_row : 0;
  if (p->sliding_window > 0) work = 0;  // visible lengths are not the raw lengths
  return plan_splits(bound, p->sliding_window, units, work, p->num_splits,
                     rpa::tuning().decode_min_chunk, decode_wave_capacity(p));
}

// Balanced decode plan: a fixed number of waves (every wave slot of the GPU once) share the
// 32-token blocks of the batch evenly; the device works the partition out from kv_lens.
bool decode_balanced() { return rpa::tuning().decode_balanced != 0; }

// The balanced plan pays for itself on ragged batches.  Rows of one known length (the host's
// sum equals rows x bound) split evenly under the fixed plan already, and small batches the
// fixed plan does not split at all finish in one launch with no partial rows.
int decode_waves_per_wg(const RpaParams* p);
int decode_wgs(const RpaParams* p);
int64_t decode_kv_bytes(const RpaParams* p);

bool use_balanced(const RpaParams* p, const SplitPlan& fixed) {
  if (!decode_balanced()) return false;
  if (p->num_splits == 1) return false;  // the caller asked for whole rows: one launch, no merge pass
  // Rows the fixed plan leaves whole finish in one launch with no merge pass: right for small,
  // latency-bound batches.  A large ragged batch is still better dealt out evenly -- one job per
  // (row, kv head) of very different lengths, about one per wave slot, ends with the longest row
  // (128 rows of 128..4096 tokens: 228 -> 205 us, 200 rows of 1000..3000: 351 -> 295 us).
  if (fixed.splits <= 1 && decode_kv_bytes(p) < (64ll << 20)) return false;
  if (p->num_splits > 0) return true;
  // too little work to hand every workgroup its minimum piece: latency-bound, keep the launch count low
  const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                     p->cu_kv_lens != nullptr);
  const int nw = decode_waves_per_wg(p);
  const int64_t units = (int64_t)((p->num_kv_heads + nw - 1) / nw) * ((p->num_q_heads / p->num_kv_heads + 15) / 16);
  const int64_t min_blocks = std::max(1, rpa::tuning().decode_min_chunk / 32);
  if ((int64_t)p->decode_end * ((bound + 31) / 32) * units <= (int64_t)decode_wgs(p) * min_blocks)
    return false;
  const bool equal_lengths = p->sum_decode_kv_len > 0 && p->max_kv_len > 0 &&
                             p->sum_decode_kv_len == (int64_t)p->decode_end * p->max_kv_len;
  if (equal_lengths) return false;
  // a sliding window clips every longer row to the same length: once the mean length reaches
  // the window most rows are clipped and the batch is as good as uniform
  if (p->sliding_window > 0 && p->sum_decode_kv_len >= (int64_t)p->decode_end * p->sliding_window) return false;
  return true;
}

// Bytes of KV the decode rows will read, as far as the host knows (its sum of lengths, or rows
// times the length bound).
int64_t decode_kv_bytes(const RpaParams* p) {
  int64_t tokens = p->sum_decode_kv_len;
  if (tokens <= 0)
    tokens = (int64_t)p->decode_end * kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                                   p->cu_kv_lens != nullptr);
  if (p->sliding_window > 0) tokens = std::min(tokens, (int64_t)p->decode_end * (p->sliding_window + 31));
  return tokens * 2 * p->num_kv_heads * p->head_dim * esize_of(p->kv_dtype);
}

// The decode rows' row of the shape table (rpa_shapes.h): waves of a workgroup = neighbouring kv heads walked
// together (their rows are adjacent in the cache), and the waves resident at once = bytes in flight.
const rpa::ShapeRule& decode_shape(const RpaParams* p) {
  rpa::ShapeKey k = {};
  k.stage = rpa::kStageDecode;
  k.kv_bits = 8 * esize_of(p->kv_dtype);
  k.head_dim = p->head_dim;
  k.heads = p->num_q_heads / p->num_kv_heads;
  k.kv_bytes = decode_kv_bytes(p);
  return rpa::select_shape(k);
}

int decode_waves_per_wg(const RpaParams* p) {
  const int forced = rpa::tuning().decode_waves_per_wg;
  const int nw = forced > 0 ? forced : decode_shape(p).waves_per_wg;
  return std::max(1, std::min(std::min(nw, 4), p->num_kv_heads));
}

// Always a whole number of workgroups, and never a workgroup count between one and two per CU, which the
// dispatcher spreads unevenly (1152 waves in 4-wave workgroups: 133 us on C2).
int decode_wave_capacity(const RpaParams* p) {
  const int env = rpa::tuning().decode_wave_capacity;
  if (env > 0) return env;
  const int cus = wave_capacity() / 8;
  const int nw = decode_waves_per_wg(p);
  return std::max(nw, cus * decode_shape(p).resident_x8 / 8 / nw * nw);
}

int decode_wgs(const RpaParams* p) { return std::max(1, decode_wave_capacity(p) / decode_waves_per_wg(p)); }

int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return RPA_OK;
  return fail(RPA_EHIP, "%s: %s", what, hipGetErrorString(e));
}

// head_dim 256, decode rows: split like the fixed plan when there are too few rows to fill the GPU
// (the row kernel keeps nothing in flight while it computes, so it wants every wave slot)
SplitPlan rows256_plan(const RpaParams* p) {
  const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                     p->cu_kv_lens != nullptr);
  const int G = p->num_q_heads / p->num_kv_heads;
  const int64_t per_row = (int64_t)p->num_kv_heads * ((G + 15) / 16);
  const int64_t units = (int64_t)p->decode_end * per_row;
  int64_t work = p->sum_decode_kv_len > 0 ? p->sum_decode_kv_len * per_row : 0;
  if (p->sliding_window > 0) work = 0;
  return plan_splits(bound, p->sliding_window, units, work, p->num_splits, 256, wave_capacity());
}

size_t rows256_workspace(const RpaParams* p) {
  if (p->decode_end <= 0) return 0;
  const SplitPlan sp = rows256_plan(p);
  if (sp.splits <= 1) return 0;
  return (size_t)p->decode_end * sp.splits * p->num_q_heads * (p->head_dim + 2) * sizeof(float);
}

// head_dim 256: every query token of sequences [seq_begin, seq_end) is a row of the row kernel
int rows256(const RpaParams* p, int seq_begin, int seq_end, void* stream, int dist_role = 0) {
  if (seq_end <= seq_begin) return RPA_OK;
  rpa::DecodeArgs a = {};
  a.q = static_cast<const uint16_t*>(p->q);
  a.out = static_cast<uint16_t*>(p->out);
  a.kv = kv_addr(p);
  a.pt = page_table(p);
  a.sm = softmax_opts(p);
  a.k_scale = p->k_scale;
  a.v_scale = p->v_scale;
  a.num_rows = seq_end;
  a.Hq = p->num_q_heads;
  a.Hkv = p->num_kv_heads;
  a.G = p->num_q_heads / p->num_kv_heads;
  a.fp8 = p->kv_dtype == RPA_KV_FP8_E4M3;
  a.dist = dist_role ? p->distribution : nullptr;
  // decode rows are one token each; other sequences are bounded by the tokens of the call
  const int rows = (dist_role != 2 && seq_end <= p->decode_end) ? (seq_end - seq_begin) : p->num_tokens;
  if (seq_begin == 0 && seq_end == p->decode_end && p->mask_mode != RPA_MASK_CUSTOM) {
    const SplitPlan sp = rows256_plan(p);
    if (sp.splits > 1) {
      const size_t need = rows256_workspace(p);
      if (!p->workspace || p->workspace_bytes < need)
        return fail(RPA_EINVAL_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, p->workspace_bytes);
      a.chunk = sp.chunk;
      a.max_splits = sp.splits;
      a.ws_o = static_cast<float*>(p->workspace);
      a.ws_ml = a.ws_o + (size_t)p->decode_end * sp.splits * p->num_q_heads * p->head_dim;
    }
  }
  return check_hip(rpa::launch_rows256(a, seq_begin, seq_end, rows, dist_role, static_cast<hipStream_t>(stream)),
                   "rpa rows256");
}

}  // namespace

// ---- rpa_attention_noalloc: the split-KV workspace as a static device array ----
// Every GPU the library is loaded on holds one copy of the array until the process ends.
constexpr size_t kNoAllocScratchBytes = (size_t)40 << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// The array's address on the current device (its name is only a host-side handle): looked up once
// per device with that device current, then kept.
int noalloc_scratch(void** out) {
  int dev = -1;
  if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (dev < 0 || dev >= kMaxDevices) return fail(RPA_EUNSUPPORTED, "device ordinal %d: at most %d devices", dev, kMaxDevices);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    if (int rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
    if (!ptr) return fail(RPA_EHIP, "hipGetSymbolAddress(scratch) returned a null address");
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return RPA_OK;
}

extern "C" {

int rpa_version(void) { return RPA_VERSION; }

const char* rpa_last_error(void) { return g_err; }

int rpa_validate(const RpaParams* p) {
  if (!p) return fail(RPA_EINVAL_NULL, "params is NULL");
  if (p->num_tokens < 0 || p->num_seqs < 0 || p->num_q_heads <= 0 || p->num_kv_heads <= 0 ||
      p->head_dim <= 0 || p->page_size <= 0 || p->total_pages <= 0)
    return fail(RPA_EINVAL_SHAPE, "expected positive shape: T=%d S=%d Hq=%d Hkv=%d D=%d P=%d pages=%d",
                p->num_tokens, p->num_seqs, p->num_q_heads, p->num_kv_heads, p->head_dim,
                p->page_size, p->total_pages);
  if (p->num_q_heads % p->num_kv_heads != 0)
    return fail(RPA_EINVAL_HEADS, "expected num_q_heads=%d to be divisible by num_kv_heads=%d",
                p->num_q_heads, p->num_kv_heads);
  if (p->head_dim != 128 && p->head_dim != 256)
    return fail(RPA_EUNSUPPORTED, "head_dim=%d: 128 and 256 are built", p->head_dim);
  if (p->kv_dtype != RPA_KV_BF16 && p->kv_dtype != RPA_KV_FP8_E4M3)
    return fail(RPA_EINVAL_DTYPE, "kv_dtype=%d is not a floating point cache dtype", p->kv_dtype);
  if (p->layout != RPA_LAYOUT_FUSED && p->layout != RPA_LAYOUT_SPLIT)
    return fail(RPA_EINVAL_SHAPE, "layout=%d unknown", p->layout);
  if (p->layout == RPA_LAYOUT_SPLIT && !p->v_pages)
    return fail(RPA_EINVAL_NULL, "split layout needs v_pages");
  if (p->sliding_window < 0) return fail(RPA_EINVAL_WINDOW, "sliding_window=%d must be positive", p->sliding_window);
  if (std::isnan(p->soft_cap)) return fail(RPA_EINVAL_SOFTCAP, "soft_cap must not be NaN");
  if (!p->distribution && (p->decode_end < 0 || p->decode_end > p->num_seqs))
    return fail(RPA_EINVAL_DISTRIBUTION, "distribution must satisfy 0 <= decode_end=%d <= num_seqs=%d",
                p->decode_end, p->num_seqs);
  if (p->num_seqs > 0) {
    if (!p->q || !p->out || !p->kv_cache || !p->kv_lens || !p->page_indices || !p->cu_q_lens)
      return fail(RPA_EINVAL_NULL, "q/out/kv_cache/kv_lens/page_indices/cu_q_lens must be non-NULL");
    if (!p->cu_kv_lens && p->pages_per_seq <= 0)
      return fail(RPA_EINVAL_SHAPE, "padded page table needs pages_per_seq > 0");
  }
  if (p->mask_value > 0.0f) return fail(RPA_EINVAL_SHAPE, "mask_value=%g must be negative", p->mask_value);
  if (p->mask_mode < RPA_MASK_CAUSAL || p->mask_mode > RPA_MASK_NONE)
    return fail(RPA_EINVAL_SHAPE, "mask_mode=%d is not an RpaMaskMode", p->mask_mode);
  if (p->mask_mode == RPA_MASK_CUSTOM && (!p->custom_mask || !p->cu_mask_lens))
    return fail(RPA_EINVAL_NULL, "RPA_MASK_CUSTOM needs custom_mask and cu_mask_lens");
  if (p->mask_mode == RPA_MASK_CUSTOM && p->mask_rows_page_aligned && !p->cu_kv_lens)
    return fail(RPA_EINVAL_NULL, "page-aligned mask rows need cu_kv_lens");
  if (p->softmax_dtype != RPA_SOFTMAX_F32 && p->softmax_dtype != RPA_SOFTMAX_BF16 && p->softmax_dtype != RPA_SOFTMAX_F16)
    return fail(RPA_EINVAL_DTYPE, "softmax_dtype=%d is not an RpaSoftmaxDtype", p->softmax_dtype);
  if (p->q_scale < 0.0f || std::isnan(p->q_scale))
    return fail(RPA_EINVAL_SHAPE, "q_scale=%g must be positive (0 = off)", p->q_scale);
  if (p->xai_temperature_len < 0.0f || std::isnan(p->xai_temperature_len))
    return fail(RPA_EINVAL_SHAPE, "xai_temperature_len=%g must be positive", p->xai_temperature_len);
  return RPA_OK;
}

int rpa_validate_host(const RpaParams* p, const int32_t* kv_lens, const int32_t* page_indices,
                      int64_t num_page_indices, const int32_t* cu_q_lens, const int32_t* cu_kv_lens,
                      const int32_t* distribution) {
  int rc = rpa_validate(p);
  if (rc != RPA_OK) return rc;
  if (!kv_lens || !page_indices || !cu_q_lens) return fail(RPA_EINVAL_NULL, "host metadata is NULL");
  int i = 0, j = 0, k = p->num_seqs;
  if (distribution) {
    i = distribution[0]; j = distribution[1]; k = distribution[2];
    if (!(i <= j && j <= k)) return fail(RPA_EINVAL_DISTRIBUTION, "distribution must satisfy i <= j <= k, got %d, %d, %d", i, j, k);
    if (k != p->num_seqs || i != p->decode_end)
      return fail(RPA_EINVAL_DISTRIBUTION, "distribution (%d,%d,%d) disagrees with decode_end=%d num_seqs=%d", i, j, k, p->decode_end, p->num_seqs);
  } else {
    i = p->decode_end;
  }
  if (cu_q_lens[k] > p->num_tokens)
    return fail(RPA_EINVAL_SHAPE, "cu_q_lens[%d]=%d exceeds max_num_tokens=%d", k, cu_q_lens[k], p->num_tokens);
  const int P = p->page_size;
  for (int s = 0; s < k; ++s) {
    const int q_len = cu_q_lens[s + 1] - cu_q_lens[s];
    const int kv_len = kv_lens[s];
    if (q_len <= 0) return fail(RPA_EINVAL_QLEN_GT_KVLEN, "Sequence %d: q_len=%d must be > 0", s, q_len);
    if (q_len > kv_len) return fail(RPA_EINVAL_QLEN_GT_KVLEN, "Sequence %d: q_len=%d > kv_len=%d", s, q_len, kv_len);
    if (s < i && q_len != 1) return fail(RPA_EINVAL_DISTRIBUTION, "Sequence %d is in the decode range but q_len=%d", s, q_len);
    const int page_cnt = (kv_len + P - 1) / P;
    int64_t start;
    if (cu_kv_lens) {
      if (cu_kv_lens[s] % P != 0) return fail(RPA_EINVAL_SHAPE, "cu_kv_lens[%d]=%d is not page aligned", s, cu_kv_lens[s]);
      if (cu_kv_lens[s + 1] - cu_kv_lens[s] < page_cnt * P)
        return fail(RPA_EINVAL_PAGE_RANGE, "Sequence %d: page_cnt=%d does not fit cu_kv_lens", s, page_cnt);
      start = cu_kv_lens[s] / P;
    } else {
      if (page_cnt > p->pages_per_seq)
        return fail(RPA_EINVAL_PAGE_RANGE, "Sequence %d: page_cnt=%d > pages_per_seq=%d", s, page_cnt, p->pages_per_seq);
      start = (int64_t)s * p->pages_per_seq;
    }
    if (start + page_cnt > num_page_indices)
      return fail(RPA_EINVAL_PAGE_RANGE, "Sequence %d: page list [%lld, %lld) exceeds page_indices length %lld", s,
                  (long long)start, (long long)(start + page_cnt), (long long)num_page_indices);
    for (int pg = 0; pg < page_cnt; ++pg) {
      const int idx = page_indices[start + pg];
      if (idx < 0 || idx >= p->total_pages)
        return fail(RPA_EINVAL_PAGE_RANGE, "Sequence %d, page %d: index=%d out of [0, %d)", s, pg, idx, p->total_pages);
    }
    if (p->max_kv_len > 0 && kv_len > p->max_kv_len)
      return fail(RPA_EINVAL_SHAPE, "Sequence %d: kv_len=%d exceeds max_kv_len=%d", s, kv_len, p->max_kv_len);
    if (s >= i && p->max_q_len > 0 && q_len > p->max_q_len)
      return fail(RPA_EINVAL_SHAPE, "Sequence %d: q_len=%d exceeds max_q_len=%d", s, q_len, p->max_q_len);
  }
  return RPA_OK;
}

// Static-shape mode: every sequence may be a decode row, nothing is known about their lengths
// beyond the page-table bound.
static RpaParams planning_view(const RpaParams* p) {
  RpaParams q = *p;
  if (p->distribution) {
    q.decode_end = p->num_seqs;
    q.sum_decode_kv_len = 0;
  }
  return q;
}

namespace {
// Workspace of the balanced decode plan: partial rows, their (max, sum) pairs, the prefix sum of
// the rows' blocks, and one 8-byte arrival word per (row, unit, wave of the workgroup).
struct BalancedLayout {
  size_t ml, cu_blocks, counters, total;  // byte offsets
};
BalancedLayout balanced_layout(const RpaParams* p) {
  const size_t groups = (size_t)decode_wgs(p) * decode_waves_per_wg(p) * 2 * 16;
  const int nw = decode_waves_per_wg(p);
  const size_t units = (size_t)((p->num_kv_heads + nw - 1) / nw) * ((p->num_q_heads / p->num_kv_heads + 15) / 16);
  BalancedLayout l;
  l.ml = groups * p->head_dim * sizeof(float);
  l.cu_blocks = l.ml + groups * 2 * sizeof(float);
  l.counters = (l.cu_blocks + ((size_t)p->decode_end + 1) * sizeof(int32_t) + 7) & ~(size_t)7;
  l.total = l.counters + (size_t)p->decode_end * units * nw * sizeof(unsigned long long);
  return l;
}
std::atomic<unsigned long long> g_decode_generation{1};
}  // namespace

static size_t prefill_optional_workspace(const RpaParams* p);

// What the decode partition cannot run without.
static size_t required_workspace_bytes(const RpaParams* p_in) {
  if (!p_in) return 0;
  const RpaParams pv = planning_view(p_in);
  const RpaParams* p = &pv;
  if (p->decode_end <= 0) return 0;
  if (p->head_dim == 256) return rows256_workspace(p);
  const SplitPlan sp = decode_plan(p);
  if (use_balanced(p, sp))
    return balanced_layout(p).total;
  if (sp.splits <= 1) return 0;
  return (size_t)p->decode_end * sp.splits * p->num_q_heads * (p->head_dim + 2) * sizeof(float);
}

size_t rpa_workspace_bytes(const RpaParams* p) {
  if (!p) return 0;
  return std::max(required_workspace_bytes(p), prefill_optional_workspace(p));
}

int rpa_gather_pages(const RpaParams* p, int32_t seq, void* k_out, void* v_out, int32_t max_tokens,
                     void* stream) {
  int rc = rpa_validate(p);
  if (rc != RPA_OK) return rc;
  if (seq < 0 || seq >= p->num_seqs) return fail(RPA_EINVAL_SHAPE, "seq=%d out of [0, %d)", seq, p->num_seqs);
  if (!k_out || !v_out) return fail(RPA_EINVAL_NULL, "k_out/v_out is NULL");
  rpa::GatherArgs a;
  a.kv = kv_addr(p);
  a.pt = page_table(p);
  a.seq = seq;
  a.Hkv = p->num_kv_heads;
  a.head_bytes = p->head_dim * esize_of(p->kv_dtype);
  a.row_bytes = a.Hkv * a.head_bytes;
  a.k_out = k_out;
  a.v_out = v_out;
  a.max_tokens = max_tokens;
  return check_hip(rpa::launch_gather(a, static_cast<hipStream_t>(stream)), "rpa_gather_pages");
}

int rpa_decode(const RpaParams* p_in, void* stream) {
  int rc = rpa_validate(p_in);
  if (rc != RPA_OK) return rc;
  const RpaParams pv = planning_view(p_in);
  const RpaParams* p = &pv;
  if (p->decode_end <= 0) return RPA_OK;
  if (p->mask_mode == RPA_MASK_CUSTOM) return RPA_OK;  // masked rows all go through the prefill kernel
  if (p->head_dim == 256) return rows256(p, 0, p->decode_end, stream, p->distribution ? 1 : 0);
  const SplitPlan sp = decode_plan(p);
  rpa::DecodeArgs a;
  a.q = static_cast<const uint16_t*>(p->q);
  a.out = static_cast<uint16_t*>(p->out);
  a.kv = kv_addr(p);
  a.pt = page_table(p);
  a.sm = softmax_opts(p);
  a.k_scale = p->k_scale;
  a.v_scale = p->v_scale;
  a.num_rows = p->decode_end;
  a.Hq = p->num_q_heads;
  a.Hkv = p->num_kv_heads;
  a.G = p->num_q_heads / p->num_kv_heads;
  a.chunk = sp.chunk;
  a.max_splits = sp.splits;
  a.fp8 = p->kv_dtype == RPA_KV_FP8_E4M3;
  a.ws_o = nullptr;
  a.ws_ml = nullptr;
  a.cu_blocks = nullptr;
  a.merge_counters = nullptr;
  a.generation = 0;
  a.dist = p->distribution;
  a.balanced = use_balanced(p, sp) ? 1 : 0;
  a.num_wgs = decode_wgs(p);
  a.waves_per_wg = decode_waves_per_wg(p);
  a.min_blocks_per_wave = std::max(1, rpa::tuning().decode_min_chunk / 32);
  a.forced_blocks_per_wave = 0;
  if (p->num_splits > 0) {  // the caller pins the partition: about num_splits pieces for the longest row
    const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                       p->cu_kv_lens != nullptr);
    a.forced_blocks_per_wave = (int32_t)std::max<int64_t>(1, ((bound + 31) / 32 + p->num_splits - 1) / p->num_splits);
  }
  if (a.balanced) {
    const size_t need = required_workspace_bytes(p);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(RPA_EINVAL_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, p->workspace_bytes);
    const BalancedLayout lay = balanced_layout(p);
    char* ws = static_cast<char*>(p->workspace);
    a.ws_o = reinterpret_cast<float*>(ws);
    a.ws_ml = reinterpret_cast<float*>(ws + lay.ml);
    a.cu_blocks = reinterpret_cast<int32_t*>(ws + lay.cu_blocks);
    // Opt-in: the wave that arrives last at a cut row merges it, and the second launch goes.
    // Every workgroup of the balanced grid is resident from the start and ends with its cut
    // piece, so all merges fall at the very end of the kernel, where they cost what the second
    // launch costs, and the written-through partial rows cost more: it measures slower.
    if (rpa::tuning().decode_merge_in_kernel != 0 && (reinterpret_cast<uintptr_t>(ws) & 7) == 0) {
      a.merge_counters = reinterpret_cast<unsigned long long*>(ws + lay.counters);
      // 48 bits, never zero: the arrival words are never cleared, and a word of zeros must not
      // look like this call's
      a.generation = (g_decode_generation.fetch_add(1, std::memory_order_relaxed) % ((1ull << 48) - 1)) + 1;
    }
  } else if (sp.splits > 1) {
    const size_t need = required_workspace_bytes(p);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(RPA_EINVAL_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, p->workspace_bytes);
    a.ws_o = static_cast<float*>(p->workspace);
    a.ws_ml = a.ws_o + (size_t)p->decode_end * sp.splits * p->num_q_heads * p->head_dim;
  }
  return check_hip(rpa::launch_decode(a, static_cast<hipStream_t>(stream)), "rpa_decode");
}

// The prefill kernels' view of a call; false when the call has no chunk for them.
static bool prefill_args(const RpaParams* p, rpa::PrefillArgs& a) {
  const bool dyn = p->distribution != nullptr;
  if (!dyn && p->num_seqs <= p->decode_end && p->mask_mode != RPA_MASK_CUSTOM) return false;
  if (dyn && p->num_seqs <= 0) return false;
  a.head_dim = p->head_dim;
  a.q = static_cast<const uint16_t*>(p->q);
  a.out = static_cast<uint16_t*>(p->out);
  a.kv = kv_addr(p);
  a.pt = page_table(p);
  a.sm = softmax_opts(p);
  a.k_scale = p->k_scale;
  a.v_scale = p->v_scale;
  a.seq_begin = (p->mask_mode == RPA_MASK_CUSTOM || dyn) ? 0 : p->decode_end;  // dyn: the kernels read it
  a.seq_end = p->num_seqs;
  a.dist = p->distribution;
  a.Hq = p->num_q_heads;
  a.Hkv = p->num_kv_heads;
  a.G = p->num_q_heads / p->num_kv_heads;
  a.max_q_len = p->max_q_len > 0 ? p->max_q_len : p->num_tokens;
  a.max_kv_len = p->max_kv_len > 0 ? p->max_kv_len : 0;
  a.fp8 = p->kv_dtype == RPA_KV_FP8_E4M3;
  a.kv_splits = 1;
  a.num_tokens = p->num_tokens;
  a.ws_o = nullptr;
  a.ws_ml = nullptr;
  a.mask_bits = nullptr;
  a.mask_pitch = 0;
  return true;
}

// What a prefill launch can use of the workspace, none of it required: the partial rows of K/V ranges cut into
// pieces (launches that would leave most of the GPU idle), and a custom mask turned into bits by a pre-pass
// (needs a bound on the lengths; RPA_MASK_BITS=0 keeps the kernels on the caller's i32 words).
namespace {
struct PrefillWorkspace {
  int splits;
  int pitch;  // 64-bit words per bit row
  size_t split_bytes, bits_offset, bits_bytes, total;
};
PrefillWorkspace prefill_workspace(const RpaParams* p, const rpa::PrefillArgs& a) {
  PrefillWorkspace w = {};
  w.splits = rpa::prefill_kv_splits(a);
  w.split_bytes = rpa::prefill_split_workspace_bytes(a, w.splits);
  w.bits_offset = (w.split_bytes + 255) & ~(size_t)255;
  if (p->mask_mode == RPA_MASK_CUSTOM && p->head_dim == 128 && p->max_kv_len > 0 && p->num_tokens > 0 &&
      rpa::tuning().mask_bits != 0) {
    w.pitch = (p->max_kv_len + 63) / 64;
    w.bits_bytes = (size_t)p->num_tokens * w.pitch * sizeof(uint64_t);
    if (w.bits_bytes > ((size_t)256 << 20)) w.bits_bytes = 0;  // a batch this large keeps the i32 words
  }
  w.total = w.bits_bytes ? w.bits_offset + w.bits_bytes : w.split_bytes;
  return w;
}
}  // namespace

// Workspace that lets a prefill launch which would leave most of the GPU idle cut its K/V ranges into
// pieces; never required: without it the launch runs whole ranges.
static size_t prefill_optional_workspace(const RpaParams* p) {
  rpa::PrefillArgs a;
  if (!prefill_args(p, a)) return 0;
  if (p->head_dim == 256 && rpa::tuning().prefill_rows256 != 0) return 0;  // the row kernel has its own plan
  return prefill_workspace(p, a).total;
}

int rpa_prefill(const RpaParams* p, void* stream) {
  int rc = rpa_validate(p);
  if (rc != RPA_OK) return rc;
  rpa::PrefillArgs a;
  if (!prefill_args(p, a)) return RPA_OK;
  // 256-wide heads take the flash kernel (two 128-dim halves per row, one workgroup per CU; e4m3
  // caches staged through registers); RPA_PREFILL_ROWS256=1 sends them through the row kernel
  if (p->head_dim == 256 && rpa::tuning().prefill_rows256 != 0)
    return rows256(p, (p->mask_mode == RPA_MASK_CUSTOM || p->distribution) ? 0 : p->decode_end, p->num_seqs, stream,
                   p->distribution ? 2 : 0);
  if (p->workspace && (reinterpret_cast<uintptr_t>(p->workspace) & 15) == 0) {
    // the decode partition is done with the workspace by the time these kernels run (same stream)
    const PrefillWorkspace w = prefill_workspace(p, a);
    char* ws = static_cast<char*>(p->workspace);
    size_t bits_at = 0;
    bool cut = false, bits = false;
    if (w.bits_bytes && p->workspace_bytes >= w.total) {
      bits = true;
      bits_at = w.bits_offset;
      cut = w.splits > 1;
    } else if (w.bits_bytes && p->workspace_bytes >= w.bits_bytes) {
      bits = true;  // room for the bits alone: they save more than the pieces
    } else if (w.splits > 1 && p->workspace_bytes >= w.split_bytes) {
      cut = true;
    }
    if (cut) {
      a.kv_splits = w.splits;
      a.ws_o = reinterpret_cast<float*>(ws);
      a.ws_ml = a.ws_o + (size_t)p->num_tokens * p->num_q_heads * w.splits * p->head_dim;
    }
    if (bits) {
      a.mask_bits = reinterpret_cast<uint64_t*>(ws + bits_at);
      a.mask_pitch = w.pitch;
    }
  }
  return check_hip(rpa::launch_prefill(a, static_cast<hipStream_t>(stream)), "rpa_prefill");
}

int rpa_attention(const RpaParams* p, void* stream) {
  int rc = rpa_decode(p, stream);
  if (rc != RPA_OK) return rc;
  return rpa_prefill(p, stream);
}

int rpa_describe_plan(const RpaParams* p_in, char* buf, size_t len) {
  int rc = rpa_validate(p_in);
  if (rc != RPA_OK) return rc;
  if (!buf || len == 0) return fail(RPA_EINVAL_NULL, "buf is NULL or empty");
  const RpaParams pv = planning_view(p_in);
  const RpaParams* p = &pv;
  size_t at = 0;
  auto put = [&](const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    const size_t from = std::min(at, len - 1);
    const int n = vsnprintf(buf + from, len - from, fmt, ap);
    va_end(ap);
    if (n > 0) at += (size_t)n;
  };
  buf[0] = 0;
  if (p->decode_end > 0 && p->mask_mode != RPA_MASK_CUSTOM) {
    const rpa::ShapeRule& r = decode_shape(p);
    if (p->head_dim == 256) {
      const SplitPlan sp = rows256_plan(p);
      put("decode: shape=%s kernel=rpa_rows256_kernel rows=%d pieces_per_row=%d", r.name, p->decode_end, sp.splits);
    } else {
      const SplitPlan sp = decode_plan(p);
      const bool bal = use_balanced(p, sp);
      put("decode: shape=%s kernel=%s rows=%d waves_per_wg=%d", r.name,
          bal ? "rpa_decode_balanced_kernel" : "rpa_decode_splitkv_kernel", p->decode_end, decode_waves_per_wg(p));
      if (bal) put(" resident_waves=%d merge=rpa_combine_balanced_kernel", decode_wave_capacity(p));
      else put(" pieces_per_row=%d chunk=%d merge=%s", sp.splits, sp.chunk, sp.splits > 1 ? "rpa_combine_kernel" : "none");
    }
    put(" workspace=%zu\n", required_workspace_bytes(p_in));
  }
  rpa::PrefillArgs a;
  if (prefill_args(p_in, a)) {
    if (p->head_dim == 256 && rpa::tuning().prefill_rows256 != 0) {
      put("prefill: kernel=rpa_rows256_kernel (RPA_PREFILL_ROWS256)\n");
    } else {
      const rpa::ShapeRule& r = rpa::prefill_shape_of(a);
      const char* kernel = r.kernel == rpa::kKernelPrefillPipe ? "rpa_prefill_pipe_kernel"
                           : (r.kernel == rpa::kKernelPrefillStaged ? "rpa_prefill_staged_kernel" : "rpa_prefill_async_kernel");
      const PrefillWorkspace w = prefill_workspace(p_in, a);
      put("prefill: shape=%s kernel=%s tile=%dx%dx%d kv_pieces_with_workspace=%d mask_bits=%s optional_workspace=%zu\n",
          r.name, kernel, r.tile_q, r.tile_heads, r.tile_kv, w.splits, w.bits_bytes ? "yes" : "no", w.total);
    }
  }
  return (int)std::min<size_t>(at, 0x7fffffff);
}

size_t rpa_noalloc_max_workspace_bytes(void) { return kNoAllocScratchBytes; }

int rpa_attention_noalloc(const RpaParams* p, void* stream) {
  int rc = rpa_validate(p);
  if (rc != RPA_OK) return rc;
  const size_t need = required_workspace_bytes(p);  // (a prefill launch cuts its K/V ranges only if the array has the room)
  if (need > kNoAllocScratchBytes)
    return fail(RPA_EINVAL_WORKSPACE,
                "this batch needs a split-KV workspace of %zu bytes, the built-in one holds %zu: call rpa_attention "
                "with a workspace of your own",
                need, kNoAllocScratchBytes);
  RpaParams q = *p;
  q.workspace = nullptr;
  q.workspace_bytes = 0;
  if (need > 0 || prefill_optional_workspace(p) > 0) {
    void* ptr = nullptr;
    if ((rc = noalloc_scratch(&ptr)) != RPA_OK) return rc;
    q.workspace = ptr;  // the device address, never the array's name
    q.workspace_bytes = kNoAllocScratchBytes;
  }
  // Nothing in the workspace has to start at zero: partial rows, their (max, sum) pairs and the block
  // prefix sums are all written by the decode kernel before the merge pass reads them.
  return rpa_attention(&q, stream);
}

int rpa_kv_write(const RpaParams* p, const void* keys, const void* values, void* stream) {
  int rc = rpa_validate(p);
  if (rc != RPA_OK) return rc;
  if (!keys || !values) return fail(RPA_EINVAL_NULL, "keys/values is NULL");
  rpa::KvWriteArgs a;
  a.kv = kv_addr(p);
  a.pt = page_table(p);
  a.keys = static_cast<const char*>(keys);
  a.values = static_cast<const char*>(values);
  a.num_seqs = p->num_seqs;
  a.dist = p->distribution;
  a.Hkv = p->num_kv_heads;
  a.head_bytes = p->head_dim * esize_of(p->kv_dtype);
  a.num_tokens = p->num_tokens;
  return check_hip(rpa::launch_kv_write(a, static_cast<hipStream_t>(stream)), "rpa_kv_write");
}

// ---------------------------------------------------------------- MLA ----

static int mla_wgs();

static SplitPlan mla_plan(const RpaMlaParams* p, int64_t rows) {
  const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                     p->cu_kv_lens != nullptr);
  // one 8-wave workgroup per (row, split, 128 heads) and per CU; every split costs a 256 KiB
  // partial write per 128 heads, so splits are kept as few as fill the CUs once
  const int64_t groups = (p->num_q_heads + 127) / 128;
  const int64_t units = rows * groups;
  int64_t work = p->sum_kv_len > 0 ? p->sum_kv_len * groups : 0;
  if (p->sliding_window > 0) work = 0;
  return plan_splits(bound, p->sliding_window, units, work, p->num_splits,
                     rpa::tuning().mla_min_chunk, mla_wgs());
}

static int mla_validate(const RpaMlaParams* p) {
  if (!p) return fail(RPA_EINVAL_NULL, "params is NULL");
  if (p->num_seqs < 0 || p->num_q_heads <= 0 || p->page_size <= 0 || p->total_pages <= 0)
    return fail(RPA_EINVAL_SHAPE, "expected positive shape");
  if (p->lkv_dim != 512 || p->rope_dim != 64)
    return fail(RPA_EUNSUPPORTED, "lkv_dim=%d rope_dim=%d: only 512+64 is built", p->lkv_dim, p->rope_dim);
  if (p->row_stride < p->rope_offset + p->rope_dim || p->rope_offset < p->lkv_dim || (p->row_stride % 8) != 0 ||
      (p->rope_offset % 8) != 0)
    return fail(RPA_EINVAL_SHAPE, "row_stride=%d rope_offset=%d do not describe [kv_c | k_pe]", p->row_stride, p->rope_offset);
  if (p->cache_dtype != RPA_KV_BF16 && p->cache_dtype != RPA_KV_FP8_E4M3)
    return fail(RPA_EINVAL_SHAPE, "cache_dtype=%d is neither RPA_KV_BF16 nor RPA_KV_FP8_E4M3", p->cache_dtype);
  if (p->cache_dtype == RPA_KV_FP8_E4M3 && ((p->row_stride % 16) != 0 || (p->rope_offset % 16) != 0))
    return fail(RPA_EINVAL_SHAPE, "fp8 latent rows: row_stride=%d and rope_offset=%d must be multiples of 16", p->row_stride,
                p->rope_offset);
  if (p->sliding_window < 0) return fail(RPA_EINVAL_WINDOW, "sliding_window=%d must be positive", p->sliding_window);
  if (p->num_seqs > 0 && (!p->ql_nope || !p->q_pe || !p->out || !p->cache_kv || !p->kv_lens || !p->page_indices || !p->cu_q_lens))
    return fail(RPA_EINVAL_NULL, "a required buffer is NULL");
  if (!p->cu_kv_lens && p->pages_per_seq <= 0 && p->num_seqs > 0)
    return fail(RPA_EINVAL_SHAPE, "padded page table needs pages_per_seq > 0");
  return RPA_OK;
}

static int mla_wgs() {
  const int forced = rpa::tuning().mla_wg_capacity;
  return std::max(1, forced > 0 ? forced : wave_capacity() / 8);
}

// same criteria as the MHA decode path: ragged sequence rows that need splitting
static bool mla_use_balanced(const RpaMlaParams* p, const SplitPlan& fixed, bool token_rows) {
  const bool on = rpa::tuning().mla_balanced != 0;
  if (!on || token_rows || p->num_splits == 1) return false;
  // Rows the fixed plan leaves whole: one workgroup job per row.  With many more jobs than
  // workgroup slots the dispatcher evens them out by itself; with up to two per slot the kernel
  // ends with the longest rows, and dealing the tiles out evenly pays (300 rows of 1000..8000
  // tokens: 832 -> 673 us; 256 rows of 2048..16384: 1214 -> 1013 us; 1000 rows of 200..2000:
  // 617 -> 659 us, so not there).
  if (fixed.splits <= 1 && (int64_t)p->num_seqs * ((p->num_q_heads + 127) / 128) > 2 * (int64_t)mla_wgs()) return false;
  if (p->num_splits > 0) return true;
  const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                     p->cu_kv_lens != nullptr);
  const int64_t units = (p->num_q_heads + 127) / 128;
  const int64_t min_tiles = std::max(1, rpa::tuning().mla_min_chunk / 32);
  if ((int64_t)p->num_seqs * ((bound + 31) / 32) * units <= (int64_t)mla_wgs() * min_tiles) return false;
  const bool equal_lengths = p->sum_kv_len > 0 && p->max_kv_len > 0 &&
                             p->sum_kv_len == (int64_t)p->num_seqs * p->max_kv_len;
  return !equal_lengths;
}

static size_t mla_workspace(const RpaMlaParams* p, int64_t rows, bool token_rows) {
  if (!p || p->num_seqs <= 0 || rows <= 0) return 0;
  const SplitPlan sp = mla_plan(p, rows);
  if (mla_use_balanced(p, sp, token_rows))
    return (size_t)mla_wgs() * 2 * 128 * (p->lkv_dim + 2) * sizeof(float) + ((size_t)p->num_seqs + 1) * sizeof(int32_t);
  if (sp.splits <= 1) return 0;
  return (size_t)rows * sp.splits * p->num_q_heads * (p->lkv_dim + 2) * sizeof(float);
}

size_t rpa_mla_workspace_bytes(const RpaMlaParams* p) { return mla_workspace(p, p ? p->num_seqs : 0, false); }

size_t rpa_mla_attention_workspace_bytes(const RpaMlaParams* p) {
  return mla_workspace(p, p ? p->num_tokens : 0, true);
}

static int mla_run(const RpaMlaParams* p, void* stream, bool token_rows) {
  int rc = mla_validate(p);
  if (rc != RPA_OK) return rc;
  if (p->num_seqs <= 0) return RPA_OK;
  if (!token_rows && p->num_seqs > p->num_tokens)
    return fail(RPA_EINVAL_SHAPE, "decode rows=%d exceed tokens=%d", p->num_seqs, p->num_tokens);
  const int64_t rows = token_rows ? p->num_tokens : p->num_seqs;
  if (rows <= 0) return RPA_OK;
  const SplitPlan sp = mla_plan(p, rows);
  rpa::MlaDecodeArgs a;
  a.ql_nope = static_cast<const uint16_t*>(p->ql_nope);
  a.q_pe = static_cast<const uint16_t*>(p->q_pe);
  a.out = static_cast<uint16_t*>(p->out);
  a.cache = static_cast<const char*>(p->cache_kv);
  a.pt.kv_lens = p->kv_lens;
  a.pt.page_indices = p->page_indices;
  a.pt.cu_q_lens = p->cu_q_lens;
  a.pt.cu_kv_lens = p->cu_kv_lens;
  a.pt.pages_per_seq = p->pages_per_seq;
  a.pt.page_size = p->page_size;
  // the scalar scales of the logits fold into sm_scale (they multiply the dot product before the soft cap)
  const float logit_scale = p->sm_scale * (p->k_scale > 0.f ? p->k_scale : 1.0f) * (p->q_scale > 0.f ? p->q_scale : 1.0f);
  a.sm = softmax_opts(logit_scale, p->soft_cap, p->mask_value, p->sliding_window);
  a.out_scale = p->v_scale > 0.f ? p->v_scale : 1.0f;
  a.dist = p->distribution;
  a.fp8 = p->cache_dtype == RPA_KV_FP8_E4M3 ? 1 : 0;
  if (p->distribution && !token_rows)
    return fail(RPA_EUNSUPPORTED, "rpa_mla_decode takes the batch composition from the host: use rpa_mla_attention");
  a.num_rows = (int32_t)rows;
  a.num_seqs = p->num_seqs;
  a.rows_are_tokens = token_rows ? 1 : 0;
  a.Hq = p->num_q_heads;
  a.row_stride = p->row_stride;
  a.rope_offset = p->rope_offset;
  a.chunk = sp.chunk;
  a.max_splits = sp.splits;
  a.ws_o = nullptr;
  a.ws_ml = nullptr;
  a.cu_tiles = nullptr;
  a.balanced = mla_use_balanced(p, sp, token_rows) ? 1 : 0;
  a.num_wgs = mla_wgs();
  a.min_tiles_per_wg = std::max(1, rpa::tuning().mla_min_chunk / 32);
  a.forced_tiles_per_wg = 0;
  a.piece_pad = rpa::tuning().mla_piece_pad >= 0
                    ? rpa::tuning().mla_piece_pad
                    : rpa::select_shape(rpa::mla_shape_key(a), rpa::mla_shape_skip(rpa::tuning())).piece_pad;
  if (p->num_splits > 0) {
    const int64_t bound = kv_len_bound(p->max_kv_len, p->pages_per_seq, p->page_size, p->total_pages,
                                       p->cu_kv_lens != nullptr);
    a.forced_tiles_per_wg = (int32_t)std::max<int64_t>(1, ((bound + 31) / 32 + p->num_splits - 1) / p->num_splits);
  }
  if (a.balanced) {
    const size_t need = mla_workspace(p, rows, token_rows);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(RPA_EINVAL_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, p->workspace_bytes);
    // partial rows are bf16 (the workspace is sized for f32 rows: room to spare)
    a.ws_o = static_cast<uint16_t*>(p->workspace);
    a.ws_ml = reinterpret_cast<float*>(a.ws_o + (size_t)a.num_wgs * 2 * 128 * p->lkv_dim);
    a.cu_tiles = reinterpret_cast<int32_t*>(a.ws_ml + (size_t)a.num_wgs * 2 * 128 * 2);
  } else if (sp.splits > 1) {
    const size_t need = mla_workspace(p, rows, token_rows);
    if (!p->workspace || p->workspace_bytes < need)
      return fail(RPA_EINVAL_WORKSPACE, "workspace of %zu bytes needed, %zu given", need, p->workspace_bytes);
    a.ws_o = static_cast<uint16_t*>(p->workspace);
    a.ws_ml = reinterpret_cast<float*>(a.ws_o + (size_t)rows * sp.splits * p->num_q_heads * p->lkv_dim);
  }
  return check_hip(rpa::launch_mla_decode(a, static_cast<hipStream_t>(stream)),
                   token_rows ? "rpa_mla_attention" : "rpa_mla_decode");
}

int rpa_mla_describe_plan(const RpaMlaParams* p, int token_rows, char* buf, size_t len) {
  int rc = mla_validate(p);
  if (rc != RPA_OK) return rc;
  if (!buf || len == 0) return fail(RPA_EINVAL_NULL, "buf is NULL or empty");
  const int64_t rows = token_rows ? p->num_tokens : p->num_seqs;
  rpa::MlaDecodeArgs a = {};
  a.pt.page_size = p->page_size;
  a.sm.soft_cap = p->soft_cap;
  a.fp8 = p->cache_dtype == RPA_KV_FP8_E4M3 ? 1 : 0;
  a.Hq = p->num_q_heads;
  a.row_stride = p->row_stride;
  const rpa::ShapeRule& r = rpa::select_shape(rpa::mla_shape_key(a), rpa::mla_shape_skip(rpa::tuning()));
  const SplitPlan sp = mla_plan(p, std::max<int64_t>(rows, 1));
  const bool bal = rows > 0 && mla_use_balanced(p, sp, token_rows != 0);
  a.sm.window = p->sliding_window;
  a.num_rows = (int32_t)rows;
  a.num_seqs = p->num_seqs;
  a.rows_are_tokens = token_rows ? 1 : 0;
  a.max_splits = sp.splits;
  a.balanced = bal ? 1 : 0;
  static const char* const kGroups[] = {"off", "eight_waves_compiled", "eight_waves", "wide"};
  const int tg = rpa::mla_token_group_mode(a, rpa::tuning(), r);
  return snprintf(buf, len, "mla: shape=%s rows=%lld waves_per_wg=%d heads_per_wg=%d share=%d token_groups=%s plan=%s "
                  "pieces_per_row=%d workgroups=%d workspace=%zu\n",
                  r.name, (long long)rows, tg == 3 ? 4 : r.waves_per_wg, tg ? 128 : r.tile_heads, tg ? 1 : r.share, kGroups[tg],
                  bal ? "balanced" : "fixed", bal ? 0 : sp.splits, bal ? mla_wgs() : 0,
                  mla_workspace(p, rows, token_rows != 0));
}

int rpa_mla_decode(const RpaMlaParams* p, void* stream) { return mla_run(p, stream, false); }

int rpa_mla_attention(const RpaMlaParams* p, void* stream) { return mla_run(p, stream, true); }

int rpa_mla_kv_write(const RpaMlaParams* p, const void* new_kv_c, const void* new_k_pe, void* stream) {
  int rc = mla_validate(p);
  if (rc != RPA_OK) return rc;
  if (!new_kv_c || !new_k_pe) return fail(RPA_EINVAL_NULL, "new_kv_c/new_k_pe is NULL");
  if (p->num_seqs <= 0 || p->num_tokens <= 0) return RPA_OK;
  rpa::MlaWriteArgs a;
  a.cache = static_cast<char*>(const_cast<void*>(p->cache_kv));
  a.pt.kv_lens = p->kv_lens;
  a.pt.page_indices = p->page_indices;
  a.pt.cu_q_lens = p->cu_q_lens;
  a.pt.cu_kv_lens = p->cu_kv_lens;
  a.pt.pages_per_seq = p->pages_per_seq;
  a.pt.page_size = p->page_size;
  a.new_kv_c = static_cast<const char*>(new_kv_c);
  a.new_k_pe = static_cast<const char*>(new_k_pe);
  a.fp8 = p->cache_dtype == RPA_KV_FP8_E4M3 ? 1 : 0;
  a.num_tokens = p->num_tokens;
  a.num_seqs = p->num_seqs;
  a.dist = p->distribution;
  a.row_stride = p->row_stride;
  a.rope_offset = p->rope_offset;
  return check_hip(rpa::launch_mla_kv_write(a, static_cast<hipStream_t>(stream)), "rpa_mla_kv_write");
}

}  // extern "C"
