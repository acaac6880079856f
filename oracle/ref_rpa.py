"""CPU restatement of the reference's pure-jnp ragged paged attention.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  The product path never touches this module.

Every function names the reference lines it follows (paths relative to the
reference checkout):

  rpa_v3 = python/sgl_jax/srt/kernels/ragged_paged_attention/ragged_paged_attention_v3.py
  rpa_v1 = python/sgl_jax/srt/kernels/ragged_paged_attention/ragged_paged_attention.py
  pool   = python/sgl_jax/srt/mem_cache/memory_pool.py
  paged  = python/sgl_jax/srt/kernels/paged_attention/paged_attention.py
  fa     = python/sgl_jax/srt/layers/attention/flashattention_backend.py

The arithmetic is torch-CPU float32 with bfloat16 rounding at exactly the
points where the reference rounds.  Parity status of each function (what pins
it, independent of this file's own formulae) is listed in tests/test_oracle_*.py:
the reference ships no stored vectors for attention, so the pins are
torch.nn.functional.scaled_dot_product_attention, a float64 scalar-loop brute
force, closed forms and invariants.  Options with no such pin are marked
"parity unpinned" below.
"""

from __future__ import annotations

import math

import numpy as np
import torch

# rpa_v3:47  DEFAULT_MASK_VALUE = -0.7 * finfo(float32).max
DEFAULT_MASK_VALUE = -0.7 * float(np.finfo(np.float32).max)


def cdiv(a: int, b: int) -> int:
    """kernels/ragged_paged_attention/util.py:7-9."""
    assert b != 0
    return (a + b - 1) // b


def align_to(x: int, a: int) -> int:
    """kernels/ragged_paged_attention/util.py:12-13."""
    return cdiv(x, a) * a


def _as_int(x) -> int:
    if isinstance(x, torch.Tensor):
        return int(x.item())
    return int(x)


def _per_head_scale(scale, num_kv_heads: int):
    """Scalar (reference, rpa_v3:1686-1687) or per-kv-head vector (generalisation
    used by the fp8 config) -> float32 tensor broadcastable over [kv, Hkv, D]."""
    if scale is None:
        return None
    s = torch.as_tensor(scale, dtype=torch.float32).reshape(-1)
    if s.numel() == 1:
        s = s.expand(num_kv_heads)
    assert s.numel() == num_kv_heads
    return s.reshape(1, num_kv_heads, 1)


def _attend_one_sequence(
    q,  # [q_len, Hq, D]  q dtype
    k,  # [kv_len, Hkv, D]
    v,  # [kv_len, Hkv, D]
    *,
    causal,
    custom_mask_row,  # None or flat [q_len*kv_len] ints
    sm_scale,
    sliding_window,
    soft_cap,
    mask_value,
    k_scale,
    v_scale,
    xai_temperature_len,
    attention_sink,
    softmax_dtype,
):
    """Body of the per-sequence loop, rpa_v3:131-200 (same order of operations)."""
    q_len, num_q_heads, head_dim = q.shape
    kv_len, num_kv_heads, _ = k.shape
    group = num_q_heads // num_kv_heads
    # rpa_v3:140-145 -- dequantise then ROUND to q dtype
    if k_scale is not None:
        k = (k.to(torch.float32) * k_scale).to(q.dtype)
    if v_scale is not None:
        v = (v.to(torch.float32) * v_scale).to(q.dtype)
    out = torch.empty((q_len, num_q_heads, v.shape[-1]), dtype=q.dtype)

    q_span = (kv_len - q_len) + torch.arange(q_len, dtype=torch.int64)[:, None]  # rpa_v3:150
    kv_span = torch.arange(kv_len, dtype=torch.int64)[None, :]  # rpa_v3:151
    if causal:
        mask = q_span < kv_span  # rpa_v3:153
    elif custom_mask_row is not None:
        mask = custom_mask_row.reshape(q_len, kv_len) < 1  # rpa_v3:154-163
    else:
        mask = torch.zeros((q_len, kv_len), dtype=torch.bool)  # rpa_v3:165
    if sliding_window is not None:
        mask = mask | (q_span - sliding_window >= kv_span)  # rpa_v3:166-167
    add_mask = torch.where(mask, torch.tensor(mask_value, dtype=torch.float32), torch.tensor(0.0))

    temp = None
    if xai_temperature_len is not None:  # rpa_v3:171-177
        qidx = torch.arange(kv_len - q_len, kv_len)
        scale = 1.0 / math.log2(float(xai_temperature_len))
        qtemp = torch.log2(qidx.to(torch.float32)) * scale
        temp = torch.where(qidx > xai_temperature_len, qtemp, torch.tensor(1.0))

    sink = None
    if attention_sink is not None:  # rpa_v3:185-193
        sink = torch.as_tensor(attention_sink, dtype=torch.float32).reshape(-1)
        if sink.numel() == 1:
            sink = sink.expand(num_q_heads)

    # jnp.repeat(k, G, axis=1) (rpa_v3:146-147): q head h reads kv head h // G.
    # Looping over kv heads bounds the [G, q, kv] score block without changing
    # any value.
    for hk in range(num_kv_heads):
        hq = slice(hk * group, (hk + 1) * group)
        qf = q[:, hq].to(torch.float32)  # [q, G, D]
        kf = k[:, hk].to(torch.float32)  # [kv, D]
        vf = v[:, hk].to(torch.float32)
        attn = torch.einsum("qgd,kd->gqk", qf, kf)  # rpa_v3:148 (f32 accumulate)
        attn = attn * sm_scale  # rpa_v3:149
        if soft_cap is not None:
            attn = soft_cap * torch.tanh(attn / soft_cap)  # rpa_v3:168-169
        if temp is not None:
            attn = attn * temp[None, :, None]
        attn = attn + add_mask[None]  # rpa_v3:179 (additive)
        if softmax_dtype is not None:
            attn = attn.to(softmax_dtype)  # rpa_v3:182-183 (parity unpinned)
        if sink is not None:
            col = sink[hq].to(attn.dtype).reshape(group, 1, 1).expand(group, q_len, 1)
            attn = torch.cat([col, attn], dim=-1)
            attn = torch.softmax(attn, dim=-1)[..., 1:]  # rpa_v3:194-196
        else:
            attn = torch.softmax(attn, dim=-1)  # rpa_v3:198
        o = torch.einsum("gqk,kd->qgd", attn.to(torch.float32), vf)  # rpa_v3:199
        out[:, hq] = o.to(q.dtype)
    return out


def ref_ragged_paged_attention(
    queries: torch.Tensor,  # [padded_num_tokens, Hq, D]
    k_pages: torch.Tensor,  # [total_pages, P, Hkv, D]
    v_pages: torch.Tensor,  # [total_pages, P, Hkv, D]
    kv_lens: torch.Tensor,  # i32[S]
    page_indices: torch.Tensor,  # i32[S, pages_per_seq]  (2-D, zero padded)
    cu_q_lens: torch.Tensor,  # i32[S+1]
    num_seqs,  # i32[1]
    *,
    custom_mask: torch.Tensor | None = None,
    causal: bool = True,
    sm_scale: float = 1.0,
    sliding_window: int | None = None,
    soft_cap: float | None = None,
    mask_value: float | None = DEFAULT_MASK_VALUE,
    k_scale=None,
    v_scale=None,
    xai_temperature_len: float | None = None,
    attention_sink=None,
    softmax_dtype=None,
) -> torch.Tensor:
    """rpa_v3:94-202.  Returns [sum(q_len), Hq, D] (not padded to T)."""
    if mask_value is None:
        mask_value = DEFAULT_MASK_VALUE
    _, page_size, num_kv_heads, head_dim = k_pages.shape
    num_q_heads = queries.shape[1]
    assert num_q_heads % num_kv_heads == 0
    n = _as_int(num_seqs[0]) if not isinstance(num_seqs, int) else num_seqs
    ks = _per_head_scale(k_scale, num_kv_heads)
    vs = _per_head_scale(v_scale, num_kv_heads)

    # rpa_v3:124-129 cumulative custom-mask offsets
    cu_mask = [0]
    for i in range(n):
        q_len = _as_int(cu_q_lens[i + 1]) - _as_int(cu_q_lens[i])
        cu_mask.append(cu_mask[-1] + q_len * _as_int(kv_lens[i]))

    outputs = []
    for i in range(n):
        q_start, q_end = _as_int(cu_q_lens[i]), _as_int(cu_q_lens[i + 1])
        kv_len = _as_int(kv_lens[i])
        indices = page_indices[i].to(torch.int64)
        q = queries[q_start:q_end]
        # rpa_v3:138-139: gather the whole page-id row, flatten, trim to kv_len
        k = k_pages[indices].reshape(-1, num_kv_heads, head_dim)[:kv_len]
        v = v_pages[indices].reshape(-1, num_kv_heads, head_dim)[:kv_len]
        row = None
        if (not causal) and custom_mask is not None:
            row = custom_mask[cu_mask[i] : cu_mask[i + 1]]
        outputs.append(
            _attend_one_sequence(
                q,
                k,
                v,
                causal=causal,
                custom_mask_row=row,
                sm_scale=sm_scale,
                sliding_window=sliding_window,
                soft_cap=soft_cap,
                mask_value=mask_value,
                k_scale=ks,
                v_scale=vs,
                xai_temperature_len=xai_temperature_len,
                attention_sink=attention_sink,
                softmax_dtype=softmax_dtype,
            )
        )
    if not outputs:
        return queries[:0].clone()
    return torch.cat(outputs, dim=0)  # rpa_v3:202


def quantise_queries(q: torch.Tensor, q_scale: float, kv_dtype: torch.dtype) -> torch.Tensor:
    """Query quantisation of the reference's kernel, rpa_v3:463-470 (the pure-jnp
    function has no q_scale; the logits are then multiplied by q_scale, :477-478,
    which a caller of this oracle folds into sm_scale).  ``q / q_scale`` is a bf16
    array there (a bf16 array divided by a Python float keeps its type); it is
    clipped to the finite range of the cache's element type and cast to it.
    Returned in q's dtype (every e4m3 value is a bf16 value).  Parity unpinned by
    reference-held data; pinned by grid membership, range and idempotence."""
    x = q / q_scale
    if kv_dtype.is_floating_point:
        info = torch.finfo(kv_dtype)
        x = torch.clamp(x.to(torch.float32), min=float(info.min), max=float(info.max)).to(q.dtype)
    return x.to(kv_dtype).to(q.dtype)


def split_fused_cache(kv_pages_fused: torch.Tensor):
    """rpa_v1:74-76: heads are stored K0,V0,K1,V1,...; K = [:, :, 0::2], V = [:, :, 1::2]."""
    return kv_pages_fused[:, :, 0::2, :], kv_pages_fused[:, :, 1::2, :]


def merge_kv(k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """pool:56-91 without the TPU packing reshape: [N, Hkv, D] x2 -> [N, 2*Hkv, D]
    with K/V interleaved per head (memory-identical to the reference's 5-D view)."""
    assert k.shape == v.shape
    n, h, d = k.shape
    return torch.stack([k, v], dim=2).reshape(n, 2 * h, d)


def ref_ragged_paged_attention_fused(
    queries, kv_pages_fused, kv_lens, page_indices, cu_q_lens, num_seqs, **kw
) -> torch.Tensor:
    """rpa_v1:35-119: identical mathematics on the head-interleaved cache."""
    k_pages, v_pages = split_fused_cache(kv_pages_fused)
    return ref_ragged_paged_attention(
        queries, k_pages, v_pages, kv_lens, page_indices, cu_q_lens, num_seqs, **kw
    )


def ragged_to_padded_page_table(page_indices_flat, cu_kv_lens, page_size, num_seqs, pages_per_seq=None):
    """Production page table (flat; sequence i owns the entries starting at
    cdiv(cu_kv_lens[i], P), rpa_v3:636-637) -> the oracle's zero-padded 2-D table
    (rpa_v3:99)."""
    flat = torch.as_tensor(page_indices_flat).to(torch.int64)
    cu = [int(x) for x in cu_kv_lens]
    counts = [cdiv(cu[i + 1], page_size) - cdiv(cu[i], page_size) for i in range(num_seqs)]
    width = pages_per_seq if pages_per_seq is not None else max(counts + [1])
    table = torch.zeros((num_seqs, width), dtype=torch.int32)
    for i in range(num_seqs):
        start = cdiv(cu[i], page_size)
        table[i, : counts[i]] = flat[start : start + counts[i]].to(torch.int32)
    return table


def gather_pages(pages: torch.Tensor, page_row, kv_len: int) -> torch.Tensor:
    """The gather of rpa_v3:138 on its own: pages[page_row].reshape(-1, ...)[:kv_len]."""
    idx = torch.as_tensor(page_row).to(torch.int64)
    g = pages[idx]
    return g.reshape((-1,) + tuple(pages.shape[2:]))[:kv_len]


def lse_combine(partial_out, partial_l, partial_m):
    """paged:292-303 (split-KV merge, natural-exp form, without the eps guard):
    m* = max_j m_j;  out = sum_j o_j e^{m_j-m*} / sum_j l_j e^{m_j-m*}.
    partial_out [n_splits, ..., D] holds UNNORMALISED accumulators."""
    m_next = partial_m.max(dim=0).values
    corr = torch.exp(partial_m - m_next[None])
    num = (partial_out * corr[..., None]).sum(dim=0)
    den = (partial_l * corr).sum(dim=0)
    return num / den[..., None]


# --------------------------------------------------------------------------
# Host metadata (fa:168-224), restated for dp_size == 1.
# --------------------------------------------------------------------------
def ref_forward_metadata(cache_loc, seq_lens, extend_seq_lens, page_size, is_decode):
    """fa:168-224 with dp_size=1: page_indices = cache_loc[::P] // P;
    cu_q_lens = arange (decode) or cumsum(extend lens); cu_kv_lens = cumsum of
    page-aligned seq lens; distribution = (n,n,n) decode / (0,n,n) extend with
    n = #(seq_lens > 0)."""
    cache_loc = np.asarray(cache_loc)
    seq_lens = np.asarray(seq_lens)
    page_indices = (cache_loc[::page_size] // page_size).astype(np.int32)
    bs = len(seq_lens)
    if is_decode:
        cu_q = np.arange(bs + 1, dtype=np.int32)
    else:
        cu_q = np.zeros(bs + 1, dtype=np.int32)
        cu_q[1:] = np.cumsum(np.asarray(extend_seq_lens))
    aligned = ((seq_lens + page_size - 1) // page_size) * page_size
    cu_kv = np.zeros(bs + 1, dtype=np.int32)
    cu_kv[1:] = np.cumsum(aligned)
    n = int(np.sum(seq_lens > 0))
    dist = np.array([n, n, n] if is_decode else [0, n, n], dtype=np.int32)
    return page_indices, cu_q, cu_kv, dist
