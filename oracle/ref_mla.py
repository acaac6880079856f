"""CPU restatement of the reference's absorbed-MLA ragged paged attention.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows python/sgl_jax/srt/kernels/mla/v1/ref.py (``mla_ref`` below) of the
reference.  Two cache layouts are accepted:

* ``padded``  -- the reference's [pages, P, align128(lkv)+align128(rope)]
  (mla_ref:41-53; P/packing and packing axes merged, which is memory-identical);
* ``compact`` -- [pages, P, lkv+rope] contiguous, the 576-wide latent row of the
  DeepSeek-V3 decode workload.  Zero padding contributes nothing to q.k, so
  both layouts give identical scores (tests/test_oracle_mla.py checks this).
"""

from __future__ import annotations

import torch

from .ref_rpa import DEFAULT_MASK_VALUE, align_to, cdiv, _as_int


def mla_update_kv_cache(new_kv_c, new_k_pe, cache_kv, kv_lens, page_indices, cu_q_lens, num_seqs, lkv_dim_in_cache):
    """mla_ref:56-105: write each sequence's q_len new latent rows at positions
    kv_len-q_len .. kv_len-1 through the padded page table
    (page_indices[i*pages_per_seq + pos // P]).  cache_kv is [pages, P, width]."""
    cache = cache_kv.clone()
    page_size = cache.shape[1]
    max_num_seqs = kv_lens.shape[0]
    pages_per_seq = page_indices.shape[0] // max_num_seqs
    lkv = new_kv_c.shape[1]
    r = new_k_pe.shape[1]
    for i in range(num_seqs):
        q_start, q_end = _as_int(cu_q_lens[i]), _as_int(cu_q_lens[i + 1])
        q_len = q_end - q_start
        kv_len = _as_int(kv_lens[i])
        for j in range(q_len):
            pos = kv_len - q_len + j
            page = _as_int(page_indices[i * pages_per_seq + pos // page_size])
            row = pos % page_size
            cache[page, row, :lkv] = new_kv_c[q_start + j]
            cache[page, row, lkv_dim_in_cache : lkv_dim_in_cache + r] = new_k_pe[q_start + j]
    return cache


def ref_mla_ragged_paged_attention(
    ql_nope: torch.Tensor,  # [T, Hq, lkv]
    q_pe: torch.Tensor,  # [T, Hq, rope]
    new_kv_c: torch.Tensor | None,  # [T, lkv] or None (cache already holds every token)
    new_k_pe: torch.Tensor | None,  # [T, rope]
    cache_kv: torch.Tensor,  # [pages, P, width]
    kv_lens: torch.Tensor,  # i32[S]
    page_indices: torch.Tensor,  # i32[S * pages_per_seq]  (padded layout, mla_ref:197-200)
    cu_q_lens: torch.Tensor,  # i32[S+1]
    distribution,  # i32[3]
    *,
    sm_scale: float = 1.0,
    sliding_window: int | None = None,
    soft_cap: float | None = None,
    mask_value: float | None = DEFAULT_MASK_VALUE,
    q_scale: float | None = None,
    k_scale: float | None = None,
    v_scale: float | None = None,
    layout: str = "compact",
):
    """mla_ref:108-248.  Returns (out [sum q_len, Hq, lkv], updated cache)."""
    if mask_value is None:
        mask_value = DEFAULT_MASK_VALUE
    lkv = ql_nope.shape[-1]
    rope = q_pe.shape[-1]
    width = cache_kv.shape[-1]
    if layout == "padded":
        lkv_c = align_to(lkv, 128)
        assert width == lkv_c + align_to(rope, 128)  # mla_ref:183
    else:
        lkv_c = lkv
        assert width == lkv + rope
    n = _as_int(distribution[-1])
    if new_kv_c is not None:
        cache_kv = mla_update_kv_cache(
            new_kv_c, new_k_pe, cache_kv, kv_lens, page_indices, cu_q_lens, n, lkv_c
        )  # mla_ref:150-158
    page_size = cache_kv.shape[1]
    max_num_seqs = kv_lens.shape[0]
    assert page_indices.shape[0] % max_num_seqs == 0
    pages_per_seq = page_indices.shape[0] // max_num_seqs

    q = torch.cat([ql_nope, q_pe], dim=-1)  # mla_ref:173 (zero pad dims dropped: no contribution)
    outputs = []
    for i in range(n):
        q_start, q_end = _as_int(cu_q_lens[i]), _as_int(cu_q_lens[i + 1])
        q_len = q_end - q_start
        kv_len = _as_int(kv_lens[i])
        q_i = q[q_start:q_end]
        start = i * pages_per_seq  # mla_ref:197
        idx = page_indices[start : start + cdiv(kv_len, page_size)].to(torch.int64)
        flat = cache_kv[idx].reshape(-1, width)[:kv_len]  # mla_ref:203-214
        k_i = torch.cat([flat[:, :lkv], flat[:, lkv_c : lkv_c + rope]], dim=-1)
        v_i = flat[:, :lkv]
        attn = torch.einsum("qnh,kh->nqk", q_i.to(torch.float32), k_i.to(torch.float32))  # :221
        attn = attn * sm_scale
        if k_scale is not None:
            attn = attn * k_scale
        if q_scale is not None:
            attn = attn * q_scale
        q_span = kv_len - q_len + torch.arange(q_len)[:, None]
        kv_span = torch.arange(kv_len)[None, :]
        mask = q_span < kv_span  # :231
        if sliding_window is not None:
            mask = mask | (q_span - sliding_window >= kv_span)  # :233
        if soft_cap is not None:
            attn = soft_cap * torch.tanh(attn / soft_cap)  # :235
        attn = torch.where(mask[None], torch.tensor(mask_value, dtype=torch.float32), attn)  # :236
        p = torch.softmax(attn, dim=-1).to(v_i.dtype)  # :237  P ROUNDED to the cache dtype
        out_i = torch.einsum("nqk,kl->qnl", p.to(torch.float32), v_i.to(torch.float32)).to(q_i.dtype)  # :240
        if v_scale is not None:
            out_i = out_i * v_scale  # :241-242
        outputs.append(out_i)
    out = torch.cat(outputs, dim=0) if outputs else q[:0, :, :lkv].clone()
    return out, cache_kv
