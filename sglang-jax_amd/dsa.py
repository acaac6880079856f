"""Sparse absorbed-MLA (DeepSeek sparse attention) on the dense MLA kernels: the reference's
``python/sgl_jax/srt/kernels/dsa/sparse_mla.py`` re-indexes the page table (or gathers rows) and
hands the result to its dense kernel; the same is done here in front of
``mla_ragged_paged_attention`` (mla.py, HIP kernels behind ``rpa_mla_*``).  All index work stays
on the device (no host reads), so a call can sit inside a captured step.

* ``compute_topk_pages``     sparse_mla.py:35-60   unique pages a top-k list touches
* ``sparse_mla_page_level``  sparse_mla.py:63-203  decode: dense kernel over the touched pages
* ``sparse_mla_via_dense``   sparse_mla.py:206-297 any T: gather the k rows, dense kernel over them
"""

from __future__ import annotations

import torch

from .mla import mla_ragged_paged_attention
from .ragged_paged_attention import _i32, _require_gpu


def _first_hits(mask: torch.Tensor, count: int) -> torch.Tensor:
    """Indices of the first ``count`` True entries of each row, ascending (what jax.lax.top_k
    returns for a 0/1 row: equal values keep index order); rows with fewer hits continue with
    the lowest unset indices, as top_k does."""
    n = mask.shape[1]
    pos = torch.arange(n, device=mask.device, dtype=torch.int64)
    key = torch.where(mask, pos, pos + n)
    return torch.sort(key, dim=1).values[:, :count] % n


def compute_topk_pages(topk_indices, *, page_size: int, pages_per_seq: int, k_pages_max: int) -> torch.Tensor:
    """i32[T, k_pages_max]: the sequence-local pages touched by each row of ``topk_indices``
    (i32[T, k], -1 = unused), ascending, padded with -1 (sparse_mla.py:35-60)."""
    idx = topk_indices.to(torch.int64)
    T = idx.shape[0]
    valid = idx >= 0
    page_local = torch.where(valid, idx // page_size, torch.full_like(idx, pages_per_seq))
    mask = torch.zeros((T, pages_per_seq + 1), dtype=torch.bool, device=idx.device)
    mask.scatter_(1, page_local, torch.ones_like(page_local, dtype=torch.bool))
    mask = mask[:, :pages_per_seq]
    n_hit = mask.sum(dim=1)
    k_eff = min(k_pages_max, pages_per_seq)
    hit = _first_hits(mask, k_eff)
    if k_eff < k_pages_max:
        hit = torch.nn.functional.pad(hit, (0, k_pages_max - k_eff))
    col = torch.arange(k_pages_max, device=idx.device)[None, :]
    return torch.where(col < n_hit[:, None], hit, torch.full_like(hit, -1)).to(torch.int32)


def sparse_mla_page_level(ql_nope, q_pe, new_kv_c, new_k_pe, cache_kv, kv_lens, topk_indices, page_indices,
                          cu_q_lens, cu_kv_lens, distribution, topk_pages=None, *, sm_scale: float, page_size: int,
                          pages_per_seq: int, kv_lora_rank: int, k_pages_max: int = 64, **_tile_hints):
    """Decode (one query token per sequence): attends the whole pages that ``topk_indices``
    touches plus the page of the new token, which goes last so that the kernel's cache write
    lands in the true slot (sparse_mla.py:63-203).  Returns ``(o_latent, cache_kv)``; the last
    page of the cache is the padding target, as in the reference."""
    _require_gpu(ql_nope, "ql_nope")
    dev = ql_nope.device
    T = ql_nope.shape[0]
    kv_lens_d, page_d = _i32(kv_lens, dev).to(torch.int64), _i32(page_indices, dev).reshape(-1).to(torch.int64)
    cu_q_d, cu_kv_d = _i32(cu_q_lens, dev).to(torch.int64), _i32(cu_kv_lens, dev).to(torch.int64)
    S = kv_lens_d.shape[0]
    tok = torch.arange(T, device=dev)
    seq_id = torch.clamp(torch.searchsorted(cu_q_d[1:].contiguous(), tok, right=True), 0, S - 1)
    tok_valid = kv_lens_d[seq_id] > 0
    seq_page_start = cu_kv_d[seq_id] // page_size
    new_abs = torch.clamp(kv_lens_d[seq_id] - 1, min=0)
    new_page_local = new_abs // page_size
    new_off = new_abs % page_size
    kp = k_pages_max
    if topk_pages is not None:
        raw = topk_pages.to(dev).to(torch.int64)[:, : kp - 1]
        ok = (raw >= 0) & (raw != new_page_local[:, None])
        n_hit = torch.clamp(ok.sum(dim=1), max=kp - 1)
        big = torch.iinfo(torch.int32).max
        hit = torch.sort(torch.where(ok, raw, torch.full_like(raw, big)), dim=1).values
        if hit.shape[1] < kp - 1:
            hit = torch.nn.functional.pad(hit, (0, kp - 1 - hit.shape[1]))
    else:
        idx = topk_indices.to(dev).to(torch.int64)
        valid = idx >= 0
        page_local = torch.where(valid, idx // page_size, torch.full_like(idx, pages_per_seq))
        mask = torch.zeros((T, pages_per_seq + 1), dtype=torch.bool, device=dev)
        mask.scatter_(1, page_local, torch.ones_like(page_local, dtype=torch.bool))
        mask = mask[:, :pages_per_seq]
        mask &= torch.arange(pages_per_seq, device=dev)[None, :] != new_page_local[:, None]
        n_hit = torch.clamp(mask.sum(dim=1), max=kp - 1)
        hit = _first_hits(mask, min(kp - 1, pages_per_seq))
        if hit.shape[1] < kp - 1:
            hit = torch.nn.functional.pad(hit, (0, kp - 1 - hit.shape[1]))
    n_used = n_hit + 1
    col = torch.arange(kp, device=dev)[None, :]
    hit_p = torch.nn.functional.pad(hit, (0, 1))
    sp_local = torch.where(col < n_hit[:, None], hit_p,
                           torch.where(col == n_hit[:, None], new_page_local[:, None], torch.zeros_like(hit_p)))
    gather_at = torch.clamp(seq_page_start[:, None] + sp_local, 0, page_d.numel() - 1)
    sentinel = cache_kv.shape[0] - 1
    sp_phys = torch.where((col < n_used[:, None]) & tok_valid[:, None], page_d[gather_at],
                          torch.full_like(gather_at, sentinel))
    sp_kv_len = (n_hit * page_size + new_off + 1).to(torch.int32)
    sp_cu_q = torch.arange(T + 1, dtype=torch.int32, device=dev)
    sp_cu_kv = sp_cu_q * (kp * page_size)
    o, cache_out = mla_ragged_paged_attention(
        ql_nope, q_pe, new_kv_c, new_k_pe, cache_kv, sp_kv_len, sp_phys.reshape(-1).to(torch.int32), sp_cu_q,
        sp_cu_kv, (T, T, T), sm_scale=sm_scale, sliding_window=None, soft_cap=None,
        max_kv_len=kp * page_size, sum_kv_len=0)
    return o[..., :kv_lora_rank], cache_out


def sparse_mla_via_dense(ql_nope, q_pe, new_kv_c, new_k_pe, cache_kv, kv_lens, topk_indices, page_indices,
                         cu_q_lens, cu_kv_lens, distribution, *, sm_scale: float, page_size: int,
                         pages_per_seq: int, kv_lora_rank: int, **_tile_hints) -> torch.Tensor:
    """Token-level sparse attention for any T: the k selected rows of every query token are
    gathered into a temporary paged buffer (k rows = one short "sequence" per token) and the
    dense kernel runs over it with ``kv_len`` = number of valid entries; the new token's row
    replaces the last valid entry, as the dense kernel's cache write does in the reference
    (sparse_mla.py:206-297).  Valid entries must come first in each row."""
    _require_gpu(ql_nope, "ql_nope")
    dev = ql_nope.device
    T = ql_nope.shape[0]
    cache3 = cache_kv.view(cache_kv.shape[0], -1, cache_kv.shape[-1]) if cache_kv.dim() == 4 else cache_kv
    width = cache3.shape[-1]
    idx = topk_indices.to(dev).to(torch.int64)
    k = idx.shape[1]
    kv_lens_d, page_d = _i32(kv_lens, dev).to(torch.int64), _i32(page_indices, dev).reshape(-1).to(torch.int64)
    cu_q_d, cu_kv_d = _i32(cu_q_lens, dev).to(torch.int64), _i32(cu_kv_lens, dev).to(torch.int64)
    S = kv_lens_d.shape[0]
    seq_id = torch.clamp(torch.searchsorted(cu_q_d[1:].contiguous(), torch.arange(T, device=dev), right=True), 0, S - 1)
    seq_page_start = cu_kv_d[seq_id] // page_size
    valid = idx >= 0
    safe = torch.where(valid, idx, torch.zeros_like(idx))
    phys = page_d[torch.clamp(seq_page_start[:, None] + safe // page_size, 0, page_d.numel() - 1)]
    slot = phys * page_size + safe % page_size
    rows = cache3.reshape(-1, width).index_select(0, slot.reshape(-1)).reshape(T, k, width)
    rows = torch.where(valid[..., None], rows, torch.zeros_like(rows))
    n_tmp = -(-k // page_size)
    tmp = torch.zeros((T * n_tmp + 1, page_size, width), dtype=cache3.dtype, device=dev)
    tmp[: T * n_tmp].view(T, n_tmp * page_size, width)[:, :k] = rows
    tmp_kv_lens = valid.sum(dim=1).to(torch.int32)
    tmp_pages = torch.arange(T * n_tmp, dtype=torch.int32, device=dev)
    tmp_cu_q = torch.arange(T + 1, dtype=torch.int32, device=dev)
    tmp_cu_kv = tmp_cu_q * (n_tmp * page_size)
    o, _ = mla_ragged_paged_attention(
        ql_nope, q_pe, new_kv_c, new_k_pe, tmp, tmp_kv_lens, tmp_pages, tmp_cu_q, tmp_cu_kv, (T, T, T),
        sm_scale=sm_scale, sliding_window=None, soft_cap=None, max_kv_len=n_tmp * page_size, sum_kv_len=0)
    return o[..., :kv_lora_rank]
