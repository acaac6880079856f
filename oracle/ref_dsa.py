"""CPU restatement of the reference's sparse absorbed-MLA oracle and of the page bookkeeping of
its dense-kernel wrappers.

TEST INFRASTRUCTURE ONLY: imported by tests/.  The product path never touches this module.

  dsa_ref = python/sgl_jax/srt/kernels/dsa/ref.py
  dsa_sp  = python/sgl_jax/srt/kernels/dsa/sparse_mla.py

Plain loops, one query token at a time (the reference vectorises over all tokens and masks).
What pins each function independently of this file's formulae is listed in
tests/test_oracle_dsa.py; the reference ships no stored vectors for this path.
"""

from __future__ import annotations

import numpy as np
import torch


def sparse_mla_ref(q, cache_kv, kv_lens, topk_indices, page_indices, cu_q_lens, cu_kv_lens, distribution, *,
                   sm_scale: float, pages_per_seq: int, v_dim: int) -> torch.Tensor:
    """dsa_ref:272-337.  q [T, H, Dqk] = [nope | rope]; cache_kv [pages, P, Dkv]; topk_indices
    i32[T, k] sequence-relative positions, -1 (or >= kv_len) = ignore; page_indices flat, sequence
    i's pages start at cu_kv_lens[i] // P.  f32 logits and softmax over the selected positions,
    values = the first v_dim dims of the selected rows; output in q's dtype."""
    T, H, _ = q.shape
    P = cache_kv.shape[1]
    n = int(distribution[-1])
    out = torch.zeros((T, H, v_dim), dtype=q.dtype)
    for s in range(n):
        q0, q1 = int(cu_q_lens[s]), int(cu_q_lens[s + 1])
        kv_len = int(kv_lens[s])
        start = int(cu_kv_lens[s]) // P
        pages = page_indices[start : start + pages_per_seq].to(torch.int64)
        flat = cache_kv[pages].reshape(-1, cache_kv.shape[-1])  # dsa_ref:316-319
        for t in range(q0, q1):
            idx = topk_indices[t].to(torch.int64)
            sel = idx[(idx >= 0) & (idx < kv_len)]  # dsa_ref:325-326
            if sel.numel() == 0:
                continue  # softmax over nothing, then zeroed (dsa_ref:331-332)
            rows = flat[sel].to(torch.float32)
            logits = torch.einsum("hd,kd->hk", q[t].to(torch.float32), rows) * sm_scale
            p = torch.softmax(logits, dim=-1)
            out[t] = (p @ rows[:, :v_dim]).to(q.dtype)
    return out


def topk_pages_ref(topk_indices, page_size: int, pages_per_seq: int, k_pages_max: int) -> np.ndarray:
    """dsa_sp:35-60: the distinct sequence-local pages of each row, ascending, -1 padded."""
    idx = np.asarray(topk_indices)
    out = np.full((idx.shape[0], k_pages_max), -1, dtype=np.int32)
    for t, row in enumerate(idx):
        pages = sorted({int(i) // page_size for i in row if i >= 0 and int(i) // page_size < pages_per_seq})
        pages = pages[:k_pages_max]
        out[t, : len(pages)] = pages
    return out


def page_level_metadata_ref(kv_lens, topk_indices, page_indices, cu_q_lens, cu_kv_lens, *, page_size: int,
                            pages_per_seq: int, k_pages_max: int, sentinel_page: int):
    """dsa_sp:107-175 for a decode batch: per query token the physical page list
    [touched pages ascending (without the new token's page) ..., new token's page, sentinel ...]
    and the length n_touched * P + offset of the new token + 1.  Returns
    (kv_len i32[T], pages i32[T, k_pages_max])."""
    idx = np.asarray(topk_indices)
    kv_lens = np.asarray(kv_lens)
    cu_q = np.asarray(cu_q_lens)
    cu_kv = np.asarray(cu_kv_lens)
    table = np.asarray(page_indices).reshape(-1)
    T = idx.shape[0]
    S = kv_lens.shape[0]
    sp_len = np.zeros(T, dtype=np.int32)
    sp_pages = np.full((T, k_pages_max), sentinel_page, dtype=np.int32)
    for t in range(T):
        s = min(int(np.searchsorted(cu_q[1:], t, side="right")), S - 1)
        kv_len = int(kv_lens[s])
        new_abs = max(kv_len - 1, 0)
        new_page, new_off = new_abs // page_size, new_abs % page_size
        touched = sorted({int(i) // page_size for i in idx[t] if i >= 0} - {new_page})
        touched = [p for p in touched if p < pages_per_seq][: k_pages_max - 1]
        sp_len[t] = len(touched) * page_size + new_off + 1
        if kv_len > 0:
            start = int(cu_kv[s]) // page_size
            local = touched + [new_page]
            sp_pages[t, : len(local)] = table[[start + p for p in local]]
    return sp_len, sp_pages
