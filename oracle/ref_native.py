"""CPU restatement of the reference's native attention (the engine's own CPU path).

TEST INFRASTRUCTURE ONLY: imported by tests/ as a second, independently structured
cross-check of oracle/ref_rpa.py.  The product path never touches this module.

  native = python/sgl_jax/srt/layers/attention/native_backend.py

It is a different algorithm from the ragged paged one: the cache is gathered token by
token through `loc` (no pages), all sequences share ONE dense score matrix
[tokens, heads, sum of kv lengths] with a block-diagonal mask, and there is no soft cap.
Where the two overlap (causal / sliding-window / sink / temperature on extend batches,
plain and sliding-window decode) they must agree; tests/test_oracle_native.py checks that.

Differences the reference itself has between the two paths, kept here as they are:
  * scores stay in the input dtype (native:252, no wider accumulator type requested) and the
    mask is finfo(dtype).min (native:253, 393, 433), not -0.7 * f32 max;
  * the decode temperature uses seq_lengths as the query position (native:271), one more
    than the ragged kernel's kv_len - 1.
"""

from __future__ import annotations

import math

import torch


def _batch_ids(lens: torch.Tensor, total: int) -> tuple[torch.Tensor, torch.Tensor]:
    """native:356-363: owner of every position of a concatenation, and the owners' starts."""
    starts = torch.cumsum(lens, 0) - lens
    marks = torch.zeros(total, dtype=torch.int64)
    marks[starts[starts < total]] = 1  # a zero-length entry shares its start with the next: set, not add
    return torch.cumsum(marks, 0) - 1, starts


def ref_forward_attention(
    q: torch.Tensor,  # [tokens, Hq, D] (or [tokens, Hq * D])
    k_cache: torch.Tensor,  # [cache tokens, Hkv, D]
    v_cache: torch.Tensor,
    seq_lengths: torch.Tensor,  # i64[S] kv length of every sequence
    loc: torch.Tensor,  # i64[sum kv]: cache row of every kv token, sequences concatenated; <= 0 is padding
    extend_prefix_lens: torch.Tensor | None,
    extend_seq_lens: torch.Tensor | None,
    num_heads: int,
    num_kv_heads: int,
    scale: float | None = None,
    is_causal: bool = True,
    mode: str = "decode",  # "decode" | "extend"
    xai_temperature_len: float | None = None,
    attention_sink: torch.Tensor | None = None,
    sliding_window_size: int | None = None,
    softmax_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """native:169-327.  Returns [tokens, Hq * Dv]."""
    seq_lengths = seq_lengths.to(torch.int64)
    # native:214-217: gather the tokens; a non-positive location reads zeros
    valid = loc > 0
    rows = torch.where(valid, loc, torch.zeros_like(loc)).to(torch.int64)
    k = k_cache[rows] * valid[:, None, None].to(k_cache.dtype)
    v = v_cache[rows] * valid[:, None, None].to(v_cache.dtype)
    if q.dim() == 2:  # native:220-224
        q = q.reshape(q.shape[0], num_heads, -1)
    tokens, _, head_dim = q.shape
    if k.shape[-1] != head_dim:  # native:237-241: queries padded up to the cache's head_dim
        q = torch.nn.functional.pad(q, (0, k.shape[-1] - head_dim))
        head_dim = k.shape[-1]
    if num_kv_heads != num_heads:  # native:246-252
        k = k.repeat_interleave(num_heads // num_kv_heads, dim=1)
        v = v.repeat_interleave(num_heads // num_kv_heads, dim=1)
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    dtype = q.dtype
    neg = torch.finfo(dtype).min
    # native:256: one matmul over all kv tokens of the batch, result in the input dtype
    logits = (torch.einsum("qhd,khd->qhk", q.float(), k.float()).to(dtype) * scale).to(dtype)
    logits = torch.where(valid[None, None, :], logits, torch.full_like(logits, neg))  # native:257-261

    total_kv = loc.shape[0]
    if mode == "extend":
        ext = extend_seq_lens.to(torch.int64)
        q_ids, q_starts = _batch_ids(ext, tokens)
        q_pos = extend_prefix_lens.to(torch.int64)[q_ids] + (torch.arange(tokens) - q_starts[q_ids])  # native:268-271
    else:
        q_pos = seq_lengths  # native:273
    if xai_temperature_len is not None and xai_temperature_len > 0:  # native:264-283
        factor = torch.log2(torch.clamp(q_pos.float(), min=1.0)) / math.log2(float(xai_temperature_len))
        regulator = torch.where(q_pos > xai_temperature_len, factor, torch.ones_like(factor))
        logits = (logits * regulator[:, None, None].to(dtype)).to(dtype)

    if mode == "extend":  # native:330-394
        k_ids, k_starts = _batch_ids(seq_lengths, total_kv)
        k_rel = torch.arange(total_kv) - k_starts[k_ids]
        mask = q_ids[:, None] == k_ids[None, :]
        if is_causal:
            mask &= q_pos[:, None] >= k_rel[None, :]
        if sliding_window_size is not None:
            mask &= (q_pos[:, None] - k_rel[None, :]) < sliding_window_size
        mask &= (torch.arange(tokens) < int(ext.sum()))[:, None]
        mask &= (torch.arange(total_kv) < int(seq_lengths.sum()))[None, :]
    else:  # native:397-435: query i is sequence i
        starts = torch.cumsum(seq_lengths, 0) - seq_lengths
        ends = starts + seq_lengths
        pos = torch.arange(total_kv)
        per_seq = (pos[None, :] >= starts[:, None]) & (pos[None, :] < ends[:, None])
        if sliding_window_size is not None:
            per_seq &= pos[None, :] >= (ends[:, None] - sliding_window_size)
        mask = torch.zeros(tokens, total_kv, dtype=torch.bool)
        mask[: seq_lengths.shape[0]] = per_seq
    logits = torch.where(mask[:, None, :], logits, torch.full_like(logits, neg))

    if softmax_dtype is not None:  # native:297-298
        logits = logits.to(softmax_dtype)
    top = logits.max(dim=-1, keepdim=True).values
    e = torch.exp(logits - top)
    den = e.sum(dim=-1, keepdim=True)
    if attention_sink is not None:  # native:305-309: a phantom token in the denominator
        den = den + torch.exp(attention_sink.to(e.dtype)[None, :, None] - top)
    w = e / den
    if softmax_dtype is not None and w.dtype != v.dtype:  # native:314-315
        w = w.to(v.dtype)
    out = torch.einsum("qhk,khd->qhd", w.float(), v.float()).to(w.dtype)  # native:318
    return out.reshape(tokens, num_heads * v.shape[-1])
