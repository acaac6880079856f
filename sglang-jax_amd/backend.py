"""Attention backend on the HIP kernels: the host metadata builder and the per-layer call
of the reference's ``FlashAttention`` backend
(python/sgl_jax/srt/layers/attention/flashattention_backend.py:123-237 metadata,
:603-760 call, :770-777 request bound) for one GPU.

The batch, layer and KV pool are duck-typed exactly as the reference reads them:

* batch: ``forward_mode`` (``ForwardMode.EXTEND`` / ``DECODE``), ``seq_lens``,
  ``cache_loc``, ``extend_seq_lens``, ``dp_size``, ``per_dp_bs_size`` (host numpy arrays,
  schedule_batch.py ModelWorkerBatch);
* layer: ``layer_id``, ``scaling``, ``head_dim``, ``sliding_window_size``, ``logit_cap``,
  ``xai_temperature_len``, ``softmax_dtype``, ``attn_type`` (layers/radix_attention.py:24-60);
* pool: ``get_fused_kv_buffer(layer_id)`` returning ``[pages, P, 2*Hkv, D]``
  (mem_cache/memory_pool.py:566-611).

The metadata arithmetic is pure numpy (no device needed); ``get_forward_metadata`` then
uploads it once per forward pass and every layer call reuses it.  Host-side bounds
(``max_kv_len``, ``max_q_len``, the decode work sum) travel with the metadata because the
library sizes its launch grids from them without reading device memory.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, field

import numpy as np
import torch

from .mla import mla_ragged_paged_attention
from .ragged_paged_attention import ragged_paged_attention


class ForwardMode(enum.Enum):
    """The two modes the metadata builder accepts (forward_batch_info.py ForwardMode)."""

    EXTEND = "extend"
    DECODE = "decode"


def _mode_name(mode) -> str:
    name = getattr(mode, "name", mode)
    return str(name).upper()


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def build_forward_metadata(
    *,
    forward_mode,
    seq_lens,
    cache_loc,
    extend_seq_lens=None,
    page_size: int,
    dp_size: int = 1,
    per_dp_bs_size: int | None = None,
    swa_index_mapping=None,
    extend_distribution_is_mixed: bool = False,
) -> dict:
    """Host arithmetic of ``FlashAttention.get_forward_metadata``
    (flashattention_backend.py:146-237), as numpy int32 arrays:

    ``page_indices = cache_loc[::P] // P`` per DP section; ``cu_q_lens`` = arange (decode) or
    cumulative extend lengths, each section starting at 0; ``cu_kv_lens`` = cumulative
    page-aligned sequence lengths; ``distribution`` = (n, n, n) for decode and (0, n, n) for
    extend with n = number of sequences of non-zero length; the sliding-window pool's page
    ids through ``swa_index_mapping`` when one is given.  The MLA backend builds the same
    arrays but declares an extend batch as (0, 0, n) (mla_backend.py:192-199):
    ``extend_distribution_is_mixed``.
    """
    seq_lens = np.asarray(seq_lens, dtype=np.int32)
    cache_loc = np.asarray(cache_loc, dtype=np.int32)
    if per_dp_bs_size is None:
        per_dp_bs_size = len(seq_lens) // max(dp_size, 1)
    if dp_size <= 0:
        raise ValueError(f"Invalid dp_size: {dp_size}")
    if per_dp_bs_size <= 0:
        raise ValueError(f"Invalid per_dp_bs_size: {per_dp_bs_size}")
    if per_dp_bs_size * dp_size != len(seq_lens):
        raise ValueError(
            "Inconsistent DP batch metadata: expected per_dp_bs_size * dp_size == len(seq_lens), "
            f"got {per_dp_bs_size} * {dp_size} != {len(seq_lens)}"
        )
    if len(cache_loc) % dp_size != 0:
        raise ValueError(
            "Inconsistent cache_loc layout for DP sharding: "
            f"len(cache_loc)={len(cache_loc)} is not divisible by dp_size={dp_size}"
        )
    mode = _mode_name(forward_mode)
    if mode not in ("EXTEND", "DECODE"):
        raise ValueError(f"Invalid forward mode: {forward_mode}")

    strided = cache_loc.reshape(dp_size, -1)[:, ::page_size]
    page_indices = (strided // page_size).astype(np.int32).ravel()

    swa_page_indices = None
    if swa_index_mapping is not None:
        swa = np.empty(strided.shape, dtype=np.int32)
        for r in range(dp_size):
            mapping = swa_index_mapping[r] if isinstance(swa_index_mapping, list) else swa_index_mapping
            swa[r] = np.asarray(mapping)[strided[r]]
        swa_page_indices = (swa // page_size).astype(np.int32).ravel()

    def sectioned_cumsum(lens):
        cu = np.zeros((dp_size, per_dp_bs_size + 1), dtype=np.int32)
        cu[:, 1:] = np.cumsum(np.asarray(lens, dtype=np.int32).reshape(dp_size, per_dp_bs_size), axis=1)
        return cu.ravel()

    if mode == "EXTEND":
        if extend_seq_lens is None:
            raise ValueError("extend_seq_lens is required in EXTEND mode")
        cu_q_lens = sectioned_cumsum(extend_seq_lens)
    else:
        cu_q_lens = np.tile(np.arange(per_dp_bs_size + 1, dtype=np.int32), dp_size)

    aligned = ((seq_lens + page_size - 1) // page_size) * page_size
    cu_kv_lens = sectioned_cumsum(aligned)

    n = np.sum(seq_lens.reshape(dp_size, per_dp_bs_size) > 0, axis=1, dtype=np.int32)
    if mode == "DECODE":
        distribution = np.repeat(n, 3).astype(np.int32)
    else:
        mid = np.zeros_like(n) if extend_distribution_is_mixed else n
        distribution = np.column_stack([np.zeros_like(n), mid, n]).ravel().astype(np.int32)

    return {
        "cu_q_lens": cu_q_lens,
        "cu_kv_lens": cu_kv_lens,
        "page_indices": page_indices,
        "swa_page_indices": swa_page_indices,
        "seq_lens": seq_lens,
        "distribution": distribution,
    }


@dataclass
class FlashAttentionMetadata:
    """Built once per forward pass, reused by every layer (flashattention_backend.py:72-120)."""

    cu_q_lens: torch.Tensor | None = None
    cu_kv_lens: torch.Tensor | None = None
    page_indices: torch.Tensor | None = None
    swa_page_indices: torch.Tensor | None = None
    seq_lens: torch.Tensor | None = None
    distribution: torch.Tensor | None = None
    custom_mask: torch.Tensor | None = None
    # host-side companions (sizes of launch grids; never read back from the device)
    host_distribution: np.ndarray | None = None
    max_kv_len: int = 0
    max_q_len: int = 0
    sum_visible: int = 0
    host_seq_lens: np.ndarray | None = field(default=None, repr=False)


class FlashAttention:
    """One-GPU counterpart of the reference's ``FlashAttention`` backend."""

    def __init__(self, num_attn_heads, num_kv_heads, head_dim, page_size: int = 1, device=None):
        self.num_heads = num_attn_heads
        self.num_kv_heads = num_kv_heads if num_kv_heads is not None else num_attn_heads
        self.head_dim = head_dim
        self.page_size = page_size
        self.device = torch.device(device) if device is not None else torch.device("cuda:0")
        self.forward_metadata = FlashAttentionMetadata()
        self.swa_index_mapping = None  # set by the owner of a sliding-window pool

    # ------------------------------------------------------------------ metadata
    def get_forward_metadata(self, batch) -> FlashAttentionMetadata:
        if getattr(batch, "dp_size", 1) != 1:
            raise NotImplementedError("one GPU: data-parallel sections (dp_size > 1) are not built")
        host = build_forward_metadata(
            forward_mode=batch.forward_mode,
            seq_lens=batch.seq_lens,
            cache_loc=batch.cache_loc,
            extend_seq_lens=getattr(batch, "extend_seq_lens", None),
            page_size=self.page_size,
            dp_size=1,
            per_dp_bs_size=getattr(batch, "per_dp_bs_size", None) or len(batch.seq_lens),
            swa_index_mapping=self.swa_index_mapping,
        )
        md = FlashAttentionMetadata()

        def up(x):
            return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(self.device, non_blocking=True)

        md.cu_q_lens = up(host["cu_q_lens"])
        md.cu_kv_lens = up(host["cu_kv_lens"])
        md.page_indices = up(host["page_indices"])
        md.swa_page_indices = up(host["swa_page_indices"])
        md.seq_lens = up(host["seq_lens"])
        md.distribution = up(host["distribution"])
        md.host_distribution = host["distribution"]
        md.host_seq_lens = host["seq_lens"]
        md.max_kv_len = int(host["seq_lens"].max()) if len(host["seq_lens"]) else 0
        q_lens = np.diff(host["cu_q_lens"])
        md.max_q_len = int(q_lens.max()) if len(q_lens) else 0
        return md

    # ------------------------------------------------------------------ layer call
    def __call__(self, q, k, v, layer, forward_batch, token_to_kv_pool, causal: int = 1, attention_sink=None):
        """q, k, v: ``[total_tokens, heads * head_dim]`` or ``[total_tokens, heads, head_dim]``.
        Returns ``(attn_output [total_tokens, num_heads * head_dim], updated fused cache)``."""
        md = self.forward_metadata
        if md.page_indices is None:
            raise ValueError("forward_metadata is not set: call get_forward_metadata(batch) first")
        head_dim = getattr(layer, "head_dim", self.head_dim)
        kv_cache_fused = token_to_kv_pool.get_fused_kv_buffer(layer.layer_id)
        scaling = getattr(layer, "scaling", None)
        scale = float(scaling) if scaling is not None else 1.0 / float(np.sqrt(head_dim))
        attn_type = getattr(layer, "attn_type", None)
        if getattr(attn_type, "value", attn_type) == "encoder_only":
            causal = 0
        if md.custom_mask is not None:
            causal = 0
        window = getattr(layer, "sliding_window_size", None) or None
        page_indices = md.page_indices
        if window is not None and md.swa_page_indices is not None:
            page_indices = md.swa_page_indices
        elif hasattr(token_to_kv_pool, "remap_cache_loc") and self.page_size == 1:
            page_indices = token_to_kv_pool.remap_cache_loc(page_indices, layer.layer_id)
        xai = getattr(layer, "xai_temperature_len", -1)
        T = q.shape[0]
        out, cache = ragged_paged_attention(
            q.reshape(T, -1, head_dim),
            k.reshape(T, -1, head_dim),
            v.reshape(T, -1, head_dim),
            kv_cache_fused,
            md.seq_lens,
            page_indices,
            md.cu_q_lens,
            md.cu_kv_lens,
            md.host_distribution,
            md.custom_mask,
            attention_sink,
            causal=causal,
            sm_scale=scale,
            sliding_window=window,
            soft_cap=getattr(layer, "logit_cap", None) or None,
            xai_temperature_len=xai if xai is not None and xai > 0 else None,
            softmax_dtype=getattr(layer, "softmax_dtype", None),
            max_kv_len=md.max_kv_len,
            max_q_len=md.max_q_len,
            host_kv_lens=md.host_seq_lens,
        )
        return out.reshape(T, -1), cache

    @staticmethod
    def get_max_running_reqests(max_context_len: int, page_size: int) -> int:
        num_page_per_req = cdiv(max_context_len, page_size)
        res = 1024 * 1024 // 2 // num_page_per_req // 4
        assert res > 0, (
            f"max running requests: {res} must larger than 0, please increase page size or decrease max context length"
        )
        return res


class MLAAttentionBackend:
    """One-GPU counterpart of the reference's absorbed-MLA backend
    (python/sgl_jax/srt/layers/attention/mla_backend.py:83-389): same metadata as the MHA
    backend except that an extend batch is declared (0, 0, n), and a layer call that takes
    the absorbed latent query, the new latent row and the two rope parts."""

    def __init__(self, num_attn_heads: int, kv_lora_rank: int, qk_nope_head_dim: int, qk_rope_head_dim: int,
                 v_head_dim: int, page_size: int = 1, device=None):
        assert page_size > 1, "MLA attention backend does not support page_size=1."
        self.num_heads = num_attn_heads
        self.kv_lora_rank = kv_lora_rank
        self.qk_nope_head_dim = qk_nope_head_dim
        self.qk_rope_head_dim = qk_rope_head_dim
        self.v_head_dim = v_head_dim
        self.page_size = page_size
        self.device = torch.device(device) if device is not None else torch.device("cuda:0")
        self.forward_metadata = FlashAttentionMetadata()

    def get_forward_metadata(self, batch) -> FlashAttentionMetadata:
        if getattr(batch, "dp_size", 1) != 1:
            raise NotImplementedError("one GPU: data-parallel sections (dp_size > 1) are not built")
        host = build_forward_metadata(
            forward_mode=batch.forward_mode,
            seq_lens=batch.seq_lens,
            cache_loc=batch.cache_loc,
            extend_seq_lens=getattr(batch, "extend_seq_lens", None),
            page_size=self.page_size,
            dp_size=1,
            per_dp_bs_size=getattr(batch, "per_dp_bs_size", None) or len(batch.seq_lens),
            extend_distribution_is_mixed=True,
        )
        md = FlashAttentionMetadata()
        for name in ("cu_q_lens", "cu_kv_lens", "page_indices", "seq_lens", "distribution"):
            setattr(md, name, torch.from_numpy(np.ascontiguousarray(host[name])).to(self.device, non_blocking=True))
        md.host_distribution = host["distribution"]
        md.host_seq_lens = host["seq_lens"]
        md.max_kv_len = int(host["seq_lens"].max()) if len(host["seq_lens"]) else 0
        q_lens = np.diff(host["cu_q_lens"])
        md.max_q_len = int(q_lens.max()) if len(q_lens) else 0
        # work of one row per query token: token j of a chunk sees kv_len - q_len + j + 1 tokens
        n = int(host["distribution"][2])
        kv, ql = host["seq_lens"][:n].astype(np.int64), q_lens[:n].astype(np.int64)
        md.sum_visible = int((ql * kv - ql * (ql - 1) // 2).sum())
        return md

    def __call__(self, q, k, v, layer, forward_batch, token_to_kv_pool, **kwargs):
        """q: ``[T, n_h, kv_lora_rank]`` (absorbed latent query), k: ``[T, 1, kv_lora_rank]`` or
        ``[T, kv_lora_rank]`` (new latent row; v is the same tensor), ``q_rope`` / ``k_rope``
        keyword arguments: the rope parts.  Returns ``(o_latent [T, n_h, kv_lora_rank], cache)``."""
        del v
        q_rope, k_rope = kwargs.get("q_rope"), kwargs.get("k_rope")
        if q_rope is None or k_rope is None:
            raise ValueError(
                "MLAAttentionBackend requires q_rope/k_rope kwargs (q_pe/k_pe) "
                "alongside the non-rope q/k tensors."
            )
        md = self.forward_metadata
        if md.page_indices is None:
            raise ValueError("forward_metadata is not set: call get_forward_metadata(batch) first")
        new_kv_c = k if k.dim() == 2 else k.squeeze(1)
        new_k_pe = k_rope if k_rope.dim() == 2 else k_rope.squeeze(1)
        cache = token_to_kv_pool.get_fused_kv_buffer(layer.layer_id)
        scaling = getattr(layer, "scaling", None)
        sm_scale = float(scaling) if scaling is not None else 1.0 / float(
            np.sqrt(self.qk_nope_head_dim + self.qk_rope_head_dim))
        return mla_ragged_paged_attention(
            q, q_rope, new_kv_c, new_k_pe, cache, md.seq_lens, md.page_indices, md.cu_q_lens, md.cu_kv_lens,
            md.host_distribution,
            sm_scale=sm_scale,
            sliding_window=getattr(layer, "sliding_window_size", None) or None,
            soft_cap=getattr(layer, "logit_cap", None) or None,
            max_kv_len=md.max_kv_len,
            sum_kv_len=getattr(md, "sum_visible", 0),
        )
