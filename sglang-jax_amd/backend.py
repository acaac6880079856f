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


def pad_page_indices(page_indices, max_num_seqs: int, fixed_capacity: int | None = None) -> np.ndarray:
    """Length bucketing of the flat page table on the speculative-decoding paths
    (flashattention_backend.py:42-69): zero-padded either to ``fixed_capacity`` entries (an error if
    it holds more already) or to ``max_num_seqs`` times the pages per sequence rounded up to a power
    of two, 16 at least -- so that the table's shape, which is part of a compiled call's signature,
    takes few distinct values.  The padding entries are valid page ids (0) that no kernel reads."""
    page_indices = np.asarray(page_indices, dtype=np.int32)
    if fixed_capacity is not None:
        target = int(fixed_capacity)
        if target < len(page_indices):
            raise ValueError(f"page_indices exceed fixed capacity: required={len(page_indices)}, capacity={target}")
    elif max_num_seqs > 0 and len(page_indices) > 0:
        per_seq = cdiv(len(page_indices), max_num_seqs)
        target = max_num_seqs * max(16, 1 << max(0, per_seq - 1).bit_length())
    else:
        return page_indices
    out = np.zeros(target, dtype=np.int32)
    out[: len(page_indices)] = page_indices
    return out


def build_verify_metadata(
    *,
    seq_lens,
    draft_token_num: int,
    logits_indices_selector,
    custom_mask=None,
    page_size: int,
    dp_size: int = 1,
    per_dp_bs_size: int | None = None,
) -> dict:
    """Host arithmetic of the target-verify branch of ``get_eagle_forward_metadata``
    (flashattention_backend.py:298-376, 430-437).

    ``seq_lens`` are the verified lengths per batch slot (0 for padding slots); the slots named by
    ``logits_indices_selector`` each get ``draft_token_num`` query tokens, which also count towards
    their kv length.  ``custom_mask`` is the flat tree mask as the draft worker builds it: slot
    after slot, ``draft_token_num`` rows of ``kv_len`` entries (a padding slot holds
    ``draft_token_num * (draft_token_num - 1)`` entries that are dropped).  It is repacked so that
    every row is as wide as the slot's page-aligned kv length -- the width the kernel reads with
    ``mask_aligned_to_cu_kv`` -- and each DP rank's part is padded to one common length, at least
    the original length per rank rounded up to a multiple of 8.
    """
    seq_lens = np.asarray(seq_lens, dtype=np.int32)
    if per_dp_bs_size is None:
        per_dp_bs_size = len(seq_lens) // max(dp_size, 1)
    if per_dp_bs_size * dp_size != len(seq_lens):
        raise ValueError(f"expected per_dp_bs_size * dp_size == len(seq_lens), got {per_dp_bs_size} * {dp_size} != {len(seq_lens)}")
    q = int(draft_token_num)
    extend = np.zeros(len(seq_lens), dtype=np.int32)
    extend[np.asarray(logits_indices_selector, dtype=np.int64)] = q
    kv = seq_lens + extend
    aligned = ((kv + page_size - 1) // page_size) * page_size

    def sectioned_cumsum(lens):
        cu = np.zeros((dp_size, per_dp_bs_size + 1), dtype=np.int32)
        cu[:, 1:] = np.cumsum(np.asarray(lens, dtype=np.int32).reshape(dp_size, per_dp_bs_size), axis=1)
        return cu.ravel()

    packed = None
    if custom_mask is not None:
        cm = np.asarray(custom_mask)
        if cm.dtype == np.bool_:
            raise ValueError("custom_mask bool dtype is not supported; use int32 instead.")
        per_rank_target = ((len(cm) // dp_size + 7) // 8) * 8 or 8
        held = np.where(kv > 0, kv, q - 1).astype(np.int64)  # entries per row as the draft worker wrote them
        start = np.concatenate([[0], np.cumsum(q * held)])
        ranks = []
        for r in range(dp_size):
            rows = []
            for s in range(r * per_dp_bs_size, (r + 1) * per_dp_bs_size):
                width = int(aligned[s])
                if kv[s] > 0:
                    m = cm[start[s] : start[s] + q * int(kv[s])].reshape(q, int(kv[s]))
                    rows.append(np.pad(m, ((0, 0), (0, width - int(kv[s])))).reshape(-1))
                elif width > 0:
                    rows.append(np.zeros(q * width, dtype=cm.dtype))
            ranks.append(np.concatenate(rows) if rows else np.zeros(0, dtype=cm.dtype))
        common = max(max(len(x) for x in ranks), per_rank_target)
        packed = np.concatenate([np.pad(x, (0, common - len(x))) for x in ranks]).astype(np.int32)

    n = np.sum(seq_lens.reshape(dp_size, per_dp_bs_size) > 0, axis=1, dtype=np.int32)
    return {
        "extend_seq_lens": extend,
        "seq_lens": kv,
        "cu_q_lens": sectioned_cumsum(extend),
        "cu_kv_lens": sectioned_cumsum(aligned),
        "distribution": np.column_stack([np.zeros_like(n), n, n]).ravel().astype(np.int32),
        "custom_mask": packed,
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
