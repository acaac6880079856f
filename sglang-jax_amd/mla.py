"""Host-side mirror of the reference's absorbed-MLA ragged paged attention
(``mla_ragged_paged_attention``, python/sgl_jax/srt/kernels/mla/v2/kernel.py:1338-1370)
on the HIP kernels behind ``rpa_mla_kv_write`` / ``rpa_mla_decode`` / ``rpa_mla_attention``
(include/rpa.h): new latent rows are written into the cache, then every query token attends to
the cache up to its own position.

The latent cache may be the compact ``[pages, P, lkv+rope]`` (576-wide rows) or
the reference's 128-aligned ``[pages, P, 512+128]`` (kernel.py:74-86; also its
packed 4-D view ``[pages, P/2, 2, 640]``, which is memory-identical).
"""

from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import _lib
from ._lib import RpaMlaParams
from .ragged_paged_attention import DEFAULT_MASK_VALUE, _host_decode_sum, _host_max, _i32, _require_gpu, _workspace


def mla_ragged_paged_attention(
    ql_nope: torch.Tensor,  # [max_num_tokens, num_q_heads, lkv_dim]
    q_pe: torch.Tensor,  # [max_num_tokens, num_q_heads, r_dim]
    new_kv_c: torch.Tensor | None,  # [max_num_tokens, lkv_dim]  (None: cache already complete)
    new_k_pe: torch.Tensor | None,  # [max_num_tokens, r_dim]
    cache_kv: torch.Tensor,  # [pages, P, width]  or  [pages, P/pack, pack, width]
    kv_lens,  # i32[max_num_seqs]
    page_indices,  # i32[flat ragged]  (or padded, when cu_kv_lens is None)
    cu_q_lens,  # i32[max_num_seqs + 1]
    cu_kv_lens,  # i32[max_num_seqs + 1] or None
    distribution,  # i32[3] host
    *,
    sm_scale: float = 1.0,
    sliding_window: int | None = None,
    soft_cap: float | None = None,
    mask_value: float | None = DEFAULT_MASK_VALUE,
    q_scale: float | None = None,
    k_scale: float | None = None,
    v_scale: float | None = None,
    chunk_prefill_size: int | None = None,
    num_kv_pages_per_block=None,
    num_queries_per_block=None,
    vmem_limit_bytes: int | None = None,
    decode_batch_size: int = 1,
    debug_mode: bool = False,
    max_kv_len: int | None = None,
    num_splits: int = 0,
    sum_kv_len: int | None = None,
):
    """Returns (output [max_num_tokens, num_q_heads, lkv_dim], cache_kv updated in place).

    ``new_kv_c`` / ``new_k_pe`` may be None when the cache already holds all ``kv_len``
    tokens.  A decode batch (``distribution = (n, n, n)``) takes the one-row-per-sequence
    entry point; anything else (prefill chunks, mixed) runs one row per query token."""
    _require_gpu(ql_nope, "ql_nope")
    _require_gpu(cache_kv, "cache_kv")
    if ql_nope.dim() != 3:
        raise ValueError(f"Expected 3D array for ql_nope.shape={tuple(ql_nope.shape)}")
    if q_pe.dim() != 3:
        raise ValueError(f"Expected 3D array for q_pe.shape={tuple(q_pe.shape)}")
    if ql_nope.shape[:2] != q_pe.shape[:2]:
        raise ValueError(f"Expected ql_nope.shape[:2]={tuple(ql_nope.shape[:2])} to be equal to q_pe.shape[:2]={tuple(q_pe.shape[:2])}")
    if sliding_window is not None and sliding_window <= 0:
        raise ValueError(f"sliding_window={sliding_window} must be positive.")
    if soft_cap is not None and soft_cap == 0.0:
        raise ValueError(f"soft_cap={soft_cap} must not be 0.0.")
    if (new_kv_c is None) != (new_k_pe is None):
        raise ValueError("new_kv_c and new_k_pe must be given together")
    for name, val in (("q_scale", q_scale), ("k_scale", k_scale), ("v_scale", v_scale)):
        if val is not None and not val > 0:
            raise ValueError(f"{name}={val} must be positive.")
    # Static-shape mode: a distribution on the GPU is never read back; the kernels take the number of
    # sequences from it and every query token runs as a row of its own (any batch composition).
    static_shapes = isinstance(distribution, torch.Tensor) and distribution.is_cuda
    if static_shapes:
        if distribution.dtype != torch.int32 or tuple(distribution.shape) != (3,):
            raise ValueError(f"Expected int32 distribution of shape (3,), got {distribution.dtype} {tuple(distribution.shape)}")
        i = j = 0
        k = int(kv_lens.shape[0])
        decode_only = False
    else:
        dist = np.asarray(distribution.cpu() if isinstance(distribution, torch.Tensor) else distribution)
        i, j, k = (int(x) for x in dist)
        if not (0 <= i <= j <= k):
            raise ValueError(f"distribution must satisfy 0 <= i <= j <= k, got ({i}, {j}, {k})")
        decode_only = i == j == k
    device = ql_nope.device
    if cache_kv.dim() == 4:
        s = cache_kv.shape
        cache_kv = cache_kv.view(s[0], s[1] * s[2], s[3])
    if not (ql_nope.is_contiguous() and q_pe.is_contiguous() and cache_kv.is_contiguous()):
        raise ValueError("ql_nope, q_pe and cache_kv must be contiguous")
    if not (ql_nope.dtype == q_pe.dtype == torch.bfloat16):
        raise ValueError("Expected bfloat16 ql_nope and q_pe")
    if cache_kv.dtype not in (torch.bfloat16, torch.float8_e4m3fn):
        raise ValueError(f"Expected a bfloat16 or float8_e4m3fn latent cache, got {cache_kv.dtype}")
    T, Hq, lkv = ql_nope.shape
    rope = q_pe.shape[2]
    total_pages, page_size, width = cache_kv.shape
    if width == lkv + rope:
        rope_offset = lkv
    elif width == -(-lkv // 128) * 128 + -(-rope // 128) * 128:
        rope_offset = -(-lkv // 128) * 128
    else:
        raise ValueError(f"Expected cache width {lkv + rope} (compact) or 128-aligned, got {width}")
    kv_lens_d, page_d, cu_q_d = _i32(kv_lens, device), _i32(page_indices, device), _i32(cu_q_lens, device)
    cu_kv_d = _i32(cu_kv_lens, device) if cu_kv_lens is not None else None
    out = torch.empty_like(ql_nope)
    p = RpaMlaParams()
    p.ql_nope = ql_nope.data_ptr()
    p.q_pe = q_pe.data_ptr()
    p.out = out.data_ptr()
    p.cache_kv = cache_kv.data_ptr()
    p.kv_lens = kv_lens_d.data_ptr()
    p.page_indices = page_d.reshape(-1).data_ptr()
    p.cu_q_lens = cu_q_d.data_ptr()
    p.cu_kv_lens = cu_kv_d.data_ptr() if cu_kv_d is not None else None
    p.num_tokens = T
    p.num_seqs = k
    p.num_q_heads = Hq
    p.lkv_dim = lkv
    p.rope_dim = rope
    p.row_stride = width
    p.cache_dtype = _lib.RPA_KV_FP8_E4M3 if cache_kv.dtype == torch.float8_e4m3fn else _lib.RPA_KV_BF16
    p.rope_offset = rope_offset
    p.page_size = page_size
    p.total_pages = total_pages
    p.pages_per_seq = (page_d.numel() // max(kv_lens_d.shape[0], 1)) if cu_kv_d is None else 0
    p.max_kv_len = int(max_kv_len) if max_kv_len is not None else _host_max(kv_lens)
    p.num_splits = int(num_splits)
    p.sum_kv_len = int(sum_kv_len) if sum_kv_len is not None else _host_decode_sum(kv_lens, k)
    p.sliding_window = int(sliding_window) if sliding_window else 0
    p.sm_scale = float(sm_scale)
    p.soft_cap = float(soft_cap) if soft_cap else 0.0
    p.mask_value = float(mask_value) if mask_value is not None else DEFAULT_MASK_VALUE
    # scalar scales (mla_v2:372-375, 408-409): 0 in the C struct means "off"
    p.q_scale = float(q_scale) if q_scale is not None else 0.0
    p.k_scale = float(k_scale) if k_scale is not None else 0.0
    p.v_scale = float(v_scale) if v_scale is not None else 0.0
    dist_d = None
    if static_shapes:
        dist_d = distribution.contiguous()
        p.distribution = dist_d.data_ptr()
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    if new_kv_c is not None:
        _require_gpu(new_kv_c, "new_kv_c")
        if new_kv_c.shape != (T, lkv) or new_k_pe.shape != (T, rope):
            raise ValueError(f"Expected new_kv_c {(T, lkv)} and new_k_pe {(T, rope)}, got "
                             f"{tuple(new_kv_c.shape)} and {tuple(new_k_pe.shape)}")
        if not (new_kv_c.dtype == new_k_pe.dtype == cache_kv.dtype):
            raise ValueError("new_kv_c / new_k_pe must have the cache dtype")
        nk, nr = new_kv_c.contiguous(), new_k_pe.contiguous()
        _lib.check(lib.rpa_mla_kv_write(ctypes.byref(p), nk.data_ptr(), nr.data_ptr(), stream))
    need = (lib.rpa_mla_workspace_bytes if decode_only else lib.rpa_mla_attention_workspace_bytes)(ctypes.byref(p))
    if need:
        ws = _workspace(device, need)
        p.workspace = ws.data_ptr()
        p.workspace_bytes = ws.numel()
    _lib.check((lib.rpa_mla_decode if decode_only else lib.rpa_mla_attention)(ctypes.byref(p), stream))
    return out, cache_kv
