"""Host-side mirror of the reference's ragged paged attention operator.

Same names, argument meaning and error behaviour as
``python/sgl_jax/srt/kernels/ragged_paged_attention/ragged_paged_attention_v3.py``
of the reference (``rpa_v3`` below), but the arrays are torch tensors on a ROCm
device and the computation is the HIP library behind the C ABI of
``include/rpa.h``.  There is no CPU path here.

Two call surfaces:

* :func:`ragged_paged_attention` -- the production signature, rpa_v3:1667-1700:
  new ``keys/values`` are written into the fused, head-interleaved cache and the
  pair ``(output, updated_cache)`` is returned (the cache is updated in place and
  returned, matching the donated-buffer aliasing of rpa_v3:1973-1976);
* :func:`ragged_paged_attention_ref_surface` -- the argument list of
  ``ref_ragged_paged_attention`` (rpa_v3:94-114): separate ``k_pages/v_pages``
  that already hold every token, a zero-padded 2-D page table and ``num_seqs``.
"""

from __future__ import annotations

import ctypes
import math

import numpy as np
import torch

from . import _lib
from ._lib import RpaParams

# rpa_v3:47
DEFAULT_MASK_VALUE = -0.7 * float(np.finfo(np.float32).max)

_workspaces: dict = {}


def _workspace(device, nbytes: int) -> torch.Tensor:
    """Grow-only scratch for the split-KV partials, one per device and stream."""
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _kv_dtype_code(dtype) -> int:
    if dtype == torch.bfloat16:
        return _lib.RPA_KV_BF16
    if dtype in (torch.float8_e4m3fn,):
        return _lib.RPA_KV_FP8_E4M3
    raise ValueError(f"Expected kv cache dtype bfloat16 or float8_e4m3fn, got {dtype}")


def _per_head(scale, num_kv_heads, device):
    if scale is None:
        return None
    t = torch.as_tensor(scale, dtype=torch.float32, device=device).reshape(-1)
    if t.numel() == 1:
        t = t.expand(num_kv_heads)
    if t.numel() != num_kv_heads:
        raise ValueError(f"Expected a scalar or {num_kv_heads} per-head scales, got {t.numel()}")
    return t.contiguous()


def _i32(t, device):
    if isinstance(t, np.ndarray):
        t = torch.from_numpy(t)
    if t.dtype != torch.int32:
        raise ValueError(f"Expected int32 dtype for metadata, got {t.dtype}")
    return t.to(device).contiguous()


def _host_max(t):
    """Upper bound taken from a HOST copy only (never synchronises a device)."""
    if isinstance(t, np.ndarray):
        return int(t.max()) if t.size else 0
    if isinstance(t, torch.Tensor) and t.device.type == "cpu":
        return int(t.max()) if t.numel() else 0
    return 0


def _prefill_q_bound(cu_q_lens, dist, chunk_prefill_size, static_shapes):
    """Bound on the query length of the sequences behind the decode rows, which sizes the prefill grid (0 = the
    token count).  A host copy of ``cu_q_lens`` gives the exact maximum.  Without one, ``chunk_prefill_size`` is
    a bound only where the reference itself takes it for one: on the PREFILL partition [i, j), launched with
    ``static_q_len = chunk_prefill_size`` (rpa_v3:2074-2082).  Sequences of the MIXED partition [j, k) may be of
    any length (``static_q_len = None``, rpa_v3:2083-2090), and with the composition on the device j and k are
    unknown here: then only the token count bounds a chunk."""
    i, j, k = (int(x) for x in dist)
    host = None
    if isinstance(cu_q_lens, np.ndarray):
        host = cu_q_lens
    elif isinstance(cu_q_lens, torch.Tensor) and cu_q_lens.device.type == "cpu":
        host = cu_q_lens.numpy()
    if host is not None and not static_shapes:
        q = np.diff(host[i:k + 1])
        return int(q.max()) if q.size else 0
    if static_shapes or not chunk_prefill_size or j != k:
        return 0
    return int(chunk_prefill_size)


def static_validate_inputs(queries, keys, values, kv_cache_fused, kv_lens, page_indices, cu_q_lens,
                           cu_kv_lens, distribution, *, causal=1, sliding_window=None, soft_cap=None,
                           chunk_prefill_size=None, skip_kv_mask=False):
    """Shape/dtype contract of rpa_v3:1314-1439 (same messages where they apply)."""
    q, k, v = queries, keys, values
    if k is not None:
        if not (q.dim() == k.dim() == v.dim() == 3):
            raise ValueError(f"Expected 3D array for q.shape={tuple(q.shape)}, k.shape={tuple(k.shape)}, v.shape={tuple(v.shape)}")
        if k.shape != v.shape:
            raise ValueError(f"Expected k.shape={tuple(k.shape)} to be equal to v.shape={tuple(v.shape)}")
        if not (q.shape[0] == k.shape[0] == v.shape[0]):
            raise ValueError(f"Expected q.shape[0]={q.shape[0]} to be equal to k.shape[0]={k.shape[0]} and v.shape[0]={v.shape[0]}")
        if not (q.shape[2] == k.shape[2] == v.shape[2]):
            raise ValueError(f"Expected q.shape[2]={q.shape[2]} to be equal to k.shape[2]={k.shape[2]} and v.shape[2]={v.shape[2]}")
        num_kv_heads = k.shape[1]
    else:
        if q.dim() != 3:
            raise ValueError(f"Expected 3D array for q.shape={tuple(q.shape)}")
        num_kv_heads = kv_cache_fused.shape[2] // 2
    if q.shape[1] % num_kv_heads != 0:
        raise ValueError(f"Expected actual_num_q_heads={q.shape[1]} to be divisible by actual_num_kv_heads={num_kv_heads}.")
    if not kv_cache_fused.dtype.is_floating_point:
        raise ValueError(f"Expected kv_cache_fused.dtype={kv_cache_fused.dtype} to be a floating point.")
    for name, t in (("kv_lens", kv_lens), ("page_indices", page_indices), ("cu_q_lens", cu_q_lens),
                    ("cu_kv_lens", cu_kv_lens), ("distribution", distribution)):
        if t.dtype != torch.int32:
            raise ValueError(f"Expected int32 dtype for {name}.dtype={t.dtype}")
    if not (kv_lens.dim() == page_indices.dim() == cu_q_lens.dim() == 1):
        raise ValueError("Expected 1D array for kv_lens, page_indices, cu_q_lens")
    max_num_seqs = kv_lens.shape[0]
    if tuple(cu_q_lens.shape) != (max_num_seqs + 1,):
        raise ValueError(f"Expected cu_q_lens.shape={tuple(cu_q_lens.shape)} to be ({max_num_seqs + 1},).")
    if tuple(cu_kv_lens.shape) != (max_num_seqs + 1,):
        raise ValueError(f"Expected cu_kv_lens.shape={tuple(cu_kv_lens.shape)} to be ({max_num_seqs + 1},).")
    if tuple(distribution.shape) != (3,):
        raise ValueError(f"Expected distribution.shape={tuple(distribution.shape)} to be (3,).")
    if sliding_window is not None and sliding_window <= 0:
        raise ValueError(f"sliding_window={sliding_window} must be positive.")
    if soft_cap is not None and soft_cap == 0.0:
        raise ValueError(f"soft_cap={soft_cap} must not be 0.0.")
    if chunk_prefill_size is not None and chunk_prefill_size <= 0:
        raise ValueError(f"chunk_prefill_size={chunk_prefill_size} must be positive.")
    if skip_kv_mask and causal == 1:
        raise ValueError("Cannot skip kv mask when using causal mask.")


def dynamic_validate_inputs(params: RpaParams, kv_lens, page_indices, cu_q_lens, cu_kv_lens, distribution):
    """Value checks of rpa_v3:1442-1487 on HOST copies of the metadata (numpy int32)."""
    lib = _lib.load()
    keep = [np.ascontiguousarray(a, dtype=np.int32) if a is not None else None
            for a in (kv_lens, page_indices, cu_q_lens, cu_kv_lens, distribution)]
    ptrs = [None if a is None else a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)) for a in keep]
    _lib.check(lib.rpa_validate_host(ctypes.byref(params), ptrs[0], ptrs[1], int(keep[1].size), ptrs[2], ptrs[3], ptrs[4]))


def _fill_common(p: RpaParams, q, out, *, num_seqs, decode_end, page_size, total_pages, num_kv_heads,
                 kv_dtype, sm_scale, sliding_window, soft_cap, mask_value, max_kv_len, max_q_len, num_splits,
                 sum_decode_kv_len=0):
    p.q = q.data_ptr()
    p.out = out.data_ptr()
    p.num_tokens = q.shape[0]
    p.num_seqs = int(num_seqs)
    p.num_q_heads = q.shape[1]
    p.num_kv_heads = int(num_kv_heads)
    p.head_dim = q.shape[2]
    p.page_size = int(page_size)
    p.total_pages = int(total_pages)
    p.kv_dtype = _kv_dtype_code(kv_dtype)
    p.decode_end = int(decode_end)
    p.max_kv_len = int(max_kv_len)
    p.max_q_len = int(max_q_len)
    p.num_splits = int(num_splits)
    p.sliding_window = int(sliding_window) if sliding_window else 0
    p.sm_scale = float(sm_scale)
    p.soft_cap = float(soft_cap) if soft_cap else 0.0
    p.mask_value = float(mask_value) if mask_value is not None else DEFAULT_MASK_VALUE
    p.sum_decode_kv_len = int(sum_decode_kv_len)


def _host_decode_sum(kv_lens, decode_end):
    """Sum of the decode rows' kv lengths, from a HOST copy only (0 when there is none)."""
    if isinstance(kv_lens, torch.Tensor) and kv_lens.device.type == "cpu":
        return int(kv_lens[:decode_end].sum()) if decode_end else 0
    if isinstance(kv_lens, np.ndarray):
        return int(kv_lens[:decode_end].sum()) if decode_end else 0
    return 0


def _require_gpu(t, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise RuntimeError(f"{name} must be a tensor on a ROCm device: this operator has no CPU path")


class RpaCall:
    """One prepared call: the filled ``RpaParams`` plus every tensor it points at.

    ``attention()`` = ``rpa_attention`` (decode rows, then prefill/mixed rows);
    ``decode()`` / ``prefill()`` run the two partitions on their own, which is how
    the benchmark times them separately.  Launches go to torch's current stream.

    The split-KV workspace is by default the one grow-only buffer of (device, stream current at
    construction), shared by every call prepared on that stream: calls that share it must be
    ordered on one stream.  A call that is kept and launched from elsewhere -- captured into a
    graph, replayed while eager calls run, issued on another stream -- takes
    ``own_workspace=True`` and holds a buffer of its own for as long as it lives.
    """

    def __init__(self, queries, kv_cache, v_pages, kv_lens_d, page_d, cu_q_d, cu_kv_d, *, num_seqs, decode_end,
                 sm_scale, sliding_window=None, soft_cap=None, mask_value=DEFAULT_MASK_VALUE, k_scale=None,
                 v_scale=None, max_kv_len=0, max_q_len=0, num_splits=0, out=None, sum_decode_kv_len=0,
                 attention_sink=None, xai_temperature_len=None, causal=True, custom_mask=None,
                 mask_aligned_to_cu_kv=False, softmax_dtype=None, q_scale=None, distribution_d=None,
                 own_workspace=False):
        self.lib = _lib.load()
        self.device = queries.device
        fused = v_pages is None
        if fused:
            total_pages, page_size, h2, _ = kv_cache.shape
            num_kv_heads = h2 // 2
        else:
            total_pages, page_size, num_kv_heads, _ = kv_cache.shape
        self.out = torch.empty_like(queries) if out is None else out
        self.ks = _per_head(k_scale, num_kv_heads, self.device)
        self.vs = _per_head(v_scale, num_kv_heads, self.device)
        self.tensors = (queries, kv_cache, v_pages, kv_lens_d, page_d, cu_q_d, cu_kv_d)
        p = RpaParams()
        _fill_common(p, queries, self.out, num_seqs=num_seqs, decode_end=decode_end, page_size=page_size,
                     total_pages=total_pages, num_kv_heads=num_kv_heads, kv_dtype=kv_cache.dtype, sm_scale=sm_scale,
                     sliding_window=sliding_window, soft_cap=soft_cap, mask_value=mask_value, max_kv_len=max_kv_len,
                     max_q_len=max_q_len, num_splits=num_splits, sum_decode_kv_len=sum_decode_kv_len)
        p.kv_cache = kv_cache.data_ptr()
        p.v_pages = None if fused else v_pages.data_ptr()
        p.layout = _lib.RPA_LAYOUT_FUSED if fused else _lib.RPA_LAYOUT_SPLIT
        p.kv_lens = kv_lens_d.data_ptr()
        p.page_indices = page_d.data_ptr()
        p.cu_q_lens = cu_q_d.data_ptr()
        p.cu_kv_lens = None if cu_kv_d is None else cu_kv_d.data_ptr()
        p.pages_per_seq = page_d.shape[1] if page_d.dim() == 2 else 0
        p.k_scale = self.ks.data_ptr() if self.ks is not None else None
        p.v_scale = self.vs.data_ptr() if self.vs is not None else None
        # ---- static-shape mode: (decode_end, prefill_end, num_seqs) stays on the device (rpa_v3:1676);
        # num_seqs is then the static bound and decode_end is not read
        self.distribution_d = None
        if distribution_d is not None:
            if distribution_d.dtype != torch.int32 or tuple(distribution_d.shape) != (3,):
                raise ValueError(f"Expected int32 distribution of shape (3,), got {distribution_d.dtype} {tuple(distribution_d.shape)}")
            self.distribution_d = distribution_d.to(self.device).contiguous()
            p.distribution = self.distribution_d.data_ptr()
        # ---- attention sink: scalar or one logit per query head (rpa_v3:185-193)
        self.sink = None
        if attention_sink is not None:
            sink = torch.as_tensor(attention_sink, dtype=torch.float32).reshape(-1)
            if sink.numel() == 1:
                sink = sink.expand(queries.shape[1])
            if sink.numel() != queries.shape[1]:
                raise ValueError(f"Expected attention_sink with {queries.shape[1]} entries, got {sink.numel()}")
            self.sink = sink.to(self.device).contiguous()
            p.attention_sink = self.sink.data_ptr()
        if xai_temperature_len is not None:
            if not xai_temperature_len > 0:
                raise ValueError(f"xai_temperature_len={xai_temperature_len} must be positive.")
            p.xai_temperature_len = float(xai_temperature_len)
        # ---- softmax_dtype (rpa_v3:181-186, kernel :522-523): logits rounded to it before the softmax
        if softmax_dtype in (None, torch.float32):
            p.softmax_dtype = _lib.SOFTMAX_F32
        elif softmax_dtype == torch.bfloat16:
            p.softmax_dtype = _lib.SOFTMAX_BF16
        elif softmax_dtype == torch.float16:
            p.softmax_dtype = _lib.SOFTMAX_F16
        elif isinstance(softmax_dtype, torch.dtype) and softmax_dtype.is_floating_point:
            raise NotImplementedError(f"softmax_dtype={softmax_dtype}: float32, bfloat16 and float16 are built")
        else:
            raise ValueError(f"Expected softmax_dtype to be a floating point dtype, got {softmax_dtype}")
        # ---- q_scale (kernel rpa_v3:463-478): queries quantised to the cache's element type
        if q_scale is not None:
            if not q_scale > 0:
                raise ValueError(f"q_scale={q_scale} must be positive.")
            p.q_scale = float(q_scale)
        # ---- mask mode (rpa_v3:152-165): causal, the caller's flat mask, or none
        self.mask = self.cu_mask = None
        if causal:
            p.mask_mode = _lib.MASK_CAUSAL
        elif custom_mask is None:
            p.mask_mode = _lib.MASK_NONE
        else:
            mask = custom_mask
            if mask.dtype == torch.bool:
                mask = mask.to(torch.int32)
            if mask.dtype != torch.int32:
                raise ValueError(f"Expected int32 (or bool) custom_mask, got {mask.dtype}")
            self.mask = mask.to(self.device).contiguous().reshape(-1)
            # cu_seq_mask_lens = [0, cumsum(q_len * row width)] on the device (rpa_v3:1801-1806)
            q_lens = (cu_q_d[1:] - cu_q_d[:-1]).to(torch.int64)
            if mask_aligned_to_cu_kv:
                if cu_kv_d is None:
                    raise ValueError("mask_aligned_to_cu_kv needs cu_kv_lens")
                widths = (cu_kv_d[1:] - cu_kv_d[:-1]).to(torch.int64)
            else:
                widths = kv_lens_d[: q_lens.shape[0]].to(torch.int64)
            cu = torch.zeros(q_lens.shape[0] + 1, dtype=torch.int64, device=self.device)
            cu[1:] = torch.cumsum(q_lens * widths[: q_lens.shape[0]], dim=0)
            self.cu_mask = cu.to(torch.int32)
            p.mask_mode = _lib.MASK_CUSTOM
            p.custom_mask = self.mask.data_ptr()
            p.cu_mask_lens = self.cu_mask.data_ptr()
            p.mask_rows_page_aligned = 1 if mask_aligned_to_cu_kv else 0
        need = self.lib.rpa_workspace_bytes(ctypes.byref(p))
        self.workspace = None
        if need:
            self.workspace = (torch.empty(need, dtype=torch.uint8, device=self.device) if own_workspace
                              else _workspace(self.device, need))
            p.workspace = self.workspace.data_ptr()
            p.workspace_bytes = self.workspace.numel()
        self.params = p

    def _stream(self):
        return ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def attention(self):
        _lib.check(self.lib.rpa_attention(ctypes.byref(self.params), self._stream()))

    def attention_noalloc(self):
        """``rpa_attention_noalloc``: the library's own workspace instead of this call's."""
        _lib.check(self.lib.rpa_attention_noalloc(ctypes.byref(self.params), self._stream()))

    def decode(self):
        _lib.check(self.lib.rpa_decode(ctypes.byref(self.params), self._stream()))

    def prefill(self):
        _lib.check(self.lib.rpa_prefill(ctypes.byref(self.params), self._stream()))

    def kv_write(self, keys, values):
        _lib.check(self.lib.rpa_kv_write(ctypes.byref(self.params), _ptr(keys), _ptr(values), self._stream()))


def ragged_paged_attention(
    queries: torch.Tensor,  # [max_num_tokens, num_q_heads, head_dim]
    keys: torch.Tensor | None,  # [max_num_tokens, num_kv_heads, head_dim] or None (cache already complete)
    values: torch.Tensor | None,
    kv_cache_fused: torch.Tensor,  # [total_num_pages, page_size, num_kv_heads * 2, head_dim]
    kv_lens,  # i32[max_num_seqs]
    page_indices,  # i32[flat]
    cu_q_lens,  # i32[max_num_seqs + 1]
    cu_kv_lens,  # i32[max_num_seqs + 1]
    distribution,  # i32[3]  (host array or tensor)
    custom_mask=None,
    attention_sink=None,
    *,
    causal: int = 1,
    sm_scale: float = 1.0,
    sliding_window: int | None = None,
    soft_cap: float | None = None,
    mask_value: float | None = DEFAULT_MASK_VALUE,
    q_scale: float | None = None,
    k_scale=None,
    v_scale=None,
    xai_temperature_len: float | None = None,
    softmax_dtype=None,
    chunk_prefill_size: int | None = None,
    d_block_sizes=None,
    p_block_sizes=None,
    m_block_sizes=None,
    vmem_limit_bytes: int | None = None,
    out_dtype=None,
    skip_kv_mask: bool = False,
    disable_semaphore_checks: bool = True,
    debug_mode: bool = False,
    mask_aligned_to_cu_kv: bool = False,
    # ---- additions of this implementation (host-side bounds, never synchronise) ----
    max_kv_len: int | None = None,
    max_q_len: int | None = None,
    num_splits: int = 0,
    validate_values: bool = False,
    host_kv_lens=None,
):
    """Ragged paged attention with fused KV cache; returns (output, updated_kv_cache_fused).

    Mirrors rpa_v3:1667-1733.  TPU tuning knobs (block sizes, vmem limit, semaphore
    checks, debug mode) are accepted and ignored.  ``k_scale``/``v_scale`` may be a
    float (reference) or one value per kv head.  ``distribution`` and the optional
    ``max_kv_len``/``max_q_len`` are host values used only to size launch grids
    (``max_q_len`` left out: the exact maximum when ``cu_q_lens`` is a host array; else
    ``chunk_prefill_size`` when the batch has no MIXED partition, whose sequences the reference lets be
    of any length; else the token count).  A sequence longer than a ``max_q_len`` the caller passes
    loses its rows past the bound: it is a promise, like a static shape.
    ``host_kv_lens`` is an optional host copy of ``kv_lens`` (the split plan balances on its
    sum) for callers that pass ``kv_lens`` as a device tensor.

    Static-shape mode: a ``distribution`` that lives on the GPU is never read back.  Grids are then
    sized from the static shapes alone (tokens, ``kv_lens.shape[0]`` sequences, the page-table
    bound) and the kernels read the batch composition themselves, as the jitted reference does
    (rpa_v3:1676): one prepared call serves every batch of a bucket.
    """
    _require_gpu(queries, "queries")
    _require_gpu(kv_cache_fused, "kv_cache_fused")
    device = queries.device
    static_shapes = isinstance(distribution, torch.Tensor) and distribution.is_cuda
    if static_shapes:
        dist = np.array([0, 0, kv_lens.shape[0]], dtype=np.int32)  # bounds only; the device holds the values
    elif isinstance(distribution, torch.Tensor):
        dist = distribution.cpu().numpy()
    elif isinstance(distribution, np.ndarray):
        dist = distribution
    else:
        dist = np.asarray(distribution, dtype=np.int32)
    dist_t = torch.as_tensor(dist)
    kv_lens_d, page_d, cu_q_d, cu_kv_d = (_i32(x, device) for x in (kv_lens, page_indices, cu_q_lens, cu_kv_lens))
    static_validate_inputs(queries, keys, values, kv_cache_fused, kv_lens_d, page_d, cu_q_d, cu_kv_d, dist_t,
                           causal=causal, sliding_window=sliding_window, soft_cap=soft_cap,
                           chunk_prefill_size=chunk_prefill_size, skip_kv_mask=skip_kv_mask)
    if kv_cache_fused.dim() == 5:  # reference's packed view [pages, P, 2Hkv/pack, pack, D]
        s = kv_cache_fused.shape
        kv_cache_fused = kv_cache_fused.view(s[0], s[1], s[2] * s[3], s[4])
    if not (queries.is_contiguous() and kv_cache_fused.is_contiguous()):
        raise ValueError("queries and kv_cache_fused must be contiguous")
    # rpa_v3 sets no query dtype; the engine hands over the model's (bf16, f16 or f32).  The matrix
    # units here take bf16 operands: wider queries are rounded to bf16 once (2^-9 relative, inside
    # the parity tolerance) and the output comes back in the query dtype as in rpa_v3:1788
    q_dtype = queries.dtype
    if q_dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise ValueError(f"Expected bfloat16, float16 or float32 queries, got {queries.dtype}")
    if q_dtype != torch.bfloat16:
        queries = queries.to(torch.bfloat16)
    if out_dtype is None:
        out_dtype = q_dtype

    # rpa_v3:1187-1241, 1270-1296: head dims that are not a multiple of 128 (64, 80, 96, 192 ...) run
    # zero-padded.  The engine's pool already stores aligned rows (memory_pool.py:70): then only the
    # queries and the new tokens are padded here.  A cache with narrow rows is padded, run and copied
    # back, as the reference does.
    actual_head_dim = queries.shape[2]
    caller_cache = kv_cache_fused
    if kv_cache_fused.shape[3] % 128 != 0:
        kv_cache_fused = torch.nn.functional.pad(kv_cache_fused, (0, -kv_cache_fused.shape[3] % 128))
    total_pages, page_size, h2, head_dim = kv_cache_fused.shape
    num_kv_heads = h2 // 2
    if not (actual_head_dim <= head_dim < actual_head_dim + 128):
        raise ValueError(f"Expected cache head_dim={caller_cache.shape[3]} to be q head_dim={actual_head_dim}, "
                         "or that rounded up to a multiple of 128")
    if actual_head_dim != head_dim:
        queries = torch.nn.functional.pad(queries, (0, head_dim - actual_head_dim))
        if keys is not None:
            keys = torch.nn.functional.pad(keys, (0, head_dim - actual_head_dim))
            values = torch.nn.functional.pad(values, (0, head_dim - actual_head_dim))
    i, j, k = (int(x) for x in dist)
    if not (i <= j <= k):
        raise ValueError(f"distribution must satisfy i <= j <= k, got {i}, {j}, {k}")
    if k > kv_lens_d.shape[0]:
        raise ValueError(f"distribution[2]={k} exceeds max_num_seqs={kv_lens_d.shape[0]}")

    # rpa_v3:1788: bfloat16 unless asked otherwise.  The kernels normalise in f32 and round the
    # finished row to bf16 once; float32 output is those values widened (one bf16 rounding more
    # than the reference's f32 accumulator leaves, far inside the parity tolerance)
    if out_dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError("out_dtype must be bfloat16, float16 or float32")
    call = RpaCall(queries, kv_cache_fused, None, kv_lens_d, page_d, cu_q_d, cu_kv_d, num_seqs=k, decode_end=i,
                   sm_scale=sm_scale, sliding_window=sliding_window, soft_cap=soft_cap, mask_value=mask_value,
                   k_scale=k_scale, v_scale=v_scale,
                   max_kv_len=max_kv_len if max_kv_len is not None else _host_max(
                       host_kv_lens if host_kv_lens is not None else kv_lens),
                   max_q_len=max_q_len if max_q_len is not None else _prefill_q_bound(
                       cu_q_lens, dist, chunk_prefill_size, static_shapes), num_splits=num_splits,
                   sum_decode_kv_len=_host_decode_sum(host_kv_lens if host_kv_lens is not None else kv_lens, i),
                   attention_sink=attention_sink, xai_temperature_len=xai_temperature_len, causal=bool(causal),
                   custom_mask=custom_mask, mask_aligned_to_cu_kv=mask_aligned_to_cu_kv,
                   softmax_dtype=softmax_dtype, q_scale=q_scale,
                   distribution_d=distribution if static_shapes else None)
    if validate_values:
        if static_shapes:
            raise ValueError("validate_values reads the metadata back to the host: not available with a device-side distribution")
        dynamic_validate_inputs(call.params, kv_lens_d.cpu().numpy(), page_d.cpu().numpy(), cu_q_d.cpu().numpy(),
                                cu_kv_d.cpu().numpy(), dist.astype(np.int32))
    if keys is not None:
        _require_gpu(keys, "keys")
        if keys.dtype != kv_cache_fused.dtype or values.dtype != kv_cache_fused.dtype:
            raise ValueError(f"Expected keys/values dtype {kv_cache_fused.dtype}, got {keys.dtype}/{values.dtype}")
        call.kv_write(keys.contiguous(), values.contiguous())
    call.attention()
    out = call.out
    if actual_head_dim != head_dim:
        out = out[:, :, :actual_head_dim].contiguous()
    if out_dtype != torch.bfloat16:
        out = out.to(out_dtype)
    if kv_cache_fused is not caller_cache:  # narrow rows: the new tokens go back into the caller's cache
        if keys is not None:
            caller_cache.copy_(kv_cache_fused[..., : caller_cache.shape[3]])
        kv_cache_fused = caller_cache
    return out, kv_cache_fused


def ragged_paged_attention_ref_surface(
    queries: torch.Tensor,  # [padded_num_tokens, num_q_heads, head_dim]
    k_pages: torch.Tensor,  # [total_num_pages, page_size, num_kv_heads, head_dim]
    v_pages: torch.Tensor,
    kv_lens,  # i32[padded_batch_size]
    page_indices,  # i32[padded_batch_size, max_pages_per_seq]
    cu_q_lens,  # i32[padded_batch_size + 1]
    num_seqs,  # i32[1] (host) or int
    *,
    causal: bool = True,
    sm_scale: float = 1.0,
    sliding_window: int | None = None,
    soft_cap: float | None = None,
    mask_value: float | None = DEFAULT_MASK_VALUE,
    k_scale=None,
    v_scale=None,
    custom_mask=None,
    xai_temperature_len: float | None = None,
    attention_sink=None,
    softmax_dtype=None,
    decode_end: int = 0,
    max_kv_len: int | None = None,
    max_q_len: int | None = None,
    num_splits: int = 0,
) -> torch.Tensor:
    """The argument list of ref_ragged_paged_attention (rpa_v3:94-114) on the HIP
    kernels.  Returns [padded_num_tokens, Hq, D]; only rows < cu_q_lens[num_seqs]
    are defined (the reference returns exactly those rows).  ``decode_end`` tells
    how many leading sequences are single-token rows (0 is always valid: the
    flash kernel handles q_len == 1 too)."""
    _require_gpu(queries, "queries")
    if sliding_window is not None and sliding_window <= 0:
        raise ValueError(f"sliding_window={sliding_window} must be positive.")
    if soft_cap is not None and soft_cap == 0.0:
        raise ValueError(f"soft_cap={soft_cap} must not be 0.0.")
    device = queries.device
    n = int(num_seqs[0]) if not isinstance(num_seqs, int) else num_seqs
    total_pages, page_size, num_kv_heads, head_dim = k_pages.shape
    if queries.shape[1] % num_kv_heads != 0:
        raise ValueError(f"Expected num_q_heads={queries.shape[1]} to be divisible by num_kv_heads={num_kv_heads}.")
    if k_pages.shape != v_pages.shape:
        raise ValueError(f"Expected k_pages.shape={tuple(k_pages.shape)} to be equal to v_pages.shape={tuple(v_pages.shape)}")
    if not (k_pages.is_contiguous() and v_pages.is_contiguous() and queries.is_contiguous()):
        raise ValueError("queries, k_pages and v_pages must be contiguous")
    kv_lens_d, cu_q_d = _i32(kv_lens, device), _i32(cu_q_lens, device)
    page_d = _i32(page_indices, device)
    if page_d.dim() != 2:
        raise ValueError(f"Expected 2D page_indices, got shape {tuple(page_d.shape)}")
    call = RpaCall(queries, k_pages, v_pages, kv_lens_d, page_d, cu_q_d, None, num_seqs=n, decode_end=decode_end,
                   sm_scale=sm_scale, sliding_window=sliding_window, soft_cap=soft_cap, mask_value=mask_value,
                   k_scale=k_scale, v_scale=v_scale,
                   max_kv_len=max_kv_len if max_kv_len is not None else _host_max(kv_lens),
                   max_q_len=max_q_len if max_q_len is not None else 0, num_splits=num_splits,
                   sum_decode_kv_len=_host_decode_sum(kv_lens, decode_end), attention_sink=attention_sink,
                   xai_temperature_len=xai_temperature_len, causal=bool(causal), custom_mask=custom_mask,
                   softmax_dtype=softmax_dtype)
    call.attention()
    return call.out


def gather_pages(kv_cache_fused: torch.Tensor, kv_lens, page_indices, cu_kv_lens, seq: int, kv_len: int):
    """K and V rows of sequence ``seq`` gathered through the page table, bit for
    bit: the indexing expression of rpa_v3:138-139 on its own.  Returns
    (k [kv_len, Hkv, D], v [kv_len, Hkv, D]) in the cache dtype."""
    _require_gpu(kv_cache_fused, "kv_cache_fused")
    device = kv_cache_fused.device
    total_pages, page_size, h2, head_dim = kv_cache_fused.shape
    num_kv_heads = h2 // 2
    kv_lens_d, page_d, cu_kv_d = _i32(kv_lens, device), _i32(page_indices, device), _i32(cu_kv_lens, device)
    k_out = torch.empty((kv_len, num_kv_heads, head_dim), dtype=kv_cache_fused.dtype, device=device)
    v_out = torch.empty_like(k_out)
    dummy = torch.zeros(2, dtype=torch.int32, device=device)
    p = RpaParams()
    p.q = dummy.data_ptr()
    p.out = dummy.data_ptr()
    p.kv_cache = kv_cache_fused.data_ptr()
    p.layout = _lib.RPA_LAYOUT_FUSED
    p.kv_lens = kv_lens_d.data_ptr()
    p.page_indices = page_d.data_ptr()
    p.cu_q_lens = dummy.data_ptr()
    p.cu_kv_lens = cu_kv_d.data_ptr()
    p.num_tokens = 0
    p.num_seqs = kv_lens_d.shape[0]
    p.num_q_heads = num_kv_heads
    p.num_kv_heads = num_kv_heads
    p.head_dim = head_dim
    p.page_size = page_size
    p.total_pages = total_pages
    p.kv_dtype = _kv_dtype_code(kv_cache_fused.dtype)
    p.sm_scale = 1.0
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    _lib.check(lib.rpa_gather_pages(ctypes.byref(p), int(seq), _ptr(k_out), _ptr(v_out), int(kv_len), stream))
    return k_out, v_out


def default_sm_scale(head_dim: int) -> float:
    """layers/attention/flashattention_backend.py:630-634: 1/sqrt(head_dim) unless the layer sets one."""
    return 1.0 / math.sqrt(head_dim)
