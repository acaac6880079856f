"""ctypes binding of ``librpa_mi355.so`` (the C ABI declared in include/rpa.h).

There is no CPU fallback: if the shared library has not been built the loader
raises, and every operator in this package raises with it.
"""

from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librpa_mi355.so")

RPA_KV_BF16 = 0
RPA_KV_FP8_E4M3 = 1
RPA_LAYOUT_FUSED = 0
RPA_LAYOUT_SPLIT = 1

STATUS_NAMES = {
    0: "RPA_OK",
    -1: "RPA_EINVAL_SHAPE",
    -2: "RPA_EINVAL_DTYPE",
    -3: "RPA_EINVAL_HEADS",
    -4: "RPA_EINVAL_PAGE_RANGE",
    -5: "RPA_EINVAL_QLEN_GT_KVLEN",
    -6: "RPA_EINVAL_WINDOW",
    -7: "RPA_EINVAL_SOFTCAP",
    -8: "RPA_EINVAL_WORKSPACE",
    -9: "RPA_EHIP",
    -10: "RPA_EINVAL_DISTRIBUTION",
    -11: "RPA_EUNSUPPORTED",
    -12: "RPA_EINVAL_NULL",
}

# every symbol include/rpa.h declares
EXPORTED_SYMBOLS = (
    "rpa_version",
    "rpa_last_error",
    "rpa_validate",
    "rpa_validate_host",
    "rpa_workspace_bytes",
    "rpa_mla_workspace_bytes",
    "rpa_gather_pages",
    "rpa_decode",
    "rpa_prefill",
    "rpa_attention",
    "rpa_describe_plan",
    "rpa_noalloc_max_workspace_bytes",
    "rpa_attention_noalloc",
    "rpa_kv_write",
    "rpa_mla_decode",
    "rpa_mla_attention_workspace_bytes",
    "rpa_mla_attention",
    "rpa_mla_kv_write",
    "rpa_mla_describe_plan",
)


class RpaParams(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("kv_cache", ctypes.c_void_p),
        ("v_pages", ctypes.c_void_p),
        ("kv_lens", ctypes.c_void_p),
        ("page_indices", ctypes.c_void_p),
        ("cu_q_lens", ctypes.c_void_p),
        ("cu_kv_lens", ctypes.c_void_p),
        ("k_scale", ctypes.c_void_p),
        ("v_scale", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("num_tokens", ctypes.c_int32),
        ("num_seqs", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("page_size", ctypes.c_int32),
        ("total_pages", ctypes.c_int32),
        ("pages_per_seq", ctypes.c_int32),
        ("layout", ctypes.c_int32),
        ("kv_dtype", ctypes.c_int32),
        ("decode_end", ctypes.c_int32),
        ("max_kv_len", ctypes.c_int32),
        ("max_q_len", ctypes.c_int32),
        ("num_splits", ctypes.c_int32),
        ("sliding_window", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("soft_cap", ctypes.c_float),
        ("mask_value", ctypes.c_float),
        ("sum_decode_kv_len", ctypes.c_int64),
        ("attention_sink", ctypes.c_void_p),
        ("custom_mask", ctypes.c_void_p),
        ("cu_mask_lens", ctypes.c_void_p),
        ("xai_temperature_len", ctypes.c_float),
        ("mask_mode", ctypes.c_int32),
        ("mask_rows_page_aligned", ctypes.c_int32),
        ("softmax_dtype", ctypes.c_int32),
        ("q_scale", ctypes.c_float),
        ("distribution", ctypes.c_void_p),
    ]


MASK_CAUSAL, MASK_CUSTOM, MASK_NONE = 0, 1, 2
SOFTMAX_F32, SOFTMAX_BF16, SOFTMAX_F16 = 0, 1, 2


class RpaMlaParams(ctypes.Structure):
    _fields_ = [
        ("ql_nope", ctypes.c_void_p),
        ("q_pe", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("cache_kv", ctypes.c_void_p),
        ("kv_lens", ctypes.c_void_p),
        ("page_indices", ctypes.c_void_p),
        ("cu_q_lens", ctypes.c_void_p),
        ("cu_kv_lens", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("num_tokens", ctypes.c_int32),
        ("num_seqs", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("lkv_dim", ctypes.c_int32),
        ("rope_dim", ctypes.c_int32),
        ("row_stride", ctypes.c_int32),
        ("rope_offset", ctypes.c_int32),
        ("page_size", ctypes.c_int32),
        ("total_pages", ctypes.c_int32),
        ("pages_per_seq", ctypes.c_int32),
        ("max_kv_len", ctypes.c_int32),
        ("num_splits", ctypes.c_int32),
        ("sliding_window", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("soft_cap", ctypes.c_float),
        ("mask_value", ctypes.c_float),
        ("sum_kv_len", ctypes.c_int64),
        ("q_scale", ctypes.c_float),
        ("k_scale", ctypes.c_float),
        ("v_scale", ctypes.c_float),
        ("distribution", ctypes.c_void_p),
        ("cache_dtype", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
    ]


class RpaLibraryMissing(RuntimeError):
    pass


_lib = None


def load() -> ctypes.CDLL:
    """Load the HIP library; raise RpaLibraryMissing when it was never built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RpaLibraryMissing(
            f"{LIB_PATH} not found: build it with `python sglang-jax_amd/build.py` "
            "(or __graft_entry__.build()); there is no CPU fallback"
        )
    lib = ctypes.CDLL(LIB_PATH)
    P = ctypes.POINTER
    i32p = P(ctypes.c_int32)
    lib.rpa_version.restype = ctypes.c_int
    lib.rpa_version.argtypes = []
    lib.rpa_last_error.restype = ctypes.c_char_p
    lib.rpa_last_error.argtypes = []
    lib.rpa_validate.restype = ctypes.c_int
    lib.rpa_validate.argtypes = [P(RpaParams)]
    lib.rpa_validate_host.restype = ctypes.c_int
    lib.rpa_validate_host.argtypes = [P(RpaParams), i32p, i32p, ctypes.c_int64, i32p, i32p, i32p]
    lib.rpa_workspace_bytes.restype = ctypes.c_size_t
    lib.rpa_workspace_bytes.argtypes = [P(RpaParams)]
    lib.rpa_mla_workspace_bytes.restype = ctypes.c_size_t
    lib.rpa_mla_workspace_bytes.argtypes = [P(RpaMlaParams)]
    lib.rpa_gather_pages.restype = ctypes.c_int
    lib.rpa_gather_pages.argtypes = [P(RpaParams), ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p,
                                     ctypes.c_int32, ctypes.c_void_p]
    lib.rpa_noalloc_max_workspace_bytes.restype = ctypes.c_size_t
    lib.rpa_noalloc_max_workspace_bytes.argtypes = []
    for name in ("rpa_decode", "rpa_prefill", "rpa_attention", "rpa_attention_noalloc"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [P(RpaParams), ctypes.c_void_p]
    lib.rpa_kv_write.restype = ctypes.c_int
    lib.rpa_kv_write.argtypes = [P(RpaParams), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.rpa_mla_decode.restype = ctypes.c_int
    lib.rpa_mla_decode.argtypes = [P(RpaMlaParams), ctypes.c_void_p]
    lib.rpa_mla_attention_workspace_bytes.restype = ctypes.c_size_t
    lib.rpa_mla_attention_workspace_bytes.argtypes = [P(RpaMlaParams)]
    lib.rpa_mla_attention.restype = ctypes.c_int
    lib.rpa_mla_attention.argtypes = [P(RpaMlaParams), ctypes.c_void_p]
    lib.rpa_mla_kv_write.restype = ctypes.c_int
    lib.rpa_mla_kv_write.argtypes = [P(RpaMlaParams), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.rpa_describe_plan.restype = ctypes.c_int
    lib.rpa_describe_plan.argtypes = [P(RpaParams), ctypes.c_char_p, ctypes.c_size_t]
    lib.rpa_mla_describe_plan.restype = ctypes.c_int
    lib.rpa_mla_describe_plan.argtypes = [P(RpaMlaParams), ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    _lib = lib
    return lib


class RpaError(ValueError):
    """A non-zero status from the C ABI.  ValueError, like the checks of the
    reference (ragged_paged_attention_v3.py:1344-1487)."""

    def __init__(self, code: int, message: str):
        super().__init__(f"{STATUS_NAMES.get(code, code)}: {message}")
        self.code = code


def check(code: int):
    if code != 0:
        raise RpaError(code, load().rpa_last_error().decode("utf-8", "replace"))


def describe_plan(params) -> str:
    """``rpa_describe_plan`` / ``rpa_mla_describe_plan``: the launch shape a call would take, as text."""
    lib = load()
    buf = ctypes.create_string_buffer(2048)
    if isinstance(params, RpaMlaParams):
        raise TypeError("use describe_mla_plan(params, token_rows)")
    n = lib.rpa_describe_plan(ctypes.byref(params), buf, len(buf))
    if n < 0:
        check(n)
    return buf.value.decode()


def describe_mla_plan(params, token_rows: bool) -> str:
    lib = load()
    buf = ctypes.create_string_buffer(1024)
    n = lib.rpa_mla_describe_plan(ctypes.byref(params), 1 if token_rows else 0, buf, len(buf))
    if n < 0:
        check(n)
    return buf.value.decode()
