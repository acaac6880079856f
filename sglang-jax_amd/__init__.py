"""MI355X-native ragged paged attention behind sglang-jax's operator surface.

The directory name carries a hyphen, so the package is registered under the
importable name ``sglang_jax_amd`` by ``__graft_entry__.load_package()``.
"""

from . import _lib  # noqa: F401
from .backend import (  # noqa: F401
    FlashAttention,
    FlashAttentionMetadata,
    ForwardMode,
    MLAAttentionBackend,
    build_forward_metadata,
    build_verify_metadata,
    pad_page_indices,
)
from .dsa import compute_topk_pages, sparse_mla_page_level, sparse_mla_via_dense  # noqa: F401
from .mla import mla_ragged_paged_attention  # noqa: F401
from .ragged_paged_attention import (  # noqa: F401
    DEFAULT_MASK_VALUE,
    gather_pages,
    ragged_paged_attention,
    ragged_paged_attention_ref_surface,
)

__all__ = [
    "FlashAttention",
    "FlashAttentionMetadata",
    "ForwardMode",
    "MLAAttentionBackend",
    "build_forward_metadata",
    "build_verify_metadata",
    "pad_page_indices",
    "DEFAULT_MASK_VALUE",
    "gather_pages",
    "mla_ragged_paged_attention",
    "ragged_paged_attention",
    "ragged_paged_attention_ref_surface",
]
