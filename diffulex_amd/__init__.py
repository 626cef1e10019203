"""diffulex_amd: MI355X (gfx950) implementation of Diffulex's dLLM decoding hot path.

Exports the operator names of ``diffulex_kernel`` (diffulex_kernel/__init__.py:1-2,
plus ``load_kvcache``) and of ``diffulex.attention`` (``Attention``, the metadata
hook) and of ``diffulex.layer.rotary_embedding`` (``RotaryEmbedding``, ``get_rope``),
all backed by hand-written HIP kernels behind the C ABI of
``include/diffulex_amd.h``.
"""
from .metadata import (AttnMetaDataBase, PagedAttnMetaData, set_fetch_fn_for_attn_metadata, set_warming_up,
                       is_warming_up, reset_warming_up)
from . import metadata
from .kv_cache_kernels import store_kvcache_distinct_layout, store_kvcache_unified_layout, load_kvcache
from .dllm_flash_attn import dllm_flash_attn_decode, dllm_flash_attn_prefill, paged_attention
from .attn_impl import Attention
from .rotary_embedding import RotaryEmbedding, get_rope


def fetch_attn_metadata(*args, **kwargs):
    """Always calls the currently installed fetch function (diffulex/attention/__init__.py:6-14)."""
    return metadata.fetch_attn_metadata(*args, **kwargs)


__all__ = [
    "AttnMetaDataBase", "PagedAttnMetaData", "set_fetch_fn_for_attn_metadata", "fetch_attn_metadata",
    "set_warming_up", "is_warming_up", "reset_warming_up",
    "store_kvcache_distinct_layout", "store_kvcache_unified_layout", "load_kvcache",
    "dllm_flash_attn_decode", "dllm_flash_attn_prefill", "paged_attention", "Attention",
    "RotaryEmbedding", "get_rope",
]
