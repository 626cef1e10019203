"""Rotary position embedding (same class, arguments and results as
diffulex/layer/rotary_embedding.py), backed by the gfx950 kernel, plus the fused
form that also stores the rotated K and V into the paged cache.

``RotaryEmbedding.forward(positions, query, key)`` returns new tensors, as the
reference does.  ``forward_and_store`` additionally writes token t's rotated key
row and its value row to cache slot ``slot_mapping[t]`` (what
``store_kvcache_unified_layout`` would do in a launch of its own, reading K and V
a second time); the caller then runs attention with
``attn_metadata.need_kv_cache_store = False``.
"""
from __future__ import annotations

from functools import lru_cache
from typing import Optional, Tuple

import torch
import torch.nn as nn

from . import _lib
from .kv_cache_kernels import _call, _scales


def _rows(x: torch.Tensor, head_size: int) -> Tuple[int, int, int]:
    """(tokens, heads, token stride in elements) of a [T, H * hd] or [T, H, hd] tensor."""
    assert x.is_cuda and x.dtype == torch.bfloat16, "rotary embedding runs on bf16 device tensors"
    assert x.dim() in (2, 3) and x.stride(-1) == 1
    if x.dim() == 3:
        assert x.shape[-1] == head_size and x.stride(1) == head_size
        return x.shape[0], x.shape[1], x.stride(0)
    assert x.shape[-1] % head_size == 0
    return x.shape[0], x.shape[-1] // head_size, x.stride(0)


class RotaryEmbedding(nn.Module):
    """rotary_embedding.py:20-66 (neox-style halves, rotary_dim == head_size)."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float) -> None:
        super().__init__()
        self.head_size = head_size
        assert rotary_dim == head_size
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))
        t = torch.arange(max_position_embeddings, dtype=torch.float)
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        self.register_buffer("cos_sin_cache", torch.cat((freqs.cos(), freqs.sin()), dim=-1), persistent=False)

    def _launch(self, positions, query, key, q_out, k_out, value=None, k_cache=None, v_cache=None,
                slot_mapping=None, attn_metadata=None, k_scale=None, v_scale=None) -> None:
        table = self.cos_sin_cache
        positions = positions.reshape(-1)
        if not positions.is_contiguous():
            positions = positions.contiguous()
        ks = vs = slots = None
        if slot_mapping is not None:
            slots = slot_mapping.reshape(-1)
            if not slots.is_contiguous():
                slots = slots.contiguous()
            Hk = key.shape[1] if key.dim() == 3 else key.shape[-1] // self.head_size
            ks, vs = _scales(k_cache, attn_metadata, k_scale, v_scale, Hk)
        _call(_lib.ops().rope_kv_store, positions, query, key, q_out, k_out, table, self.head_size, value, k_cache,
              v_cache, slots, ks, vs)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor
                ) -> Tuple[torch.Tensor, torch.Tensor]:
        q_out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        k_out = torch.empty(key.shape, dtype=key.dtype, device=key.device)
        self._launch(positions, query, key, q_out, k_out)
        return q_out, k_out

    def forward_and_store(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                          value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                          slot_mapping: torch.Tensor, attn_metadata=None,
                          k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None
                          ) -> Tuple[torch.Tensor, torch.Tensor]:
        """forward() and store_kvcache_unified_layout(rotated key, value, ...) in one launch -- or
        store_kvcache_distinct_layout(...) where the caches are in that layout (k_cache [pages, H_kv, hd / 8,
        page, 8], v_cache [pages, H_kv, hd, page], bf16)."""
        q_out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        k_out = torch.empty(key.shape, dtype=key.dtype, device=key.device)
        self._launch(positions, query, key, q_out, k_out, value, k_cache, v_cache, slot_mapping,
                     attn_metadata, k_scale, v_scale)
        return q_out, k_out


@lru_cache(1)
def get_rope(head_size: int, rotary_dim: int, max_position: int, base: float,
             rope_scaling: dict | None = None):
    """rotary_embedding.py:69-79."""
    assert rope_scaling is None
    return RotaryEmbedding(head_size, rotary_dim, max_position, base)
