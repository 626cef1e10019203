"""The ``Attention`` module: the operator boundary the model layers call.

Mirrors diffulex/attention/attn_impl.py:13-72: reshape, optional KV-cache store,
prefill / decode dispatch, flatten heads.  ``k_cache`` / ``v_cache`` are assigned
from outside (diffulex/engine/model_runner.py:239-243).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import metadata as _metadata
from .dllm_flash_attn import dllm_flash_attn_decode, dllm_flash_attn_prefill, rope_supported
from .kv_cache_kernels import store_kvcache_distinct_layout, store_kvcache_unified_layout


class Attention(nn.Module):
    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])
        self.fuse_kv_store = True  # False: store in a launch of its own, as the reference does
        self.fuse_kv_store_max_bytes = 6 << 20  # bf16 bytes of fresh K plus V up to which the store is fused
        # looked up at call time so that a later set_fetch_fn_for_attn_metadata() is seen
        self.fetch_attn_metadata = lambda: _metadata.fetch_attn_metadata()

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask=None, rope=None) -> torch.Tensor:
        """``rope=(rotary_embedding, positions)`` (extension): q and k are the projections BEFORE the rotary
        embedding (diffulex/model/dream.py:94-99 applies it right before this call); it is applied inside
        the attention launch where that launch can (decode, unified layout, ``rope_supported``), by the
        rotary embedding's own launch otherwise -- which then also stores the block, in either cache layout,
        where a store is due."""
        stored = False
        if rope is not None:
            rotary, positions = rope
            md = self.fetch_attn_metadata()
            fused = (not md.is_prefill and md.kv_cache_layout == "unified" and self.k_cache.numel() > 0 and
                     rope_supported(self.num_heads, self.num_kv_heads, self.head_dim, int(md.max_seqlen_q or 0),
                                    self.k_cache.shape[1], md.cu_seqlens_q.numel() - 1, q.device))
            if fused:
                rope = (rotary.cos_sin_cache, positions)
            else:
                rope = None
                if (self.k_cache.numel() and self.v_cache.numel() and md.need_kv_cache_store
                        and self.k_cache.dtype == torch.bfloat16 and md.slot_mapping.numel() == k.shape[0]):
                    q, k = rotary.forward_and_store(positions, q, k, v, self.k_cache, self.v_cache, md.slot_mapping, md)
                    stored = True
                else:
                    q, k = rotary(positions, q, k)
        q = q.view(q.shape[0], self.num_heads, self.head_dim)
        k = k.view(k.shape[0], self.num_kv_heads, self.head_dim)
        v = v.view(v.shape[0], self.num_kv_heads, self.head_dim)

        attn_metadata = self.fetch_attn_metadata()
        k_cache, v_cache = self.k_cache, self.v_cache
        is_unified_layout = attn_metadata.kv_cache_layout == "unified"

        # Decode on the unified layout: the store rides in the attention launch (the block being
        # stored follows the attended context, so the two never touch the same slots).
        fused_slots = None
        if k_cache.numel() and v_cache.numel():
            if attn_metadata.need_kv_cache_store and not stored:
                slots = attn_metadata.slot_mapping
                # (worth it while the block is small: measured on an MI355X the fused form saves a
                # launch's worth of time up to about 4 MB of fresh K+V and loses beyond 8 MB, where a
                # store kernel of its own has far more loads in flight than the attention grid)
                if (self.fuse_kv_store and is_unified_layout and not attn_metadata.is_prefill
                        and (k.numel() * 4 <= self.fuse_kv_store_max_bytes or rope is not None)
                        and slots.is_contiguous() and slots.dtype in (torch.int32, torch.int64)):
                    fused_slots = slots
                else:
                    assert rope is None, "the rotary embedding inside the attention launch stores through that launch"
                    store_kvcache = store_kvcache_unified_layout if is_unified_layout else store_kvcache_distinct_layout
                    store_kvcache(k, v, k_cache, v_cache, slots, attn_metadata)

        if attn_metadata.is_prefill:
            o = dllm_flash_attn_prefill(q, k, v, self.scale, attn_metadata)
        else:
            if is_unified_layout:
                o = dllm_flash_attn_decode(q, k, v, k_cache, v_cache, self.scale, attn_metadata,
                                           store_slot_mapping=fused_slots, rope=rope)
            else:
                # (the reference raises NotImplementedError here, attn_impl.py:66-69)
                o = dllm_flash_attn_decode(q, k, v, k_cache, v_cache, self.scale, attn_metadata,
                                           kv_cache_layout="distinct")

        return o.reshape(o.shape[0], self.num_heads * self.head_dim).contiguous()
