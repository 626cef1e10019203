"""Paged KV-cache store / load operators (same names, arguments and assertions as
diffulex_kernel/python/kv_cache_kernels.py), backed by the gfx950 kernels.

An FP8 cache is recognised by its dtype (``torch.float8_e4m3fn``, or ``uint8``
holding the codes); its per-KV-head scales come from the ``k_scale`` /
``v_scale`` keyword arguments or, if absent, from attributes of the same names
on ``attn_metadata``.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

_FP8_DTYPES = (torch.float8_e4m3fn, torch.uint8)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _index_type(t: torch.Tensor) -> int:
    if t.dtype == torch.int32:
        return _lib.DFX_INDEX_I32
    if t.dtype == torch.int64:
        return _lib.DFX_INDEX_I64
    raise AssertionError(f"slot_mapping must be int32 or int64, got {t.dtype}")


def _scales(cache: torch.Tensor, attn_metadata, k_scale, v_scale, n_heads: int):
    """(k_scale, v_scale) as fp32 device tensors for an FP8 cache, (None, None) otherwise."""
    if cache.dtype not in _FP8_DTYPES:
        assert cache.element_size() == 2, f"unsupported cache dtype {cache.dtype}"
        return None, None
    ks = k_scale if k_scale is not None else getattr(attn_metadata, "k_scale", None)
    vs = v_scale if v_scale is not None else getattr(attn_metadata, "v_scale", None)
    assert ks is not None and vs is not None, "an FP8 KV cache needs k_scale and v_scale"
    ks = ks.to(device=cache.device, dtype=torch.float32).contiguous()
    vs = vs.to(device=cache.device, dtype=torch.float32).contiguous()
    assert ks.numel() == n_heads and vs.numel() == n_heads
    return ks, vs


def _call(op, *args):
    """Run an operator of torch.ops.diffulex_amd; a status the C ABI returned surfaces as DfxError."""
    try:
        return op(*args)
    except RuntimeError as e:
        if "dfx_" in str(e):
            raise _lib.DfxError(str(e).split("\n")[0]) from None
        raise


def store_kvcache_unified_layout(key: torch.Tensor, value: torch.Tensor,
                                 k_cache: torch.Tensor, v_cache: torch.Tensor,
                                 slot_mapping: torch.Tensor, attn_metadata,
                                 k_scale: Optional[torch.Tensor] = None,
                                 v_scale: Optional[torch.Tensor] = None) -> None:
    """kv_cache_kernels.py:110-124.  key/value: [N, H_kv, hd]; caches: [pages, page, H_kv, hd]."""
    N, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == D and v_cache.stride(1) == D
    assert N == slot_mapping.numel(), f"`N`: {N}, `slot_mapping.numel()`: {slot_mapping.numel()}"
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert key.is_cuda and k_cache.is_cuda and slot_mapping.is_cuda
    assert key.element_size() == 2 and value.element_size() == 2
    ks, vs = _scales(k_cache, attn_metadata, k_scale, v_scale, num_heads)
    slots = slot_mapping.reshape(-1)
    if not slots.is_contiguous():
        slots = slots.contiguous()
    _index_type(slots)
    _call(_lib.ops().kv_store_unified, key, value, k_cache, v_cache, slots, ks, vs)


def store_kvcache_distinct_layout(key: torch.Tensor, value: torch.Tensor,
                                  k_cache: torch.Tensor, v_cache: torch.Tensor,
                                  slot_mapping: torch.Tensor, attn_metadata) -> None:
    """kv_cache_kernels.py:86-107.  k_cache: [pages, H, hd // x, page, x]; v_cache: [pages, H, hd, page]."""
    NBlks, NHeads, HDim_x, Blk_sz, x = k_cache.shape
    HDim = HDim_x * x
    N = key.shape[0]
    assert HDim == key.shape[-1] and NHeads == key.shape[1]
    assert N == slot_mapping.numel()
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == HDim and value.stride(1) == HDim
    assert key.element_size() == 2 and k_cache.element_size() == 2 and v_cache.element_size() == 2
    slots = slot_mapping.reshape(-1)
    if not slots.is_contiguous():
        slots = slots.contiguous()
    _index_type(slots)
    _call(_lib.ops().kv_store_distinct, key, value, k_cache, v_cache, slots)


def load_kvcache(k_cache: torch.Tensor, v_cache: torch.Tensor, attn_metadata,
                 k_new: torch.Tensor, v_new: torch.Tensor,
                 k_scale: Optional[torch.Tensor] = None,
                 v_scale: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """kv_cache_kernels.py:230-279.  Returns (k_out, v_out): [sum(ctx + new), H_kv, hd] in
    the cache's dtype.  Unlike the reference kernel a context that fills its last page
    exactly is copied completely."""
    assert k_cache.shape == v_cache.shape
    assert k_new.shape == v_new.shape
    N_BLOCKS, PAGE_SIZE, H_KV, HEAD_DIM = k_cache.shape
    NUM_SEQS, MAX_SEQ_BLOCKS = attn_metadata.block_tables.shape
    ctxlens = attn_metadata.context_lens
    seqlens = attn_metadata.seq_lens_ts
    cu_seqlens_q = attn_metadata.cu_seqlens_q
    cu_seqlens_k = attn_metadata.cu_seqlens_k
    assert cu_seqlens_q.shape == cu_seqlens_k.shape
    assert cu_seqlens_q.shape[0] == NUM_SEQS + 1
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_new.stride(-1) == 1 and k_new.stride(1) == HEAD_DIM
    assert v_new.stride(-1) == 1 and v_new.stride(1) == HEAD_DIM
    for t in (ctxlens, seqlens, cu_seqlens_q, cu_seqlens_k, attn_metadata.block_tables):
        assert t.dtype == torch.int32 and t.is_cuda
    # one host read, as the reference's `.item()` (kv_cache_kernels.py:252)
    total = int(cu_seqlens_k[-1].item())
    seq_lens_host = getattr(attn_metadata, "seq_lens", None)
    if seq_lens_host is not None:
        assert sum(seq_lens_host) == k_new.shape[0]
    max_total = int(getattr(attn_metadata, "max_seqlen_k", 0) or 0)
    if max_total <= 0:
        max_total = int((ctxlens + seqlens).max().item()) if NUM_SEQS else 0
    ks, vs = _scales(k_cache, attn_metadata, k_scale, v_scale, H_KV)
    k_output = torch.empty((total, H_KV, HEAD_DIM), device=k_cache.device, dtype=k_cache.dtype)
    v_output = torch.empty_like(k_output)
    bt = attn_metadata.block_tables
    assert bt.stride(1) == 1
    _call(_lib.ops().kv_load, k_cache, v_cache, k_new, v_new, k_output, v_output, bt, ctxlens, seqlens,
          cu_seqlens_q, cu_seqlens_k, max_total, ks, vs)
    return k_output, v_output
