"""Paged KV-cache store / load operators (same names, arguments and assertions as
diffulex_kernel/python/kv_cache_kernels.py), backed by the gfx950 kernels.

An FP8 cache is recognised by its dtype (``torch.float8_e4m3fn``, or ``uint8``
holding the codes); its per-KV-head scales come from the ``k_scale`` /
``v_scale`` keyword arguments or, if absent, from attributes of the same names
on ``attn_metadata``.
"""
from __future__ import annotations

from typing import Optional, Tuple

import ctypes as C
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
    """(kv_dtype, k_scale_ptr, v_scale_ptr, keepalive)."""
    if cache.dtype not in _FP8_DTYPES:
        assert cache.element_size() == 2, f"unsupported cache dtype {cache.dtype}"
        return _lib.DFX_KV_BF16, None, None, ()
    ks = k_scale if k_scale is not None else getattr(attn_metadata, "k_scale", None)
    vs = v_scale if v_scale is not None else getattr(attn_metadata, "v_scale", None)
    assert ks is not None and vs is not None, "an FP8 KV cache needs k_scale and v_scale"
    ks = ks.to(device=cache.device, dtype=torch.float32).contiguous()
    vs = vs.to(device=cache.device, dtype=torch.float32).contiguous()
    assert ks.numel() == n_heads and vs.numel() == n_heads
    return _lib.DFX_KV_FP8_E4M3, ks.data_ptr(), vs.data_ptr(), (ks, vs)


def store_kvcache_unified_layout(key: torch.Tensor, value: torch.Tensor,
                                 k_cache: torch.Tensor, v_cache: torch.Tensor,
                                 slot_mapping: torch.Tensor, attn_metadata,
                                 k_scale: Optional[torch.Tensor] = None,
                                 v_scale: Optional[torch.Tensor] = None) -> None:
    """kv_cache_kernels.py:110-124.  key/value: [N, H_kv, hd]; caches: [pages, page, H_kv, hd]."""
    lib = _lib.load()
    N, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == D and v_cache.stride(1) == D
    assert N == slot_mapping.numel(), f"`N`: {N}, `slot_mapping.numel()`: {slot_mapping.numel()}"
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert key.is_cuda and k_cache.is_cuda and slot_mapping.is_cuda
    assert key.element_size() == 2 and value.element_size() == 2
    kv_dtype, ksp, vsp, keep = _scales(k_cache, attn_metadata, k_scale, v_scale, num_heads)
    slots = slot_mapping.reshape(-1)
    if not slots.is_contiguous():
        slots = slots.contiguous()
    n_slots = k_cache.shape[0] * k_cache.shape[1]
    rc = lib.dfx_kv_store_unified(key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0),
                                  k_cache.data_ptr(), v_cache.data_ptr(), slots.data_ptr(), _index_type(slots),
                                  N, n_slots, num_heads, head_dim, kv_dtype, ksp, vsp, _stream())
    _lib.check(rc, "dfx_kv_store_unified")


def store_kvcache_distinct_layout(key: torch.Tensor, value: torch.Tensor,
                                  k_cache: torch.Tensor, v_cache: torch.Tensor,
                                  slot_mapping: torch.Tensor, attn_metadata) -> None:
    """kv_cache_kernels.py:86-107.  k_cache: [pages, H, hd // x, page, x]; v_cache: [pages, H, hd, page]."""
    lib = _lib.load()
    NBlks, NHeads, HDim_x, Blk_sz, x = k_cache.shape
    HDim = HDim_x * x
    N = key.shape[0]
    assert HDim == key.shape[-1] and NHeads == key.shape[1]
    assert N == slot_mapping.numel()
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == HDim and value.stride(1) == HDim
    assert key.element_size() == 2 and k_cache.element_size() == 2 and v_cache.element_size() == 2
    kcs = (C.c_int64 * 5)(*k_cache.stride())
    vcs = (C.c_int64 * 4)(*v_cache.stride())
    slots = slot_mapping.reshape(-1)
    if not slots.is_contiguous():
        slots = slots.contiguous()
    rc = lib.dfx_kv_store_distinct(key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0),
                                   k_cache.data_ptr(), v_cache.data_ptr(), kcs, vcs, slots.data_ptr(),
                                   _index_type(slots), N, NBlks, Blk_sz, x, NHeads, HDim, _stream())
    _lib.check(rc, "dfx_kv_store_distinct")


def load_kvcache(k_cache: torch.Tensor, v_cache: torch.Tensor, attn_metadata,
                 k_new: torch.Tensor, v_new: torch.Tensor,
                 k_scale: Optional[torch.Tensor] = None,
                 v_scale: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """kv_cache_kernels.py:230-279.  Returns (k_out, v_out): [sum(ctx + new), H_kv, hd] in
    the cache's dtype.  Unlike the reference kernel a context that fills its last page
    exactly is copied completely."""
    lib = _lib.load()
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
    kv_dtype, ksp, vsp, keep = _scales(k_cache, attn_metadata, k_scale, v_scale, H_KV)
    k_output = torch.empty((total, H_KV, HEAD_DIM), device=k_cache.device, dtype=k_cache.dtype)
    v_output = torch.empty_like(k_output)
    bt = attn_metadata.block_tables
    assert bt.stride(1) == 1
    # an empty tensor has a null data pointer; no fresh row is read then, any valid pointer serves
    kn_ptr = k_new.data_ptr() if k_new.numel() else k_cache.data_ptr()
    vn_ptr = v_new.data_ptr() if v_new.numel() else v_cache.data_ptr()
    rc = lib.dfx_kv_load(k_cache.data_ptr(), v_cache.data_ptr(), kn_ptr, vn_ptr,
                         k_new.stride(0), v_new.stride(0), k_output.data_ptr(), v_output.data_ptr(),
                         bt.data_ptr(), bt.stride(0), ctxlens.data_ptr(), seqlens.data_ptr(),
                         cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), NUM_SEQS, MAX_SEQ_BLOCKS,
                         N_BLOCKS, PAGE_SIZE, H_KV, HEAD_DIM, max_total, kv_dtype, ksp, vsp, _stream())
    _lib.check(rc, "dfx_kv_load")
    return k_output, v_output
