"""Paged KV-cache store / load restated on the CPU with numpy index arithmetic.

Test infrastructure only (see ``oracle/__init__.py``).  All copies are done on
the raw bit patterns, so "equal" below always means bit-exact.

Tensors are CPU ``torch`` tensors (numpy has no bf16); they are viewed as
unsigned integers of the same width and indexed with numpy.
"""
from __future__ import annotations

import numpy as np
import torch

from . import fp8_e4m3


def bits(t: torch.Tensor) -> np.ndarray:
    """Writable numpy view of a CPU tensor's raw bits (uint8 / uint16 / uint32)."""
    assert t.device.type == "cpu"
    width = t.element_size()
    view_dtype = {1: torch.uint8, 2: torch.int16, 4: torch.int32}[width]
    np_dtype = {1: np.uint8, 2: np.uint16, 4: np.uint32}[width]
    return t.view(view_dtype).numpy().view(np_dtype)


def _f32(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.float32).numpy()


def store_unified(key, value, k_cache, v_cache, slot_mapping, k_scale=None, v_scale=None) -> None:
    """In-place scatter of new K/V rows into the unified-layout cache.

    Follows diffulex_kernel/python/kv_cache_kernels.py:11-32 (kernel) and
    :110-124 (wrapper): with D = H_kv*hd and the caches seen as [slots, D],
    ``cache[slot] = key[t]`` for every token t whose slot is >= 0.

    key/value: [N, H_kv, hd]; caches: [pages, page, H_kv, hd]; slot_mapping: [N].
    With ``k_scale``/``v_scale`` (fp32 [H_kv]) and a 1-byte cache the rows are
    quantised to e4m3fn (``fp8_e4m3.quantize_per_head``) instead of copied.
    """
    n, h, hd = key.shape
    d = h * hd
    slots = np.asarray(slot_mapping.numpy() if isinstance(slot_mapping, torch.Tensor) else slot_mapping)
    slots = slots.reshape(-1).astype(np.int64)
    assert slots.shape[0] == n
    keep = np.nonzero(slots >= 0)[0]
    for src, cache, scale in ((key, k_cache, k_scale), (value, v_cache, v_scale)):
        cb = bits(cache).reshape(-1, d)
        if cache.element_size() == 1:
            assert scale is not None
            sc = scale.numpy() if isinstance(scale, torch.Tensor) else scale
            rows = fp8_e4m3.quantize_per_head(_f32(src), sc).reshape(n, d)
        else:
            assert cache.element_size() == src.element_size()
            rows = bits(src.contiguous()).reshape(n, d)
        cb[slots[keep]] = rows[keep]


def store_distinct(key, value, k_cache, v_cache, slot_mapping) -> None:
    """In-place scatter into the vLLM-style "distinct" layout.

    Follows diffulex_kernel/python/kv_cache_kernels.py:35-83,86-107:
    k_cache: [pages, H, hd/x, page, x], v_cache: [pages, H, hd, page];
    element (h, d) of token t with slot s goes to
    ``k_cache[s // page, h, d // x, s % page, d % x]`` and
    ``v_cache[s // page, h, d, s % page]``.
    """
    n, h, hd = key.shape
    _, hh, hd_x, page, x = k_cache.shape
    assert hh == h and hd_x * x == hd
    slots = slot_mapping.numpy().reshape(-1).astype(np.int64)
    keep = np.nonzero(slots >= 0)[0]
    blk = slots[keep] // page
    off = slots[keep] % page
    kb = bits(k_cache)
    vb = bits(v_cache)
    krows = bits(key.contiguous())[keep]  # [n', H, hd]
    vrows = bits(value.contiguous())[keep]
    # k: [n', H, hd/x, x] -> cache[blk, :, :, off, :]
    kb[blk, :, :, off, :] = krows.reshape(len(keep), h, hd_x, x)
    vb[blk, :, :, off] = vrows


def load(k_cache, v_cache, block_tables, context_lens, seq_lens_new, cu_seqlens_q, cu_seqlens_k,
         k_new, v_new, k_scale=None, v_scale=None):
    """Gather each sequence's cached context and append its fresh K/V.

    Follows the *checker* semantics of the reference, CHECK_LOADING
    (diffulex_legacy/layers/attention/ops/kv_cache_kernels.py:365-394) and the
    gather of its decode test oracle
    (tests/python/kernel/test_dllm_flash_attn_decode_kernel.py:63-87): page p
    of sequence s contributes ``min(page, ctx_s - p*page)`` rows.  (The Triton
    kernel, diffulex_kernel/python/kv_cache_kernels.py:165-168, drops a full
    last page when ``ctx % page == 0``; that is a defect, not the semantics.)

    Output row layout follows kv_cache_kernels.py:186-227: sequence s occupies
    ``[cu_seqlens_k[s], cu_seqlens_k[s+1])``, context first, then the
    ``seq_lens_new[s]`` fresh rows taken from ``k_new[cu_seqlens_q[s] : ...]``.
    Returns (k_out, v_out): [cu_seqlens_k[-1], H_kv, hd] in the cache's dtype.
    """
    pages, page, h, hd = k_cache.shape
    bt = np.asarray(block_tables.numpy(), dtype=np.int64)
    ctx = np.asarray(context_lens.numpy(), dtype=np.int64)
    new = np.asarray(seq_lens_new.numpy(), dtype=np.int64)
    cu_q = np.asarray(cu_seqlens_q.numpy(), dtype=np.int64)
    cu_k = np.asarray(cu_seqlens_k.numpy(), dtype=np.int64)
    total = int(cu_k[-1])
    outs = []
    for cache, fresh, scale in ((k_cache, k_new, k_scale), (v_cache, v_new, v_scale)):
        out = torch.zeros((total, h, hd), dtype=cache.dtype)
        ob = bits(out)
        cb = bits(cache)
        if cache.element_size() == 1 and fresh.element_size() != 1:
            sc = scale.numpy() if isinstance(scale, torch.Tensor) else scale
            fb = fp8_e4m3.quantize_per_head(_f32(fresh), sc)
        else:
            fb = bits(fresh.contiguous())
        for s in range(bt.shape[0]):
            o = int(cu_k[s])
            c = int(ctx[s])
            assert int(cu_k[s + 1]) - o == c + int(new[s])
            for p in range(-(-c // page)):
                m = min(page, c - p * page)
                ob[o + p * page: o + p * page + m] = cb[bt[s, p], :m]
            qs = int(cu_q[s])
            ob[o + c: o + c + int(new[s])] = fb[qs: qs + int(new[s])]
        outs.append(out)
    return outs[0], outs[1]
