"""Block-diffusion paged attention restated on the CPU.

Test infrastructure only (see ``oracle/__init__.py``).

Two routines:

* ``paged_attention_fp32``: the accuracy oracle.  Everything is upcast to
  fp32, the softmax is written out explicitly (no library attention call), so
  that it can be pinned *against* the library SDPA in the tests.
* ``paged_attention_sdpa``: the reference's own PyTorch path, i.e. what its
  kernel tests compare against, a per-sequence gather followed by
  ``F.scaled_dot_product_attention`` on the input dtype.  This is the routine
  timed as the CPU baseline.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

from . import fp8_e4m3

MASK_FULL = 0          # every fresh token visible (block-diffusion block / reference D2F)
MASK_BLOCK_CAUSAL = 1  # fresh token j visible to query i iff j < (i // DBS + 1) * DBS


def gather_context(cache, block_table_row, context_len, page_size):
    """Rows [0, context_len) of one sequence, page by page.

    Follows tests/python/kernel/test_dllm_flash_attn_decode_kernel.py:63-76:
    negative table entries are skipped, page p contributes
    ``min(p*page + page, ctx) - p*page`` rows while ``p*page < ctx``.
    """
    parts = []
    for p, page_id in enumerate(block_table_row.tolist()):
        if page_id < 0:
            continue
        start = p * page_size
        if start < context_len:
            n = min(start + page_size, context_len) - start
            parts.append(cache[page_id, :n])
    if parts:
        return torch.cat(parts, dim=0)
    return cache[:0].reshape(0, *cache.shape[2:])


def _dequant(rows, scale):
    """fp8 rows [n, H, hd] -> fp32 via decode(code) * scale[h]
    (diffulex_legacy/layers/attention/ops/prefix_prefill.py:126-129)."""
    codes = rows.view(torch.uint8).numpy()
    sc = scale.numpy() if isinstance(scale, torch.Tensor) else scale
    return torch.from_numpy(fp8_e4m3.dequantize_per_head(codes, sc))


def visible_mask(q_len, ctx, n_new, mask_mode, dbs):
    """Boolean [q_len, ctx + n_new]: which keys each query may attend to.

    The whole cached prefix is always visible
    (diffulex_kernel/python/dllm_flash_attn.py:259-298 masks only
    ``pos >= context_len``).  Fresh tokens: all of them in MASK_FULL (no mask
    inside the block: test_dllm_flash_attn_decode_kernel.py:93-101,
    ``is_causal=False``); in MASK_BLOCK_CAUSAL the prefill kernel's rule
    ``kv_j < (q_i // DBS + 1) * DBS`` (dllm_flash_attn.py:109-116, and the test
    mask tests/python/kernel/test_dllm_flash_attn_prefill_kernel.py:57-62).
    """
    m = torch.ones(q_len, ctx + n_new, dtype=torch.bool)
    if mask_mode == MASK_BLOCK_CAUSAL:
        i = torch.arange(q_len).unsqueeze(1)
        j = torch.arange(n_new).unsqueeze(0)
        m[:, ctx:] = j < (i // dbs + 1) * dbs
    return m


def paged_attention_fp32(q, k_new, v_new, k_cache, v_cache, block_tables, context_lens,
                         cu_seqlens_q, cu_seqlens_new, scale, mask_mode=MASK_FULL, dbs=32,
                         k_scale=None, v_scale=None):
    """fp32 oracle.  q: [T_q, H_q, hd]; k_new/v_new: [T_new, H_kv, hd];
    caches: [pages, page, H_kv, hd] (bf16, or fp8 with per-head scales) or None;
    cu_seqlens_new indexes the *fresh* K/V rows.  Returns fp32 [T_q, H_q, hd].

    Semantics: diffulex_kernel/python/dllm_flash_attn.py:163-347 as restated by
    its test oracle (test_dllm_flash_attn_decode_kernel.py:14-105), with the
    ``scale`` argument honoured (the TileLang kernel hard-codes 1/sqrt(hd),
    dllm_flash_attn.py:184) and GQA by ``kv_head = q_head // (H_q / H_kv)``.
    """
    t_q, h_q, hd = q.shape
    h_kv = k_new.shape[1]
    g = h_q // h_kv
    out = torch.zeros(t_q, h_q, hd, dtype=torch.float32)
    num_seqs = len(cu_seqlens_q) - 1
    page = k_cache.shape[1] if k_cache is not None else 0
    for s in range(num_seqs):
        q0, q1 = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        n0, n1 = int(cu_seqlens_new[s]), int(cu_seqlens_new[s + 1])
        ctx = int(context_lens[s]) if (context_lens is not None and k_cache is not None) else 0
        if q1 == q0:
            continue
        if ctx > 0:
            kc = gather_context(k_cache, block_tables[s], ctx, page)
            vc = gather_context(v_cache, block_tables[s], ctx, page)
            ctx = kc.shape[0]  # fewer than context_len if pages were skipped (negative table entries)
            if k_cache.element_size() == 1:
                kc, vc = _dequant(kc, k_scale), _dequant(vc, v_scale)
            kk = torch.cat([kc.float(), k_new[n0:n1].float()], 0)
            vv = torch.cat([vc.float(), v_new[n0:n1].float()], 0)
        else:
            kk, vv = k_new[n0:n1].float(), v_new[n0:n1].float()
        if kk.shape[0] == 0:
            # No key at all (every page of the context skipped, no fresh rows): the softmax is over
            # an empty set.  The reference's kernel divides 0 by 0 there; this build defines zeros.
            continue
        allowed = visible_mask(q1 - q0, ctx, n1 - n0, mask_mode, dbs)
        qq = q[q0:q1].float()
        for h in range(h_q):
            kv_h = h // g
            sc = (qq[:, h] @ kk[:, kv_h].T) * scale
            sc = sc.masked_fill(~allowed, float("-inf"))
            sc = sc - sc.max(dim=-1, keepdim=True).values
            p = torch.exp(sc)
            p = p / p.sum(dim=-1, keepdim=True)
            out[q0:q1, h] = p @ vv[:, kv_h]
    return out


def paged_attention_sdpa(q, k_new, v_new, k_cache, v_cache, block_tables, context_lens,
                         cu_seqlens_q, cu_seqlens_new, scale, mask_mode=MASK_FULL, dbs=32,
                         k_scale=None, v_scale=None, compute_dtype=None):
    """The reference's PyTorch path: per-sequence gather + library SDPA in the
    input dtype (test_dllm_flash_attn_decode_kernel.py:49-103), block mask as
    in test_dllm_flash_attn_prefill_kernel.py:57-75.  ``compute_dtype=float32``
    turns it into a second, library-based fp32 evaluation."""
    t_q, h_q, hd = q.shape
    out = torch.zeros_like(q if compute_dtype is None else q.to(compute_dtype))
    num_seqs = len(cu_seqlens_q) - 1
    page = k_cache.shape[1] if k_cache is not None else 0
    for s in range(num_seqs):
        q0, q1 = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        n0, n1 = int(cu_seqlens_new[s]), int(cu_seqlens_new[s + 1])
        ctx = int(context_lens[s]) if (context_lens is not None and k_cache is not None) else 0
        if q1 == q0:
            continue
        dt = q.dtype if compute_dtype is None else compute_dtype
        ks, vs = k_new[n0:n1].to(dt), v_new[n0:n1].to(dt)
        if ctx > 0:
            kc = gather_context(k_cache, block_tables[s], ctx, page)
            vc = gather_context(v_cache, block_tables[s], ctx, page)
            ctx = kc.shape[0]  # fewer than context_len if pages were skipped
            if k_cache.element_size() == 1:
                kc, vc = _dequant(kc, k_scale), _dequant(vc, v_scale)
            ks = torch.cat([kc.to(dt), ks], 0)
            vs = torch.cat([vc.to(dt), vs], 0)
        mask = None
        if mask_mode == MASK_BLOCK_CAUSAL:
            mask = visible_mask(q1 - q0, ctx, n1 - n0, mask_mode, dbs)
        o = F.scaled_dot_product_attention(
            q[q0:q1].to(dt).permute(1, 0, 2).unsqueeze(0),
            ks.permute(1, 0, 2).unsqueeze(0),
            vs.permute(1, 0, 2).unsqueeze(0),
            attn_mask=mask, dropout_p=0.0, is_causal=False, scale=scale, enable_gqa=True)
        out[q0:q1] = o[0].permute(1, 0, 2).to(out.dtype)
    return out


def algorithmic_bytes(context_lens, q_lens, new_lens, h_q, h_kv, hd, kv_elt_bytes):
    """Bytes one pass over the path must move: K+V prefix read once per KV head,
    Q read, O written, fresh K/V read (bf16)."""
    ctx = int(np.sum(np.asarray(context_lens, dtype=np.int64)))
    tq = int(np.sum(np.asarray(q_lens, dtype=np.int64)))
    tn = int(np.sum(np.asarray(new_lens, dtype=np.int64)))
    return ctx * h_kv * hd * 2 * kv_elt_bytes + 2 * tq * h_q * hd * 2 + tn * h_kv * hd * 2 * 2


def algorithmic_flops(context_lens, q_lens, new_lens, h_q, hd, mask_mode=MASK_FULL, dbs=32):
    """4 * H_q * hd * (number of visible (query, key) pairs)."""
    pairs = 0
    for c, ql, nl in zip(context_lens, q_lens, new_lens):
        c, ql, nl = int(c), int(ql), int(nl)
        if mask_mode == MASK_BLOCK_CAUSAL:
            vis = sum(min(nl, (i // dbs + 1) * dbs) for i in range(ql))
        else:
            vis = ql * nl
        pairs += ql * c + vis
    return 4 * h_q * hd * pairs
