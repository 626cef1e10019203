"""Attention metadata and the module-global fetch hook.

Mirrors diffulex/attention/metadata.py:7-45 (``AttnMetaDataBase``, the
``set_fetch_fn_for_attn_metadata`` / ``fetch_attn_metadata`` hook and the
warm-up flag) plus the fields the strategy subclasses add and the operators
read (diffulex/strategy/block_diffusion/attention/metadata.py:11-19,
diffulex/strategy/d2f/attention/metadata.py:11-26).  The operators are
duck-typed: any object with these attributes works.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional

import torch


@dataclass
class AttnMetaDataBase:
    is_prefill: bool = False
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_k: Optional[torch.Tensor] = None
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    slot_mapping: Optional[torch.Tensor] = None
    context_lens: Optional[torch.Tensor] = None
    block_tables: Optional[torch.Tensor] = None
    page_block_size: int = 32
    attn_type: str = "block_attention"
    diffusion_block_size: int = 32
    decode_mode: str = "static"

    @property
    def num_seqs(self) -> int:
        return len(self.cu_seqlens_q) - 1


@dataclass
class PagedAttnMetaData(AttnMetaDataBase):
    """The union of the block-diffusion and D2F metadata fields, plus the FP8
    scales and the decode mask selector this build adds."""
    seq_lens: Optional[List[int]] = None
    seq_lens_ts: Optional[torch.Tensor] = None
    seqs: Optional[list] = None
    kv_cache_layout: str = "unified"
    need_kv_cache_store: bool = True
    k_scale: Optional[torch.Tensor] = None   # fp32 [H_kv], FP8 caches only
    v_scale: Optional[torch.Tensor] = None
    decode_mask: str = "full"                # "full" | "block_causal"

    def __post_init__(self):
        if self.context_lens is not None:
            if self.seq_lens_ts is not None:
                self.total_lens = self.seq_lens_ts + self.context_lens
            else:
                self.total_lens = self.diffusion_block_size + self.context_lens


def build_decode_metadata(strategy: str, *, block_tables: torch.Tensor, block_state: torch.Tensor,
                          page_size: int, diffusion_block_size: int, num_tokens: Optional[torch.Tensor] = None,
                          num_pages: Optional[torch.Tensor] = None, prompt_len: Optional[torch.Tensor] = None,
                          num_diffusion_blocks: Optional[torch.Tensor] = None, token_capacity: int,
                          padded_seqs: int = 0, padded_tokens: int = 0, out: Optional[dict] = None,
                          kv_cache_layout: str = "unified", sync_summary: bool = False,
                          token_ids: Optional[torch.Tensor] = None) -> "PagedAttnMetaData":
    """The metadata of one decode step from per-sequence state kept on the device
    (``dfx_build_decode_metadata``): what ``prepare_decode`` of the reference's runners computes
    in Python loops and copies over (block_diffusion/engine/model_runner.py:114-173,
    d2f/engine/model_runner.py:137-262).

    ``strategy``: "block_diffusion" (``num_tokens`` [B] int32, ``block_state`` [B] uint8 = state of
    the last diffusion block, ``num_pages`` [B] int32) or "d2f" (``prompt_len`` [B],
    ``num_diffusion_blocks`` [B], ``block_state`` [B, max_blocks] uint8, ``num_tokens`` optional).
    ``out``: a dict of preallocated output tensors (``positions``, ``slot_mapping``,
    ``cu_seqlens_q``, ``cu_seqlens_k``, ``context_lens``, ``seq_lens``, ``summary``), e.g. the
    buffers a graph was captured on, padded to ``padded_seqs`` / ``padded_tokens``; by default new
    tensors are made.  Nothing is read back unless ``sync_summary`` is set: ``max_seqlen_q`` is then
    the true maximum, otherwise an upper bound from the shapes (enough for the attention operators).
    ``token_ids`` (int64 [B, max_len], the sequences' tokens kept on the device): the step's
    ``input_ids`` -- every fed token's id, the concatenation of ``cur_input_ids`` in the reference's
    loops -- are gathered in the same launch and attached as ``md.input_ids`` (``out["input_ids"]``
    if given).
    Returns the metadata object with ``positions`` and ``summary`` attached as attributes."""
    from . import _lib
    from .kv_cache_kernels import _call
    dev = block_tables.device
    B = block_tables.shape[0]
    rows = max(B, padded_seqs)
    cap = max(int(token_capacity), int(padded_tokens))
    i32 = dict(dtype=torch.int32, device=dev)
    o = dict(out) if out is not None else {}
    o.setdefault("positions", torch.empty(cap, dtype=torch.int64, device=dev))
    o.setdefault("slot_mapping", torch.empty(cap, **i32))
    o.setdefault("cu_seqlens_q", torch.empty(rows + 1, **i32))
    o.setdefault("cu_seqlens_k", torch.empty(rows + 1, **i32))
    o.setdefault("context_lens", torch.empty(rows, **i32))
    o.setdefault("seq_lens", torch.empty(rows, **i32))
    o.setdefault("summary", torch.empty(8, **i32))
    if token_ids is not None:
        o.setdefault("input_ids", torch.empty(cap, dtype=torch.int64, device=dev))
    code = {"block_diffusion": _lib.DFX_META_BLOCK_DIFFUSION, "d2f": _lib.DFX_META_D2F}[strategy]
    _call(_lib.ops().build_decode_metadata, code, block_tables, block_state, int(page_size), int(diffusion_block_size),
          num_tokens, num_pages, prompt_len, num_diffusion_blocks, o["positions"], o["slot_mapping"], o["cu_seqlens_q"],
          o["cu_seqlens_k"], o["context_lens"], o["seq_lens"], o["summary"], cap, int(padded_seqs), int(padded_tokens),
          token_ids, o["input_ids"] if token_ids is not None else None)
    d2f = strategy == "d2f"
    n_tokens = cap
    max_q = max_k = 0
    need_store = True
    if sync_summary:
        host = o["summary"].tolist()
        if host[5]:
            raise ValueError(f"token_capacity {cap} is too small for {max(host[0], host[1])} tokens")
        if host[6]:
            raise ValueError(f"sequence {host[6] - 1} is in a state the decode step cannot be prepared from")
        n_tokens, max_q, max_k, need_store = host[0], host[2], host[3], bool(host[4])
    elif not d2f:
        n_tokens, max_q, max_k = B * diffusion_block_size, diffusion_block_size, diffusion_block_size
    else:
        max_q = block_state.shape[-1] * diffusion_block_size if block_state.dim() == 2 else cap
    n_tokens = max(n_tokens, int(padded_tokens))
    md = PagedAttnMetaData(
        is_prefill=False, cu_seqlens_q=o["cu_seqlens_q"][:rows + 1], cu_seqlens_k=o["cu_seqlens_k"][:rows + 1],
        max_seqlen_q=max_q, max_seqlen_k=max_k, slot_mapping=o["slot_mapping"][:n_tokens],
        context_lens=o["context_lens"][:rows], block_tables=block_tables, page_block_size=int(page_size),
        attn_type="full_attention" if d2f else "block_attention", diffusion_block_size=int(diffusion_block_size),
        decode_mode="varlen" if d2f else "static", seq_lens_ts=o["seq_lens"][:rows] if d2f else None,
        kv_cache_layout=kv_cache_layout, need_kv_cache_store=need_store)
    md.positions = o["positions"][:n_tokens]
    md.input_ids = o["input_ids"][:n_tokens] if token_ids is not None else None
    md.summary = o["summary"]
    return md


FN_TYPE_AttnMetaDataFetch = Callable[[], AttnMetaDataBase]

fetch_attn_metadata: FN_TYPE_AttnMetaDataFetch = ...


def set_fetch_fn_for_attn_metadata(fn: FN_TYPE_AttnMetaDataFetch) -> None:
    global fetch_attn_metadata
    fetch_attn_metadata = fn


WARMING_UP = False


def set_warming_up(is_warming_up: bool) -> None:
    global WARMING_UP
    WARMING_UP = is_warming_up


def is_warming_up() -> bool:
    return WARMING_UP


def reset_warming_up() -> None:
    global WARMING_UP
    WARMING_UP = False
