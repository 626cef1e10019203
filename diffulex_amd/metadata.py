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
