"""Shared helpers of the GPU parity tests."""
import torch

from diffulex_amd import PagedAttnMetaData
from diffulex_amd.workloads import Workload, MASK_BLOCK_CAUSAL
from oracle import attention as oat

ATOL_BF16 = 2e-2   # max-abs tolerance vs the fp32 oracle, bf16 KV
ATOL_FP8 = 6e-2    # max-abs tolerance vs the fp32 oracle, FP8 KV


def metadata_for(wl: Workload, decode_mode="static", is_prefill=False, attn_type="block_attention"):
    """Metadata as the reference's runners build it: static mode indexes the fresh K/V with
    cu_seqlens_k, varlen mode lets cu_seqlens_k span context + fresh rows."""
    return PagedAttnMetaData(
        is_prefill=is_prefill,
        cu_seqlens_q=wl.cu_seqlens_q,
        cu_seqlens_k=wl.cu_seqlens_q if decode_mode == "static" else wl.cu_seqlens_k,
        max_seqlen_q=wl.q_len, max_seqlen_k=int(wl.extra.get("max_seqlen_k", 0)),
        slot_mapping=wl.slot_mapping, context_lens=wl.context_lens, block_tables=wl.block_tables,
        page_block_size=wl.page_size, attn_type=attn_type, diffusion_block_size=wl.diffusion_block_size,
        decode_mode=decode_mode, seq_lens_ts=wl.seq_lens_new, k_scale=wl.k_scale, v_scale=wl.v_scale,
        decode_mask="block_causal" if wl.mask_mode == MASK_BLOCK_CAUSAL else "full")


def oracle_fp32(wl: Workload, seqs=None, **kw):
    """fp32 oracle on the CPU copy of a workload (optionally only for some sequences)."""
    c = wl.to("cpu")
    args = dict(q=c.q, k_new=c.k_new, v_new=c.v_new, k_cache=c.k_cache, v_cache=c.v_cache,
                block_tables=c.block_tables, context_lens=c.context_lens, cu_seqlens_q=c.cu_seqlens_q,
                cu_seqlens_new=c.cu_seqlens_q, scale=c.scale, mask_mode=c.mask_mode,
                dbs=c.diffusion_block_size, k_scale=c.k_scale, v_scale=c.v_scale)
    args.update(kw)
    if seqs is not None:
        cu = c.cu_seqlens_q.tolist()
        outs = []
        for s in seqs:
            a = dict(args)
            a["block_tables"] = args["block_tables"][s:s + 1]
            a["context_lens"] = args["context_lens"][s:s + 1] if args["context_lens"] is not None else None
            a["cu_seqlens_q"] = torch.tensor([cu[s], cu[s + 1]])
            a["cu_seqlens_new"] = torch.tensor([cu[s], cu[s + 1]])
            outs.append(oat.paged_attention_fp32(**a)[cu[s]:cu[s + 1]])
        return outs
    return oat.paged_attention_fp32(**args)


def max_abs_err(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.float().cpu() - b.float().cpu()).abs().max())
