"""Block-diffusion attention operators (same names and arguments as
diffulex_kernel/python/dllm_flash_attn.py:539-637), backed by one gfx950 kernel.

Both decode modes of the reference run the same fused paged kernel here: it reads
the cached prefix through the block table and the fresh K/V from the operands, so
the "varlen" mode needs no ``load_kvcache`` gather and no second pass over K/V.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .kv_cache_kernels import _FP8_DTYPES, _stream

class _Workspace:
    __slots__ = ("tensor", "zeroed")

    def __init__(self, tensor):
        self.tensor = tensor
        self.zeroed = False  # an executed (not merely captured) fill has cleared the arrival counters


_workspaces = {}   # (device index, stream handle | "capture") -> _Workspace
_retired = []      # outgrown workspaces stay alive: graphs captured earlier still point at them


def _workspace(device: torch.device, stream: int, nbytes: int) -> torch.Tensor:
    """Scratch of ``dfx_paged_attn`` for this device and stream.  Eager calls use one workspace per
    stream; calls recorded into a graph share one per device (replays run on whatever stream is
    current then, so the capture stream means nothing), which every eager call keeps allocated and
    cleared at the size it needs itself: the usual warm-up-then-capture order records nothing extra.
    A capture that finds no cleared workspace records a fill of the counter area in front of the
    launch, and keeps doing so in every capture until an eager call has cleared it for real."""
    capturing = torch.cuda.is_current_stream_capturing()
    nbytes = max(int(nbytes), _lib.DFX_WORKSPACE_COUNTER_BYTES)

    def get(key):
        ws = _workspaces.get(key)
        if ws is None or ws.tensor.numel() < nbytes:
            if ws is not None:
                _retired.append(ws.tensor)
            ws = _Workspace(torch.empty(nbytes, dtype=torch.uint8, device=device))
            _workspaces[key] = ws
        if not ws.zeroed:
            ws.tensor[:_lib.DFX_WORKSPACE_COUNTER_BYTES].zero_()  # a fill kernel, never a memset node
            ws.zeroed = not capturing
        return ws

    if capturing:
        return get((device.index, "capture")).tensor
    get((device.index, "capture"))
    return get((device.index, stream)).tensor


_workspace_need = {}   # launch shape -> dfx_paged_attn_workspace_bytes


def paged_attention(q, k, v, k_cache, v_cache, scale, *, block_tables, context_lens, cu_seqlens_q,
                    cu_seqlens_new, max_seqlen_q, mask_mode=_lib.DFX_MASK_FULL, diffusion_block_size=32,
                    k_scale=None, v_scale=None, max_workgroups=0, out=None, flags=0,
                    store_slot_mapping=None, static_scratch=False, plan_cache=None,
                    cache_layout="unified", rope=None, k_rotated=None) -> torch.Tensor:
    """Launch ``dfx_paged_attn`` on the current stream through ``torch.ops.diffulex_amd.paged_attention``
    (which checks the tensors and fills ``dfx_attn_params``).  q: [T, H_q, hd]; k, v: [T_new, H_kv, hd];
    caches [pages, page, H_kv, hd] or None.  ``store_slot_mapping`` ([T_new] int32/int64): the same
    launch also writes the fresh rows into those cache slots (what
    ``store_kvcache_unified_layout`` does in a launch of its own); the slots must lie outside
    every attended context.  ``static_scratch``: launch through ``dfx_paged_attn_static``, which
    keeps its scratch in a static device array of the library instead of a workspace tensor (the C
    call then allocates nothing; pass ``out`` to keep this wrapper from allocating either).
    ``plan_cache`` (a dict): the launch plan (``dfx_paged_attn_plan``: partition of the batch over
    the workgroups, page address of every tile) is built on the first call and reused by later
    calls with the same dict -- the attention layers of one decoding step, whose lengths and block
    tables are the same.  In-place updates of those tensors and graph captures are noticed (they
    change the cache key); a caller that rewrites them behind PyTorch's back, or rewrites tensors made
    under ``torch.inference_mode()`` (which carry no version counter) in place, drops the dict.
    ``cache_layout="distinct"``: k_cache [pages, H_kv, hd / 8, page, 8], v_cache [pages, H_kv, hd,
    page] (what ``store_kvcache_distinct_layout`` writes); bf16, no fused store; head_dim 128 with pages of
    a multiple of 64 tokens streams (and takes a plan), other shapes take the generic tile path.
    ``rope=(cos_sin_cache, positions)``: q and k are the projections BEFORE the rotary embedding, which the
    launch applies itself (``dfx_attn_params.rope_cos_sin``): query rows on their way into the matrix
    instructions, fresh key rows into ``k_rotated`` (a new [T_new, H_kv, hd] tensor by default) and, with
    ``store_slot_mapping``, into the cache.  Raises ``DfxError`` (unsupported shape) where the pipelined
    kernels do not run; ``rope_supported()`` tells beforehand."""
    ops = _lib.ops()
    T, H_q, hd = q.shape
    H_kv = k.shape[1]
    num_seqs = cu_seqlens_q.numel() - 1
    if out is None:
        out = torch.empty((T, H_q, hd), dtype=q.dtype, device=q.device)
    has_cache = k_cache is not None and k_cache.numel() > 0
    assert cache_layout in ("unified", "distinct")
    distinct = cache_layout == "distinct"
    fp8 = has_cache and not distinct and k_cache.dtype in _FP8_DTYPES
    ks = vs = None
    if fp8:
        assert k_scale is not None and v_scale is not None, "an FP8 KV cache needs k_scale and v_scale"
        ks = k_scale.to(device=q.device, dtype=torch.float32).contiguous()
        vs = v_scale.to(device=q.device, dtype=torch.float32).contiguous()
    if not has_cache:
        k_cache = v_cache = block_tables = context_lens = None
    if store_slot_mapping is not None:
        assert store_slot_mapping.numel() == k.shape[0], \
            f"`N`: {k.shape[0]}, `slot_mapping.numel()`: {store_slot_mapping.numel()}"
    layout = _lib.DFX_CACHE_DISTINCT if distinct else _lib.DFX_CACHE_UNIFIED
    tail = (float(scale), int(max_seqlen_q), int(mask_mode), int(diffusion_block_size), int(max_workgroups),
            int(flags), layout)
    head = (q, k, v, k_cache, v_cache, out, block_tables, context_lens, cu_seqlens_q, cu_seqlens_new, ks, vs,
            store_slot_mapping)
    if rope is not None:
        table, positions = rope
        positions = positions.reshape(-1)
        if k_rotated is None:
            k_rotated = torch.empty((k.shape[0], H_kv, hd), dtype=k.dtype, device=k.device)
        tail = tail + (table, positions if positions.is_contiguous() else positions.contiguous(), k_rotated)
    else:
        tail = tail + (None, None, None)
    plan = None
    page_size = (k_cache.shape[3] if distinct else k_cache.shape[1]) if has_cache else 0
    if plan_cache is not None and has_cache:
        # A plan is only as good as the lengths and tables it was made from: see plan_key().
        key = plan_key(q, k, k_cache, fp8, tail, (block_tables, context_lens, cu_seqlens_q, cu_seqlens_new),
                       int(ops.stream_capture_id()), v_cache if distinct else None)
        plan = plan_cache.get(key, False)
        if plan is False:
            plan = plan_cache[key] = _build_plan(ops, head, tail, H_q // H_kv, int(max_seqlen_q), num_seqs,
                                                 block_tables.shape[1], page_size, k.shape[0])
    try:
        if static_scratch:
            ops.paged_attention(*head, plan, *tail, None, True)
            return out
        # (what dfx_paged_attn_workspace_bytes looks at: the shapes, the flags, whether k and v share
        # their head stride -- which decides the tile path -- and the device's compute-unit count)
        k_eff = k_rotated if rope is not None else k
        shape_key = (q.device.index, num_seqs, H_q, H_kv, hd, tail[1:7], has_cache, fp8, k_eff.stride(1) == v.stride(1),
                     page_size, distinct and (k_cache.stride()[2:], v_cache.stride()[2:]))
        need = _workspace_need.get(shape_key)
        if need is None:
            need = _workspace_need[shape_key] = int(ops.paged_attention_workspace_bytes(*head, None, *tail))
        ws = _workspace(q.device, _stream(), need)
        ops.paged_attention(*head, plan, *tail, ws, False)
    except RuntimeError as e:
        if "dfx_" in str(e):
            raise _lib.DfxError(str(e).split("\n")[0]) from None
        raise
    return out


def _content_token(t: torch.Tensor):
    """What tells two states of a metadata tensor apart, as far as PyTorch can tell: its address and
    its version counter, which every in-place update through PyTorch bumps.  Tensors created under
    ``torch.inference_mode()`` (the reference's runners build their metadata there:
    strategy/block_diffusion/engine/model_runner.py:206, strategy/d2f/engine/model_runner.py:291)
    track no version and reading it raises; for them the address alone stands, and the plan lives as
    long as the dict it is kept in -- the metadata object of one decoding step."""
    return (t.data_ptr(), -1 if t.is_inference() else t._version)


def plan_key(q, k, k_cache, fp8, tail, meta, capture_id, v_cache=None):
    """Cache key of a launch plan: everything ``dfx_paged_attn_plan`` depends on (shapes, strides, the
    metadata tensors and their contents as far as ``_content_token`` sees them) and the graph capture
    the call is recorded into (a plan built outside that capture is not part of its graph)."""
    k_eff = tail[9] if tail[7] is not None else k   # (with the rotary embedding in the launch the tiles come from k_rotated)
    # (v_cache: the distinct layout, whose two caches have strides of their own; its page size is a dimension)
    cache = k_cache.stride()[:3] if v_cache is None else (k_cache.stride(), v_cache.stride(), k_cache.shape[3])
    return (q.shape[1], k.shape[1], q.shape[2], bool(fp8), tail[1:7], k_eff.stride(0), k_eff.stride(1), cache,
            meta[2].numel() - 1, tuple(_content_token(t) for t in meta), int(capture_id))


# Launches whose units (an upper bound from the shapes) number fewer than this per workgroup are not planned.
PLAN_MIN_UNITS_PER_WORKGROUP = 2
_cu_count = {}


def _compute_units(device) -> int:
    n = _cu_count.get(device.index)
    if n is None:
        n = _cu_count[device.index] = torch.cuda.get_device_properties(device).multi_processor_count
    return n


def _build_plan(ops, head, tail, group, max_seqlen_q, num_seqs, max_pages, page_size, t_new):
    """Launch ``dfx_paged_attn_plan`` for this configuration; None where no plan applies (generic
    tile path).  The unit capacity is an upper bound from the shapes alone: no device data is read."""
    row_tiles = -(-group * max_seqlen_q // 128)
    tiles = num_seqs * (-(-max_pages * page_size // 64) + 1) + t_new // 64
    h_kv = head[1].shape[1]
    # (a launch of at most a tile or two per compute unit has nothing to plan: the plan kernels would cost
    # it more than they save -- 2 sequences x 2 KV heads of 3 tiles: 15.2 us with a plan, 12.4 without)
    n_wg = tail[4] if tail[4] > 0 else _compute_units(head[0].device)   # (max_workgroups, or a workgroup per compute unit)
    if h_kv * row_tiles * tiles < PLAN_MIN_UNITS_PER_WORKGROUP * n_wg:
        return None
    nbytes = int(ops.paged_attention_plan_bytes(*head, None, *tail, h_kv * row_tiles * tiles))
    if nbytes < 0:
        return None
    plan = torch.empty(nbytes, dtype=torch.uint8, device=head[0].device)
    ops.paged_attention_plan(*head, None, *tail, plan)
    return plan


def _plan_cache_of(attn_metadata):
    """The per-step plan cache, kept on the metadata object: the reference's runners build a new
    metadata object for every step (strategy/*/attention/metadata.py setters), so the plan is
    rebuilt exactly when lengths and block tables change.  Objects that cannot take the attribute
    simply get no plan."""
    cache = getattr(attn_metadata, "dfx_plan_cache", None)
    if cache is None:
        cache = {}
        try:
            attn_metadata.dfx_plan_cache = cache
        except (AttributeError, TypeError):
            return None
    return cache


def _max_seqlen_q(attn_metadata, cu_seqlens_q) -> int:
    m = int(getattr(attn_metadata, "max_seqlen_q", 0) or 0)
    if m <= 0:  # not supplied: one host read
        m = int((cu_seqlens_q[1:] - cu_seqlens_q[:-1]).max().item())
    return m


def dllm_flash_attn_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                            attn_metadata) -> torch.Tensor:
    """dllm_flash_attn.py:539-596: varlen self-attention of each sequence; every key visible
    for ``attn_type == "full_attention"``, the block-causal mask
    ``kv_j < (q_i // DBS + 1) * DBS`` for ``"block_attention"`` (dllm_flash_attn.py:109-116)."""
    if attn_metadata.attn_type == "full_attention":
        mask = _lib.DFX_MASK_FULL
    elif attn_metadata.attn_type == "block_attention":
        mask = _lib.DFX_MASK_BLOCK_CAUSAL
    else:
        raise ValueError(f"unknown attn_type {attn_metadata.attn_type!r}")
    return paged_attention(
        q, k, v, None, None, scale, block_tables=None, context_lens=None,
        cu_seqlens_q=attn_metadata.cu_seqlens_q, cu_seqlens_new=attn_metadata.cu_seqlens_k,
        max_seqlen_q=_max_seqlen_q(attn_metadata, attn_metadata.cu_seqlens_q), mask_mode=mask,
        diffusion_block_size=attn_metadata.diffusion_block_size)


def dllm_flash_attn_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, scale: float, attn_metadata,
                           k_scale: Optional[torch.Tensor] = None,
                           v_scale: Optional[torch.Tensor] = None,
                           store_slot_mapping: Optional[torch.Tensor] = None,
                           kv_cache_layout: str = "unified", rope=None) -> torch.Tensor:
    """dllm_flash_attn.py:599-637.  ``store_slot_mapping`` (extension): also store the fresh
    K/V rows into these cache slots in the same launch (see ``paged_attention``).
    ``kv_cache_layout="distinct"`` (extension): the caches are in the layout
    ``store_kvcache_distinct_layout`` writes.  ``rope=(cos_sin_cache, positions)`` (extension): q and k
    are the projections before the rotary embedding, which the launch applies (see ``paged_attention``).

    ``decode_mode == "static"``: ``cu_seqlens_k`` indexes the fresh K/V rows
    (strategy/block_diffusion/engine/model_runner.py:134-139).
    ``decode_mode == "varlen"``: ``cu_seqlens_k`` spans context + fresh rows and the
    fresh rows are addressed through ``cu_seqlens_q``
    (strategy/d2f/engine/model_runner.py:161-167, kv_cache_kernels.py:186-227).
    ``scale`` is honoured in both modes.  ``attn_metadata.decode_mask ==
    "block_causal"`` (optional attribute) selects the block-causal mask among the
    in-flight blocks; the default is the reference's behaviour, all fresh tokens visible.
    """
    if attn_metadata.decode_mode == "static":
        cu_new = attn_metadata.cu_seqlens_k
    elif attn_metadata.decode_mode == "varlen":
        cu_new = attn_metadata.cu_seqlens_q
    else:
        raise ValueError(f"unknown decode_mode {attn_metadata.decode_mode!r}")
    mask = _lib.DFX_MASK_FULL
    if getattr(attn_metadata, "decode_mask", "full") == "block_causal":
        mask = _lib.DFX_MASK_BLOCK_CAUSAL
    if kv_cache_layout == "distinct":
        return paged_attention(
            q, k, v, k_cache, v_cache, scale, block_tables=attn_metadata.block_tables,
            context_lens=attn_metadata.context_lens, cu_seqlens_q=attn_metadata.cu_seqlens_q,
            cu_seqlens_new=cu_new, max_seqlen_q=_max_seqlen_q(attn_metadata, attn_metadata.cu_seqlens_q),
            mask_mode=mask, diffusion_block_size=attn_metadata.diffusion_block_size, cache_layout="distinct",
            plan_cache=_plan_cache_of(attn_metadata))
    if k_cache.dtype in _FP8_DTYPES:
        k_scale = k_scale if k_scale is not None else getattr(attn_metadata, "k_scale", None)
        v_scale = v_scale if v_scale is not None else getattr(attn_metadata, "v_scale", None)
    return paged_attention(
        q, k, v, k_cache, v_cache, scale, block_tables=attn_metadata.block_tables,
        context_lens=attn_metadata.context_lens, cu_seqlens_q=attn_metadata.cu_seqlens_q,
        cu_seqlens_new=cu_new, max_seqlen_q=_max_seqlen_q(attn_metadata, attn_metadata.cu_seqlens_q),
        mask_mode=mask, diffusion_block_size=attn_metadata.diffusion_block_size,
        k_scale=k_scale, v_scale=v_scale, store_slot_mapping=store_slot_mapping,
        plan_cache=_plan_cache_of(attn_metadata), rope=rope)


def rope_supported(num_heads: int, num_kv_heads: int, head_dim: int, max_seqlen_q: int, page_size: int, num_seqs: int,
                   device=None) -> bool:
    """Whether ``dfx_paged_attn`` can apply the rotary embedding itself for this shape (the
    software-pipelined kernels: head_dim 128, page size a multiple of 16, more than 64 query rows per KV
    head and sequence or at most two (sequence, KV head) items per compute unit)."""
    if head_dim != 128 or page_size % 16 != 0 or num_heads % num_kv_heads != 0:
        return False
    rows = num_heads // num_kv_heads * max_seqlen_q
    cus = torch.cuda.get_device_properties(device if device is not None else torch.cuda.current_device()).multi_processor_count
    return rows > 64 or num_seqs * num_kv_heads <= 2 * cus
