"""Seeded synthetic inputs for the paged-attention / KV-cache operators.

The five named workloads are the configurations the headline metric and the
parity tests are defined on (C1 the small CPU-runnable case ... C5 the FP8 KV
case).  Inputs are drawn from a seeded generator: fp32 N(0,1) rounded to bf16,
prefix lengths uniform in a range, physical pages a random permutation dealt to
the sequences in order, block tables padded with -1.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

MASK_FULL = 0
MASK_BLOCK_CAUSAL = 1
E4M3_MAX = 448.0


@dataclass
class Workload:
    name: str
    num_seqs: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    page_size: int
    q_len: int                      # query (= fresh K/V) tokens per sequence
    diffusion_block_size: int
    mask_mode: int
    kv_fp8: bool
    scale: float
    q: torch.Tensor                 # [T, H_q, hd] bf16
    k_new: torch.Tensor             # [T, H_kv, hd] bf16
    v_new: torch.Tensor
    k_cache: torch.Tensor           # [pages, page, H_kv, hd] bf16 | float8_e4m3fn
    v_cache: torch.Tensor
    block_tables: torch.Tensor      # int32 [B, max_pages], -1 padded
    context_lens: torch.Tensor      # int32 [B]
    seq_lens_new: torch.Tensor      # int32 [B]
    cu_seqlens_q: torch.Tensor      # int32 [B+1]
    cu_seqlens_k: torch.Tensor      # int32 [B+1], spans context + fresh tokens
    slot_mapping: torch.Tensor      # int32 [T]: where the fresh tokens would be cached
    k_scale: Optional[torch.Tensor] = None   # fp32 [H_kv]
    v_scale: Optional[torch.Tensor] = None
    extra: dict = field(default_factory=dict)

    def to(self, device) -> "Workload":
        kw = {}
        for k, v in self.__dict__.items():
            kw[k] = v.to(device) if isinstance(v, torch.Tensor) else v
        return Workload(**kw)

    @property
    def total_q_tokens(self) -> int:
        return int(self.q.shape[0])


SPECS = {
    # name: (B, H_q, H_kv, hd, page, ctx_lo, ctx_hi, q_len, dbs, mask, fp8, seed)
    "c1": dict(num_seqs=2, h_q=4, h_kv=2, hd=64, page=16, ctx=[64, 100], q_len=32, dbs=32,
               mask=MASK_FULL, fp8=False, seed=0),
    "c2": dict(num_seqs=64, h_q=4, h_kv=4, hd=128, page=256, ctx=(256, 2048), q_len=32, dbs=32,
               mask=MASK_FULL, fp8=False, seed=1),
    "c3": dict(num_seqs=64, h_q=28, h_kv=4, hd=128, page=256, ctx=(512, 2048), q_len=32, dbs=32,
               mask=MASK_FULL, fp8=False, seed=2),
    "c4": dict(num_seqs=32, h_q=32, h_kv=32, hd=128, page=256, ctx=(1024, 4096), q_len=96, dbs=32,
               mask=MASK_BLOCK_CAUSAL, fp8=False, seed=3),
    "c5": dict(num_seqs=128, h_q=28, h_kv=4, hd=128, page=256, ctx=(2048, 8192), q_len=32, dbs=32,
               mask=MASK_FULL, fp8=True, seed=4),
}


def _randn_bf16(shape, gen, device):
    n = 1
    for s in shape:
        n *= int(s)
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    flat = out.view(-1)
    step = 1 << 24
    for i in range(0, n, step):
        m = min(step, n - i)
        flat[i:i + m] = torch.randn(m, generator=gen, dtype=torch.float32, device=device).to(torch.bfloat16)
    return out


def quantize_fp8_reference_cast(x_bf16: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """clamp(float32(x) / scale[h], +-448) cast with the library's RNE e4m3fn cast."""
    y = x_bf16.to(torch.float32) / scale.to(x_bf16.device).view(*([1] * (x_bf16.dim() - 2)), -1, 1)
    return y.clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)


def make_workload(name: str = "c3", *, device="cpu", seed: Optional[int] = None, **override) -> Workload:
    """Build one of the named workloads (``override`` replaces fields of its spec,
    e.g. ``num_seqs=8`` for a bounded slice of the same shape)."""
    spec = dict(SPECS[name])
    spec.update(override)
    seed = spec["seed"] if seed is None else seed
    cpu_gen = torch.Generator("cpu").manual_seed(seed)
    dev = torch.device(device)
    gen = cpu_gen if dev.type == "cpu" else torch.Generator(dev).manual_seed(seed)

    b, h_q, h_kv, hd = spec["num_seqs"], spec["h_q"], spec["h_kv"], spec["hd"]
    page, q_len, dbs = spec["page"], spec["q_len"], spec["dbs"]
    ctx = spec["ctx"]
    if isinstance(ctx, (list,)):
        assert len(ctx) == b
        context_lens = torch.tensor(ctx, dtype=torch.int64)
    else:
        context_lens = torch.randint(ctx[0], ctx[1] + 1, (b,), generator=cpu_gen)
    new_lens = torch.full((b,), q_len, dtype=torch.int64)

    pages_per_seq = (context_lens + new_lens + page - 1) // page
    n_pages = int(pages_per_seq.sum()) + 3  # a few pages that belong to no sequence
    max_pages = int(pages_per_seq.max()) + 1  # one padded column
    perm = torch.randperm(n_pages, generator=cpu_gen)
    block_tables = torch.full((b, max_pages), -1, dtype=torch.int32)
    cur = 0
    for s in range(b):
        n = int(pages_per_seq[s])
        block_tables[s, :n] = perm[cur:cur + n].to(torch.int32)
        cur += n

    t = b * q_len
    q = _randn_bf16((t, h_q, hd), gen, dev)
    k_new = _randn_bf16((t, h_kv, hd), gen, dev)
    v_new = _randn_bf16((t, h_kv, hd), gen, dev)
    k_src = _randn_bf16((n_pages, page, h_kv, hd), gen, dev)
    v_src = _randn_bf16((n_pages, page, h_kv, hd), gen, dev)
    k_scale = v_scale = None
    if spec["fp8"]:
        k_scale = (k_src.float().abs().amax(dim=(0, 1, 3)) / E4M3_MAX).to(torch.float32)
        v_scale = (v_src.float().abs().amax(dim=(0, 1, 3)) / E4M3_MAX).to(torch.float32)
        k_cache = quantize_fp8_reference_cast(k_src, k_scale)
        v_cache = quantize_fp8_reference_cast(v_src, v_scale)
    else:
        k_cache, v_cache = k_src, v_src
    del k_src, v_src

    cu_q = torch.zeros(b + 1, dtype=torch.int32)
    cu_q[1:] = torch.cumsum(new_lens, 0)
    cu_k = torch.zeros(b + 1, dtype=torch.int32)
    cu_k[1:] = torch.cumsum(context_lens + new_lens, 0)

    # slots right after each context, inside that sequence's own pages
    pos = context_lens.view(b, 1) + torch.arange(q_len).view(1, q_len)           # [B, q_len]
    page_ids = torch.gather(block_tables.to(torch.int64), 1, pos // page)
    slot_mapping = (page_ids * page + pos % page).reshape(-1).to(torch.int32)

    wl = Workload(
        name=name, num_seqs=b, num_q_heads=h_q, num_kv_heads=h_kv, head_dim=hd, page_size=page,
        q_len=q_len, diffusion_block_size=dbs, mask_mode=spec["mask"], kv_fp8=spec["fp8"],
        scale=float(hd) ** -0.5, q=q, k_new=k_new, v_new=v_new, k_cache=k_cache, v_cache=v_cache,
        block_tables=block_tables, context_lens=context_lens.to(torch.int32),
        seq_lens_new=new_lens.to(torch.int32), cu_seqlens_q=cu_q, cu_seqlens_k=cu_k,
        slot_mapping=slot_mapping, k_scale=k_scale, v_scale=v_scale,
    )
    return wl.to(dev) if dev.type != "cpu" else wl
