"""Caches larger than 4 GiB: the pages a launch touches lie beyond byte offset 2^32 of the cache
tensor (a 288 GB device holds KV caches of many GiB per layer).  Each case runs the same small
workload twice through the C ABI -- on its own compact cache and on a big, otherwise
uninitialised cache whose last pages hold the same contents -- and compares bits; the compact run
is checked against the oracle elsewhere."""
import pytest
import torch

import diffulex_amd as dfx
from diffulex_amd import _lib
from diffulex_amd.rotary_embedding import RotaryEmbedding
from diffulex_amd.workloads import make_workload
from util import ATOL_BF16, ATOL_FP8, metadata_for, oracle_fp32, max_abs_err

pytestmark = pytest.mark.gpu
GIB = 1 << 30


def _bits(t):
    return t.view({1: torch.uint8, 2: torch.int16}[t.element_size()])


def _big_like(cache, min_bytes=int(4.25 * GIB)):
    """(big cache, index of the first page that mirrors `cache`): all mirrored pages start beyond 4 GiB."""
    page_bytes = cache[0].numel() * cache.element_size()
    base = -(-min_bytes // page_bytes)
    big = torch.empty((base + cache.shape[0],) + tuple(cache.shape[1:]), dtype=cache.dtype, device=cache.device)
    big[base:] = cache
    assert base * page_bytes > 4 * GIB
    return big, base


def _attn(g, k_cache, v_cache, block_tables, flags):
    out = dfx.paged_attention(g.q, g.k_new, g.v_new, k_cache, v_cache, g.scale, block_tables=block_tables,
                              context_lens=g.context_lens, cu_seqlens_q=g.cu_seqlens_q,
                              cu_seqlens_new=g.cu_seqlens_q, max_seqlen_q=g.q_len, mask_mode=g.mask_mode,
                              diffusion_block_size=g.diffusion_block_size, k_scale=g.k_scale, v_scale=g.v_scale,
                              flags=flags)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("name,over,flags,tol", [
    ("c3", dict(num_seqs=5, ctx=(300, 1500)), 0, ATOL_BF16),
    ("c3", dict(num_seqs=3, ctx=(100, 700)), _lib.DFX_ATTN_GENERIC_PATH, ATOL_BF16),
    ("c5", dict(num_seqs=4, ctx=(500, 2500)), 0, ATOL_FP8),
    ("c4", dict(num_seqs=3, ctx=(200, 900)), 0, ATOL_BF16),
])
def test_attention_reads_pages_beyond_4_gib(dev, name, over, flags, tol):
    wl = make_workload(name, seed=5, **over)
    g = wl.to(dev)
    small = _attn(g, g.k_cache, g.v_cache, g.block_tables, flags)
    assert max_abs_err(small[:g.q_len], oracle_fp32(wl, seqs=[0])[0]) <= tol
    big_k, base = _big_like(g.k_cache)
    big_v, _ = _big_like(g.v_cache)
    bt = torch.where(g.block_tables >= 0, g.block_tables + base, g.block_tables)
    big = _attn(g, big_k, big_v, bt, flags)
    assert torch.equal(_bits(big), _bits(small))


@pytest.mark.parametrize("name", ["c2", "c5"])
def test_store_and_load_beyond_4_gib(dev, name):
    wl = make_workload(name, num_seqs=6, ctx=(100, 900), seed=8)
    g = wl.to(dev)
    md = metadata_for(g, decode_mode="varlen")
    page = g.k_cache.shape[1]
    # compact run
    kc, vc = g.k_cache.clone(), g.v_cache.clone()
    dfx.store_kvcache_unified_layout(g.k_new, g.v_new, kc, vc, g.slot_mapping, md)
    k_small, v_small = dfx.load_kvcache(kc, vc, md, g.k_new, g.v_new)
    # same pages at the end of a > 4 GiB cache, slots as int64
    big_k, base = _big_like(g.k_cache)
    big_v, _ = _big_like(g.v_cache)
    slots = torch.where(g.slot_mapping >= 0, g.slot_mapping.long() + base * page, g.slot_mapping.long())
    dfx.store_kvcache_unified_layout(g.k_new, g.v_new, big_k, big_v, slots, md)
    md_big = metadata_for(g, decode_mode="varlen")
    md_big.block_tables = torch.where(g.block_tables >= 0, g.block_tables + base, g.block_tables)
    k_big, v_big = dfx.load_kvcache(big_k, big_v, md_big, g.k_new, g.v_new)
    torch.cuda.synchronize()
    assert torch.equal(_bits(big_k[base:]), _bits(kc)) and torch.equal(_bits(big_v[base:]), _bits(vc))
    assert torch.equal(_bits(k_big), _bits(k_small)) and torch.equal(_bits(v_big), _bits(v_small))


def test_rotary_store_beyond_4_gib(dev):
    T, hq, hkv, hd, page = 96, 28, 4, 128, 256
    gen = torch.Generator().manual_seed(3)
    qkv = torch.randn(T, (hq + 2 * hkv) * hd, generator=gen).to(torch.bfloat16).to(dev)
    pos = torch.randint(0, 4096, (T,), generator=gen).to(dev)
    q, k, v = qkv[:, :hq * hd], qkv[:, hq * hd:(hq + hkv) * hd], qkv[:, (hq + hkv) * hd:]
    rope = RotaryEmbedding(hd, hd, 4096, 1.0e6).to(dev)
    small = torch.zeros(2, page, hkv, hd, dtype=torch.bfloat16, device=dev)
    kc, vc = small.clone(), small.clone()
    slots = torch.randperm(2 * page, generator=gen)[:T].to(dev)
    q1, k1 = rope.forward_and_store(pos, q, k, v, kc, vc, slots)
    big_k, base = _big_like(small)
    big_v, _ = _big_like(small)
    q2, k2 = rope.forward_and_store(pos, q, k, v, big_k, big_v, slots + base * page)
    torch.cuda.synchronize()
    assert torch.equal(_bits(q1), _bits(q2)) and torch.equal(_bits(k1), _bits(k2))
    assert torch.equal(_bits(big_k[base:]), _bits(kc)) and torch.equal(_bits(big_v[base:]), _bits(vc))
