"""GPU parity of the KV-cache store / load kernels against the CPU oracle: bit-exact."""
import json
import os

import numpy as np
import pytest
import torch

import diffulex_amd as dfx
from diffulex_amd.workloads import make_workload
from oracle import kv_cache as okv
from util import metadata_for

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _bits(t):
    t = t.cpu()
    return t.view({1: torch.uint8, 2: torch.int16}[t.element_size()])


def _sentinel_like(t):
    n = t.numel()
    pat = (torch.arange(n, dtype=torch.int32) % 251 + 3).to(torch.uint8 if t.element_size() == 1 else torch.int16)
    return pat.view(t.dtype).reshape(t.shape).clone()


@pytest.mark.parametrize("name,over", [
    ("c1", {}), ("c2", {}), ("c2", dict(num_seqs=3, hd=64, h_kv=2, h_q=2, page=32, ctx=[0, 32, 95])),
    ("c5", dict(num_seqs=6, ctx=(100, 700))), ("c5", dict(num_seqs=4, ctx=(50, 300), hd=64, page=16)),
])
@pytest.mark.parametrize("slot_dtype", [torch.int32, torch.int64])
def test_store_unified_bit_exact(dev, name, over, slot_dtype):
    wl = make_workload(name, **over)
    slots = wl.slot_mapping.clone()
    slots[::5] = -1                              # skipped tokens
    kc0, vc0 = _sentinel_like(wl.k_cache), _sentinel_like(wl.v_cache)
    want_k, want_v = kc0.clone(), vc0.clone()
    okv.store_unified(wl.k_new, wl.v_new, want_k, want_v, slots, wl.k_scale, wl.v_scale)
    g = wl.to(dev)
    kc, vc = kc0.to(dev), vc0.to(dev)
    dfx.store_kvcache_unified_layout(g.k_new, g.v_new, kc, vc, slots.to(dev).to(slot_dtype), metadata_for(g))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc), _bits(want_k))
    assert torch.equal(_bits(vc), _bits(want_v))


def test_store_unified_strided_rows_and_scalar_fallback(dev):
    g = torch.Generator().manual_seed(21)
    n, h, hd = 37, 3, 12                        # hd % 8 != 0: element-wise kernel
    wide = torch.randn(n, 2 * h * hd + 4, generator=g).to(torch.bfloat16)
    key = wide[:, :h * hd].view(n, h, hd)       # row stride larger than H*hd
    value = wide[:, h * hd:2 * h * hd].view(n, h, hd)
    slots = torch.randperm(64, generator=g)[:n].to(torch.int32)
    slots[3] = -1
    kc0 = _sentinel_like(torch.empty(4, 16, h, hd, dtype=torch.bfloat16))
    want_k, want_v = kc0.clone(), kc0.clone()
    okv.store_unified(key, value, want_k, want_v, slots)
    kc, vc = kc0.to(dev), kc0.to(dev)
    wd = wide.to(dev)
    dfx.store_kvcache_unified_layout(wd[:, :h * hd].view(n, h, hd), wd[:, h * hd:2 * h * hd].view(n, h, hd), kc, vc,
                                     slots.to(dev), None)
    assert torch.equal(_bits(kc), _bits(want_k)) and torch.equal(_bits(vc), _bits(want_v))


def test_store_asserts_like_the_reference(dev):
    wl = make_workload("c1").to(dev)
    md = metadata_for(wl)
    with pytest.raises(AssertionError):
        dfx.store_kvcache_unified_layout(wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.slot_mapping[:-1], md)
    with pytest.raises(AssertionError):
        dfx.store_kvcache_unified_layout(wl.k_new.transpose(1, 2), wl.v_new.transpose(1, 2), wl.k_cache, wl.v_cache,
                                         wl.slot_mapping, md)


def test_store_captured_slot_mapping_fixture(dev):
    fx = json.load(open(os.path.join(HERE, "golden", "mimic_slot_mapping.json")))
    slots = torch.full((fx["length"],), -1, dtype=torch.int64)
    slots[fx["run_offset"]:fx["run_offset"] + fx["run_length"]] = torch.arange(
        fx["run_first_slot"], fx["run_first_slot"] + fx["run_length"])
    g = torch.Generator().manual_seed(3)
    h, hd = 4, 128
    key = torch.randn(fx["length"], h, hd, generator=g).to(torch.bfloat16)
    value = torch.randn(fx["length"], h, hd, generator=g).to(torch.bfloat16)
    kc0 = _sentinel_like(torch.empty(5, 256, h, hd, dtype=torch.bfloat16))
    want_k, want_v = kc0.clone(), kc0.clone()
    okv.store_unified(key, value, want_k, want_v, slots)
    kc, vc = kc0.to(dev), kc0.to(dev)
    dfx.store_kvcache_unified_layout(key.to(dev), value.to(dev), kc, vc, slots.to(dev), None)
    assert torch.equal(_bits(kc), _bits(want_k)) and torch.equal(_bits(vc), _bits(want_v))


def test_store_distinct_bit_exact_and_rearrangement_identity(dev):
    wl = make_workload("c2", num_seqs=5, ctx=(10, 300), page=64)
    pages, page, h, hd, x = wl.k_cache.shape[0], 64, 4, 128, 8
    slots = wl.slot_mapping.clone()
    slots[1::4] = -1
    kd0 = _sentinel_like(torch.empty(pages, h, hd // x, page, x, dtype=torch.bfloat16))
    vd0 = _sentinel_like(torch.empty(pages, h, hd, page, dtype=torch.bfloat16))
    want_k, want_v = kd0.clone(), vd0.clone()
    okv.store_distinct(wl.k_new, wl.v_new, want_k, want_v, slots)
    kd, vd = kd0.to(dev), vd0.to(dev)
    dfx.store_kvcache_distinct_layout(wl.k_new.to(dev), wl.v_new.to(dev), kd, vd, slots.to(dev), None)
    assert torch.equal(_bits(kd), _bits(want_k)) and torch.equal(_bits(vd), _bits(want_v))
    # the identity the reference's example script checks, on zero-initialised caches
    ku = torch.zeros(pages, page, h, hd, dtype=torch.bfloat16, device=dev)
    vu = torch.zeros_like(ku)
    kd2 = torch.zeros(pages, h, hd // x, page, x, dtype=torch.bfloat16, device=dev)
    vd2 = torch.zeros(pages, h, hd, page, dtype=torch.bfloat16, device=dev)
    dfx.store_kvcache_unified_layout(wl.k_new.to(dev), wl.v_new.to(dev), ku, vu, slots.to(dev), None)
    dfx.store_kvcache_distinct_layout(wl.k_new.to(dev), wl.v_new.to(dev), kd2, vd2, slots.to(dev), None)
    assert torch.equal(kd2.permute(0, 3, 1, 2, 4).reshape(pages, page, h, hd), ku)
    assert torch.equal(vd2.permute(0, 3, 1, 2), vu)


@pytest.mark.parametrize("hd,h,page,x,scatter", [
    (128, 4, 64, 8, False), (128, 4, 64, 8, True), (64, 2, 32, 8, True), (128, 3, 16, 8, True),
    (128, 4, 64, 4, True),      # x != 8: the element-wise kernel
    (96, 2, 32, 8, True),       # head_dim the tiled kernel has no variant for
])
def test_store_distinct_tiled_and_elementwise_kernels(dev, hd, h, page, x, scatter):
    """Both kernels behind dfx_kv_store_distinct against the CPU restatement: slots in runs (a
    block stored into its pages) and scattered one by one, skipped rows, rows beyond the cache."""
    g = torch.Generator().manual_seed(hd + page + x)
    n = 201
    pages = max(7, -(-n // page) + 2)
    key = torch.randn(n, h, hd, generator=g).to(torch.bfloat16)
    value = torch.randn(n, h, hd, generator=g).to(torch.bfloat16)
    if scatter:
        slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    else:
        slots = (torch.arange(n, dtype=torch.int32) + 40)
    slots[5::9] = -1
    kd0 = _sentinel_like(torch.empty(pages, h, hd // x, page, x, dtype=torch.bfloat16))
    vd0 = _sentinel_like(torch.empty(pages, h, hd, page, dtype=torch.bfloat16))
    want_k, want_v = kd0.clone(), vd0.clone()
    okv.store_distinct(key, value, want_k, want_v, slots)
    for slot_dtype in (torch.int32, torch.int64):
        kd, vd = kd0.to(dev), vd0.to(dev)
        s = slots.to(slot_dtype).clone()
        dfx.store_kvcache_distinct_layout(key.to(dev), value.to(dev), kd, vd, s.to(dev), None)
        assert torch.equal(_bits(kd), _bits(want_k)) and torch.equal(_bits(vd), _bits(want_v))
    # a slot beyond the cache is skipped
    s = slots.clone()
    s[0] = pages * page + 3
    s0 = slots.clone()
    s0[0] = -1
    okv.store_distinct(key, value, (wk := kd0.clone()), (wv := vd0.clone()), s0)
    kd, vd = kd0.to(dev), vd0.to(dev)
    dfx.store_kvcache_distinct_layout(key.to(dev), value.to(dev), kd, vd, s.to(dev), None)
    assert torch.equal(_bits(kd), _bits(wk)) and torch.equal(_bits(vd), _bits(wv))


@pytest.mark.parametrize("name,over", [
    ("c1", {}), ("c2", {}),
    ("c2", dict(num_seqs=5, page=32, ctx=[0, 32, 64, 33, 500], hd=64, h_kv=2, h_q=2)),   # exact page multiples
    ("c5", dict(num_seqs=5, ctx=(100, 900))),
])
def test_load_bit_exact(dev, name, over):
    wl = make_workload(name, **over)
    want_k, want_v = okv.load(wl.k_cache, wl.v_cache, wl.block_tables, wl.context_lens, wl.seq_lens_new,
                              wl.cu_seqlens_q, wl.cu_seqlens_k, wl.k_new, wl.v_new, wl.k_scale, wl.v_scale)
    g = wl.to(dev)
    md = metadata_for(g, decode_mode="varlen")
    k_out, v_out = dfx.load_kvcache(g.k_cache, g.v_cache, md, g.k_new, g.v_new)
    assert k_out.dtype == g.k_cache.dtype and k_out.shape == want_k.shape
    assert torch.equal(_bits(k_out), _bits(want_k))
    assert torch.equal(_bits(v_out), _bits(want_v))


def test_store_then_load_round_trip_full_size_c2(dev):
    """Size-independent property at the full C2 shape: what is stored behind each context is what
    a load with the grown context returns."""
    wl = make_workload("c2", device=dev)
    md = metadata_for(wl, decode_mode="varlen")
    dfx.store_kvcache_unified_layout(wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.slot_mapping, md)
    grown = wl.context_lens + wl.seq_lens_new
    md2 = dfx.PagedAttnMetaData(
        cu_seqlens_q=torch.zeros_like(wl.cu_seqlens_q), cu_seqlens_k=wl.cu_seqlens_k, context_lens=grown,
        block_tables=wl.block_tables, seq_lens_ts=torch.zeros_like(wl.seq_lens_new), decode_mode="varlen")
    k_out, v_out = dfx.load_kvcache(wl.k_cache, wl.v_cache, md2, wl.k_new[:0], wl.v_new[:0])
    cu_k = wl.cu_seqlens_k.tolist()
    ctx = wl.context_lens.tolist()
    idx = torch.cat([torch.arange(cu_k[s] + ctx[s], cu_k[s + 1]) for s in range(wl.num_seqs)]).to(dev)
    assert torch.equal(k_out[idx].view(torch.int16), wl.k_new.view(torch.int16))
    assert torch.equal(v_out[idx].view(torch.int16), wl.v_new.view(torch.int16))
    # and the context part equals a direct gather of the pages
    s = 7
    pages = wl.block_tables[s, : -(-ctx[s] // wl.page_size)].long()
    direct = wl.k_cache[pages].reshape(-1, wl.num_kv_heads, wl.head_dim)[: ctx[s]]
    assert torch.equal(k_out[cu_k[s]: cu_k[s] + ctx[s]].view(torch.int16), direct.view(torch.int16))


def test_fp8_store_all_bf16_patterns_bit_exact(dev):
    """Every finite bf16 value through the quantising store, several scales."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    x = x[torch.isfinite(x.float())]
    n = x.numel() // 128 * 128
    key = x[:n].reshape(-1, 1, 128).contiguous()
    for scale in (1.0, 0.0123, 3.7, 11.0):
        ks = torch.tensor([scale], dtype=torch.float32)
        t = key.shape[0]
        slots = torch.arange(t, dtype=torch.int32)
        want_k = torch.zeros(1, t, 1, 128, dtype=torch.uint8).view(torch.float8_e4m3fn)
        want_v = want_k.clone()
        okv.store_unified(key, key, want_k, want_v, slots, ks, ks)
        kc = torch.zeros(1, t, 1, 128, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        vc = kc.clone()
        dfx.store_kvcache_unified_layout(key.to(dev), key.to(dev), kc, vc, slots.to(dev), None,
                                         k_scale=ks.to(dev), v_scale=ks.to(dev))
        assert torch.equal(_bits(kc), _bits(want_k)) and torch.equal(_bits(vc), _bits(want_v))


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_store_and_load_bit_exact(dev, seed):
    """Seeded random shapes (heads, head_dim, page sizes, ragged and empty contexts, bf16 and FP8):
    store the fresh block, then gather; both against the oracle, bit for bit."""
    rng = np.random.default_rng(500 + seed)
    h_kv = int(rng.choice([1, 2, 4, 8]))
    over = dict(num_seqs=int(rng.integers(1, 9)), h_q=h_kv, h_kv=h_kv, hd=int(rng.choice([64, 128])),
                page=int(rng.choice([16, 32, 64, 256])), q_len=int(rng.choice([32, 64, 96])))
    over["ctx"] = [int(x) for x in rng.choice([0, 1, 31, 32, 33, 255, 256, 257, 600], over["num_seqs"])]
    fp8 = bool(rng.random() < 0.4)
    wl = make_workload("c5" if fp8 else "c2", seed=seed, **over)
    slots = wl.slot_mapping.clone()
    slots[rng.random(slots.numel()) < 0.2] = -1
    want_kc, want_vc = wl.k_cache.clone(), wl.v_cache.clone()
    okv.store_unified(wl.k_new, wl.v_new, want_kc, want_vc, slots, wl.k_scale, wl.v_scale)
    want_k, want_v = okv.load(want_kc, want_vc, wl.block_tables, wl.context_lens, wl.seq_lens_new,
                              wl.cu_seqlens_q, wl.cu_seqlens_k, wl.k_new, wl.v_new, wl.k_scale, wl.v_scale)
    g = wl.to(dev)
    md = metadata_for(g, decode_mode="varlen")
    dfx.store_kvcache_unified_layout(g.k_new, g.v_new, g.k_cache, g.v_cache,
                                     slots.to(dev).to(torch.int64 if seed % 2 else torch.int32), md)
    k_out, v_out = dfx.load_kvcache(g.k_cache, g.v_cache, md, g.k_new, g.v_new)
    torch.cuda.synchronize()
    assert torch.equal(_bits(g.k_cache), _bits(want_kc)) and torch.equal(_bits(g.v_cache), _bits(want_vc))
    assert torch.equal(_bits(k_out), _bits(want_k)) and torch.equal(_bits(v_out), _bits(want_v))
