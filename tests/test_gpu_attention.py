"""GPU parity of the paged block-diffusion attention kernel against the fp32 CPU oracle.

Tolerances: max-abs 2e-2 for bf16 KV, 6e-2 for FP8 KV (outputs are O(1))."""
import os

import numpy as np
import pytest
import torch

import diffulex_amd as dfx
from diffulex_amd import _lib
from diffulex_amd import dllm_flash_attn as dfa
from diffulex_amd.workloads import make_workload, MASK_FULL, MASK_BLOCK_CAUSAL
from util import ATOL_BF16, ATOL_FP8, metadata_for, oracle_fp32, max_abs_err

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


GENERIC = _lib.DFX_ATTN_GENERIC_PATH   # force the generic tile path where the streaming path would apply
PATHS = [0, GENERIC]


def _run(wl, max_workgroups=0, **kw):
    args = dict(block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
                cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode,
                diffusion_block_size=wl.diffusion_block_size, k_scale=wl.k_scale, v_scale=wl.v_scale,
                max_workgroups=max_workgroups)
    args.update(kw)
    out = dfx.paged_attention(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, **args)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("max_wg", [1, 3, 0])
def test_c1_against_oracle_and_golden(dev, max_wg, flags):
    wl = make_workload("c1")
    want = oracle_fp32(wl)
    got = _run(wl.to(dev), max_wg, flags=flags)
    assert max_abs_err(got, want) <= ATOL_BF16
    fx = np.load(os.path.join(HERE, "golden", "c1_attention.npz"))
    assert np.array_equal(fx["q_bits"], wl.q.view(torch.int16).numpy()), "seeded inputs differ from the fixture"
    assert float(np.abs(got.float().cpu().numpy() - fx["out_fp32"]).max()) <= ATOL_BF16


# the shapes of the reference's decode kernel tests (tests/python/kernel/test_dllm_flash_attn_decode_kernel.py
# :223-391): 1/2/4 sequences, GQA 4 and 8, head_dim 64/128, pages 32/64, DBS 32/64, context 128-512
REF_CASES = [
    dict(num_seqs=1, h_q=8, h_kv=2, hd=128, page=32, ctx=[128], q_len=32, dbs=32),
    dict(num_seqs=4, h_q=32, h_kv=8, hd=128, page=32, ctx=[256] * 4, q_len=32, dbs=32),
    dict(num_seqs=2, h_q=16, h_kv=2, hd=128, page=64, ctx=[512] * 2, q_len=64, dbs=64),
    dict(num_seqs=2, h_q=8, h_kv=1, hd=64, page=32, ctx=[128, 128], q_len=32, dbs=32),
    dict(num_seqs=4, h_q=32, h_kv=4, hd=64, page=64, ctx=[256] * 4, q_len=64, dbs=64),
]


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("case", REF_CASES)
@pytest.mark.parametrize("max_wg", [2, 0])
def test_reference_test_shapes(dev, case, max_wg, flags):
    wl = make_workload("c1", seed=17, **case)
    want = oracle_fp32(wl)
    got = _run(wl.to(dev), max_wg, flags=flags)
    assert max_abs_err(got, want) <= ATOL_BF16


EDGE_CASES = [
    # ragged contexts incl. 0, exact page multiples, one token, prime lengths; page sizes incl. non power of two
    dict(num_seqs=6, h_q=4, h_kv=2, hd=64, page=16, ctx=[0, 1, 16, 63, 64, 65]),
    dict(num_seqs=5, h_q=14, h_kv=2, hd=128, page=256, ctx=[255, 256, 257, 0, 777]),
    dict(num_seqs=3, h_q=6, h_kv=3, hd=128, page=24, ctx=[23, 24, 100]),
    dict(num_seqs=3, h_q=4, h_kv=4, hd=64, page=1, ctx=[5, 0, 70]),
    # more rows than one row tile (GQA 8 x 64 query tokens = 512 rows)
    dict(num_seqs=2, h_q=8, h_kv=1, hd=128, page=32, ctx=[100, 200], q_len=64, dbs=64),
    dict(num_seqs=2, h_q=12, h_kv=1, hd=64, page=32, ctx=[90, 10], q_len=96, dbs=32),
]


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("case", EDGE_CASES)
@pytest.mark.parametrize("mask", [MASK_FULL, MASK_BLOCK_CAUSAL])
@pytest.mark.parametrize("max_wg", [1, 5, 0])
def test_edge_cases(dev, case, mask, max_wg, flags):
    wl = make_workload("c1", seed=23, mask=mask, **case)
    want = oracle_fp32(wl)
    got = _run(wl.to(dev), max_wg, flags=flags)
    assert max_abs_err(got, want) <= ATOL_BF16


def test_ragged_query_lengths_and_empty_sequences(dev):
    """Sequences with different numbers of in-flight blocks, one with none."""
    wl = make_workload("c4", num_seqs=4, h_q=8, h_kv=8, hd=128, page=32, ctx=[100, 300, 50, 0], seed=5)
    q_lens = [96, 32, 0, 64]
    cu = torch.tensor([0, 96, 128, 128, 192], dtype=torch.int32)
    wl.q, wl.k_new, wl.v_new = wl.q[:192], wl.k_new[:192], wl.v_new[:192]
    wl.cu_seqlens_q = cu
    want = oracle_fp32(wl)
    g = wl.to(dev)
    for flags in PATHS:
        for max_wg in (1, 7, 0):
            got = _run(g, max_wg, max_seqlen_q=96, flags=flags)
            assert max_abs_err(got, want) <= ATOL_BF16


@pytest.mark.parametrize("over", [
    dict(num_seqs=4, ctx=(200, 900)),                                       # Dream shape, bf16, small batch
    dict(num_seqs=3, ctx=[256, 0, 511], h_q=8, h_kv=2, hd=64, page=32),
])
def test_fp8_kv_against_oracle(dev, over):
    wl = make_workload("c5", **over)
    want = oracle_fp32(wl)
    for max_wg in (1, 6, 0):
        got = _run(wl.to(dev), max_wg)
        assert max_abs_err(got, want) <= ATOL_FP8


FP8_EDGE_CASES = [
    # 4 waves (at most 128 rows), 8 waves, several row tiles; page sizes that are / are not multiples of 16
    dict(num_seqs=5, h_q=4, h_kv=2, hd=128, page=16, ctx=[0, 1, 64, 65, 300], q_len=32, dbs=32),
    dict(num_seqs=4, h_q=14, h_kv=2, hd=128, page=256, ctx=[255, 256, 257, 1000], q_len=32, dbs=32),
    dict(num_seqs=3, h_q=7, h_kv=1, hd=128, page=48, ctx=[47, 500, 0], q_len=64, dbs=32),
    dict(num_seqs=2, h_q=8, h_kv=1, hd=128, page=32, ctx=[100, 200], q_len=64, dbs=64),
    dict(num_seqs=3, h_q=6, h_kv=3, hd=128, page=24, ctx=[23, 24, 100], q_len=32, dbs=32),
    dict(num_seqs=70, h_q=4, h_kv=1, hd=128, page=64, ctx=(0, 200), q_len=32, dbs=32),   # more units than one plan holds
    dict(num_seqs=40, h_q=14, h_kv=2, hd=128, page=64, ctx=(0, 1500), q_len=32, dbs=32),  # the same with 8 waves: long runs of plain steps across plans
    # head_dim 64: 4 waves with one (up to 128 rows) or two (up to 256 rows) query blocks each, several row tiles
    dict(num_seqs=4, h_q=8, h_kv=2, hd=64, page=32, ctx=[0, 63, 64, 500], q_len=32, dbs=32),
    dict(num_seqs=3, h_q=14, h_kv=2, hd=64, page=256, ctx=[255, 700, 1300], q_len=32, dbs=32),
    dict(num_seqs=3, h_q=16, h_kv=2, hd=64, page=16, ctx=[100, 300, 17], q_len=64, dbs=32),
]


@pytest.mark.parametrize("flags", PATHS + [_lib.DFX_ATTN_NO_PIPELINE])
@pytest.mark.parametrize("case", FP8_EDGE_CASES)
@pytest.mark.parametrize("mask", [MASK_FULL, MASK_BLOCK_CAUSAL])
def test_fp8_edge_cases(dev, case, mask, flags):
    wl = make_workload("c5", seed=29, mask=mask, **case)
    want = oracle_fp32(wl)
    g = wl.to(dev)
    for max_wg in (1, 5, 0):
        got = _run(g, max_wg, flags=flags)
        assert max_abs_err(got, want) <= ATOL_FP8
    if flags == 0:
        # a planned launch with the same cut points gives the same bits
        assert torch.equal(_run(g, 0, plan_cache={}, flags=_lib.DFX_ATTN_EQUAL_RANGES), _run(g, 0))


def test_fresh_k_and_v_with_different_strides(dev):
    """K and V rows cut out of differently shaped parents (the streaming path assumes one layout
    for both and must hand such calls to the generic path)."""
    for name in ("c4", "c5"):
        wl = make_workload(name, num_seqs=3, ctx=(50, 400))
        want = oracle_fp32(wl)
        g = wl.to(dev)
        t, h, d = g.v_new.shape
        parent = torch.zeros(t, h + 1, d + 64, dtype=g.v_new.dtype, device=dev)
        parent[:, 1:, :d] = g.v_new
        g.v_new = parent[:, 1:, :d]
        assert g.v_new.stride() != g.k_new.stride()
        got = _run(g)
        assert max_abs_err(got, want) <= (ATOL_FP8 if name == "c5" else ATOL_BF16)


@pytest.mark.parametrize("flags", PATHS + [_lib.DFX_ATTN_NO_PIPELINE])
@pytest.mark.parametrize("name,over", [
    ("c3", dict(num_seqs=6, ctx=(100, 900))),            # 8 waves, the pipelined tile loop
    ("c1", {}),                                          # head_dim 64, two workgroups per compute unit
    ("c5", dict(num_seqs=4, ctx=(200, 900))),            # FP8 cache: fresh rows fetched by the widening step
    ("c4", dict(num_seqs=3, ctx=(100, 500))),            # block-causal, 96 fresh rows per sequence
    ("c3", dict(num_seqs=6, ctx=(100, 900), hd=64)),     # 8 waves, the pipelined tile loop for head_dim 64
])
def test_fresh_v_sliced_out_of_the_projection(dev, name, over, flags):
    """What a decoder layer passes: K rotated into a buffer of its own, V still a column slice of
    the fused QKV projection, so fresh V rows lie further apart than fresh K rows (same head
    stride).  The streaming kernels take that as it is; with and without a plan, and with the fused
    store, the result equals the one on contiguous copies, bit for bit."""
    wl = make_workload(name, seed=101, **over).to(dev)
    t, h, d = wl.v_new.shape
    qkv = torch.randn(t, (wl.num_q_heads + 2 * h) * d, device=dev).to(torch.bfloat16)
    v_view = qkv[:, (wl.num_q_heads + h) * d:].view(t, h, d)
    v_view.copy_(wl.v_new)
    assert v_view.stride(0) != wl.k_new.stride(0) and v_view.stride(1) == wl.k_new.stride(1)
    want = _run(wl, flags=flags)
    assert max_abs_err(want, oracle_fp32(wl)) <= (ATOL_FP8 if name == "c5" else ATOL_BF16)
    contiguous_v = wl.v_new
    wl.v_new = v_view
    for max_wg in (0, 5):
        ref = _run(wl, max_wg, flags=flags) if max_wg == 0 else None
        got = _run(wl, max_wg, flags=flags | _lib.DFX_ATTN_EQUAL_RANGES, plan_cache={})   # (the cut points of a launch without a plan)
        if ref is not None:
            assert torch.equal(ref, want) and torch.equal(got, want)
        else:
            wl.v_new = contiguous_v
            assert torch.equal(got, _run(wl, max_wg, flags=flags))
            wl.v_new = v_view
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    dfx.store_kvcache_unified_layout(wl.k_new, contiguous_v, kc, vc, wl.slot_mapping, metadata_for(wl, "static"))
    kc2, vc2 = wl.k_cache.clone(), wl.v_cache.clone()
    got = dfx.paged_attention(wl.q, wl.k_new, wl.v_new, kc2, vc2, wl.scale, block_tables=wl.block_tables,
                              context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q,
                              max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode, diffusion_block_size=wl.diffusion_block_size,
                              k_scale=wl.k_scale, v_scale=wl.v_scale, flags=flags, store_slot_mapping=wl.slot_mapping)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert torch.equal(kc2.view(torch.uint8), kc.view(torch.uint8)) and torch.equal(vc2.view(torch.uint8), vc.view(torch.uint8))


@pytest.mark.parametrize("flags", PATHS)
def test_d2f_block_causal_small_c4(dev, flags):
    wl = make_workload("c4", num_seqs=3, ctx=(100, 700))
    want = oracle_fp32(wl)
    got = _run(wl.to(dev), flags=flags)
    assert max_abs_err(got, want) <= ATOL_BF16
    # with every fresh token visible (the reference's current D2F behaviour) the result differs
    full = _run(wl.to(dev), mask_mode=MASK_FULL)
    assert max_abs_err(full, oracle_fp32(wl, mask_mode=MASK_FULL)) <= ATOL_BF16
    assert max_abs_err(full, want) > 1e-3


def test_operator_signatures_static_varlen_prefill(dev):
    wl = make_workload("c1").to(dev)
    want = oracle_fp32(wl)
    o_static = dfx.dllm_flash_attn_decode(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale,
                                          metadata_for(wl, "static"))
    o_varlen = dfx.dllm_flash_attn_decode(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale,
                                          metadata_for(wl, "varlen"))
    assert max_abs_err(o_static, want) <= ATOL_BF16
    assert torch.equal(o_static, o_varlen)
    # scale is honoured
    o2 = dfx.dllm_flash_attn_decode(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, 0.5 * wl.scale,
                                    metadata_for(wl, "static"))
    assert max_abs_err(o2, oracle_fp32(wl, scale=0.5 * wl.scale)) <= ATOL_BF16
    # prefill: varlen self attention, block-causal and full
    pw = make_workload("c1", num_seqs=3, q_len=160, ctx=[0, 0, 0], h_q=8, h_kv=2, hd=128, seed=31)
    cu = torch.tensor([0, 160, 224, 480], dtype=torch.int32)      # ragged: 160, 64, 256
    pw.cu_seqlens_q = cu
    for attn_type, mask in (("block_attention", MASK_BLOCK_CAUSAL), ("full_attention", MASK_FULL)):
        wantp = oracle_fp32(pw, k_cache=None, v_cache=None, mask_mode=mask)
        g = pw.to(dev)
        md = dfx.PagedAttnMetaData(is_prefill=True, cu_seqlens_q=g.cu_seqlens_q, cu_seqlens_k=g.cu_seqlens_q,
                                   max_seqlen_q=256, max_seqlen_k=256, attn_type=attn_type, diffusion_block_size=32)
        gotp = dfx.dllm_flash_attn_prefill(g.q, g.k_new, g.v_new, g.scale, md)
        assert max_abs_err(gotp, wantp) <= ATOL_BF16


def test_attention_module_store_then_decode(dev):
    """Attention.forward: store the fresh block into the cache, attend, flatten heads
    (diffulex/attention/attn_impl.py:42-72)."""
    wl = make_workload("c1").to(dev)
    want = oracle_fp32(wl)
    att = dfx.Attention(wl.num_q_heads, wl.head_dim, wl.scale, wl.num_kv_heads)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    att.k_cache, att.v_cache = kc, vc
    md = metadata_for(wl, "static")
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    t = wl.q.shape[0]
    o = att(wl.q.reshape(t, -1), wl.k_new.reshape(t, -1), wl.v_new.reshape(t, -1))
    assert o.shape == (t, wl.num_q_heads * wl.head_dim) and o.is_contiguous()
    assert max_abs_err(o.view(t, wl.num_q_heads, wl.head_dim), want) <= ATOL_BF16
    slots = wl.slot_mapping.long()
    assert torch.equal(kc.view(-1, wl.num_kv_heads, wl.head_dim)[slots], wl.k_new)


def _to_distinct(cache, x=8):
    """[pages, page, H, hd] -> K [pages, H, hd / x, page, x] and V [pages, H, hd, page], the
    rearrangement the reference's layout check spells out (examples: 'b h n s x -> b s h (n x)')."""
    pages, page, h, hd = cache.shape
    k = cache.view(pages, page, h, hd // x, x).permute(0, 2, 3, 1, 4).contiguous()
    v = cache.permute(0, 2, 3, 1).contiguous()
    return k, v


@pytest.mark.parametrize("name,over", [
    ("c1", dict(page=16)),
    ("c1", dict(num_seqs=3, ctx=[100, 0, 37], page=8)),
    ("c3", dict(num_seqs=5, ctx=(50, 900), page=32)),
    ("c3", dict(num_seqs=3, ctx=[700, 513, 1000])),
    ("c4", dict(num_seqs=2, ctx=[300, 95], page=48)),
    ("c3", dict(num_seqs=4, ctx=(100, 600), h_q=8, h_kv=2, hd=64, page=64)),
])
@pytest.mark.parametrize("max_wg", [0, 3])
def test_decode_on_the_distinct_cache_layout(dev, name, over, max_wg):
    """The reference stores into the distinct layout but refuses to decode from it
    (diffulex/attention/attn_impl.py:66-69); here the same attention runs on it: equal, bit for
    bit, to the generic path on the unified cache holding the same values, and within tolerance
    of the oracle.  Skipped pages (negative table entries) behave alike."""
    wl = make_workload(name, seed=89, **over)
    bt = wl.block_tables.clone()
    if wl.num_seqs > 2:
        bt[2, 1] = -1
        wl.block_tables = bt
    want = oracle_fp32(wl)
    g = wl.to(dev)
    kd = _to_distinct(g.k_cache)[0]
    vd = _to_distinct(g.v_cache)[1]
    args = dict(block_tables=g.block_tables, context_lens=g.context_lens, cu_seqlens_q=g.cu_seqlens_q,
                cu_seqlens_new=g.cu_seqlens_q, max_seqlen_q=g.q_len, mask_mode=g.mask_mode,
                diffusion_block_size=g.diffusion_block_size, max_workgroups=max_wg)
    got = dfx.paged_attention(g.q, g.k_new, g.v_new, kd, vd, g.scale, cache_layout="distinct", flags=GENERIC, **args)
    same = dfx.paged_attention(g.q, g.k_new, g.v_new, g.k_cache, g.v_cache, g.scale, flags=GENERIC, **args)
    # (without the flag: head_dim 128 with pages of a multiple of 64 tokens streams, other shapes run the same kernel)
    dflt = dfx.paged_attention(g.q, g.k_new, g.v_new, kd, vd, g.scale, cache_layout="distinct", **args)
    torch.cuda.synchronize()
    assert max_abs_err(got, want) <= ATOL_BF16
    assert torch.equal(got, same)
    assert max_abs_err(dflt, want) <= ATOL_BF16


STREAMED_DISTINCT = [
    ("c3", dict(num_seqs=6, ctx=(300, 1500)), 0),                                  # Dream heads, 256-token pages, cut items
    ("c3", dict(num_seqs=5, ctx=[0, 1, 7, 64, 129], page=64), 0),                  # no context, a context inside one chunk of 8 tokens
    ("c3", dict(num_seqs=4, ctx=[63, 65, 200, 511], page=128), 5),                 # tile and page ends, five workgroups
    ("c3", dict(num_seqs=3, ctx=[700, 513, 1000]), 3),
    ("c4", dict(num_seqs=3, ctx=(100, 700)), 0),                                   # 96 fresh rows: two fresh tiles, block-causal
    ("c4", dict(num_seqs=2, ctx=(100, 300), h_q=8, h_kv=2, q_len=128, dbs=32), 7), # several row tiles per sequence and head
    ("c3", dict(num_seqs=9, ctx=(30, 400), h_q=8, h_kv=8, q_len=32, page=64), 0),  # 32 rows per item: most waves only fetch
]


@pytest.mark.parametrize("name,over,max_wg", STREAMED_DISTINCT)
@pytest.mark.parametrize("planned", [False, True])
def test_distinct_layout_on_the_streaming_path(dev, name, over, max_wg, planned, monkeypatch):
    """head_dim 128 and pages of a multiple of 64 tokens: the distinct layout streams (K tile chunk-major, V tile
    d-major, the layout's own shapes).  Against the oracle, and against the generic kernel on the same cache; what
    lies in a page behind a sequence's end (NaN here, in K and in V) must not reach the result, nor must a page
    without a table entry."""
    monkeypatch.setattr(dfa, "PLAN_MIN_UNITS_PER_WORKGROUP", 0)   # (plan the tiny cases too)
    wl = make_workload(name, seed=97, **over)
    bt = wl.block_tables.clone()
    if wl.num_seqs > 2 and int(wl.context_lens[2]) > wl.page_size:
        bt[2, 1] = -1
        wl.block_tables = bt
    want = oracle_fp32(wl)
    g = wl.to(dev)
    kc, vc = g.k_cache.clone(), g.v_cache.clone()
    for s in range(g.num_seqs):   # poison the rest of the page that holds the sequence's end
        ctx = int(g.context_lens[s])
        p, used = divmod(ctx, g.page_size)
        if used and int(g.block_tables[s, p]) >= 0:
            kc[int(g.block_tables[s, p]), used:] = float("nan")
            vc[int(g.block_tables[s, p]), used:] = float("nan")
    kd, vd = _to_distinct(kc)[0], _to_distinct(vc)[1]
    args = dict(block_tables=g.block_tables, context_lens=g.context_lens, cu_seqlens_q=g.cu_seqlens_q,
                cu_seqlens_new=g.cu_seqlens_q, max_seqlen_q=g.q_len, mask_mode=g.mask_mode,
                diffusion_block_size=g.diffusion_block_size, max_workgroups=max_wg)
    cache = {} if planned else None
    got = dfx.paged_attention(g.q, g.k_new, g.v_new, kd, vd, g.scale, cache_layout="distinct", plan_cache=cache, **args)
    again = dfx.paged_attention(g.q, g.k_new, g.v_new, kd, vd, g.scale, cache_layout="distinct", plan_cache=cache, **args)
    gen = dfx.paged_attention(g.q, g.k_new, g.v_new, kd, vd, g.scale, cache_layout="distinct", flags=GENERIC, **args)
    # the compiler-scheduled step on the same tiles (the default is the generated one)
    cs = dfx.paged_attention(g.q, g.k_new, g.v_new, kd, vd, g.scale, cache_layout="distinct", flags=_lib.DFX_ATTN_NO_PIPELINE,
                             plan_cache={} if planned else None, **args)
    torch.cuda.synchronize()
    if planned:
        assert len(cache) == 1 and next(iter(cache.values())) is not None, "the streaming path takes a plan"
    for out in (got, cs):
        assert torch.isfinite(out.float()).all()
        assert max_abs_err(out, want) <= ATOL_BF16
        assert max_abs_err(out, gen) <= 1e-2
    assert max_abs_err(got, cs) <= 1e-2
    assert torch.equal(got, again)


def test_distinct_layout_streams_with_v_sliced_out_of_the_projection(dev):
    """Fresh V as a column slice of the QKV projection (another token stride than K's) on the distinct layout's
    streaming path: the fresh tile's V rows land row-major and are transposed inside LDS."""
    wl = make_workload("c3", seed=99, num_seqs=4, ctx=(200, 900)).to(dev)
    want = oracle_fp32(wl)
    T, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    qkv = torch.empty(T, (hq + 2 * hkv) * hd, dtype=torch.bfloat16, device=dev)
    q, k, v = (x.view(T, -1, hd) for x in qkv.split([hq * hd, hkv * hd, hkv * hd], dim=-1))
    q.copy_(wl.q), k.copy_(wl.k_new), v.copy_(wl.v_new)
    kd, vd = _to_distinct(wl.k_cache)[0], _to_distinct(wl.v_cache)[1]
    got = dfx.paged_attention(q, k.contiguous(), v, kd, vd, wl.scale, cache_layout="distinct", block_tables=wl.block_tables,
                              context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q,
                              max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode, diffusion_block_size=wl.diffusion_block_size)
    torch.cuda.synchronize()
    assert max_abs_err(got, want) <= ATOL_BF16


def test_attention_module_on_the_distinct_layout(dev):
    """Attention.forward with kv_cache_layout == "distinct": store through
    store_kvcache_distinct_layout, then decode from that cache."""
    wl = make_workload("c3", seed=91, num_seqs=4, ctx=(100, 700), page=32).to(dev)
    want = oracle_fp32(wl)
    att = dfx.Attention(wl.num_q_heads, wl.head_dim, wl.scale, wl.num_kv_heads)
    att.k_cache, att.v_cache = _to_distinct(wl.k_cache)[0], _to_distinct(wl.v_cache)[1]
    md = metadata_for(wl, "static")
    md.kv_cache_layout = "distinct"
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    t = wl.q.shape[0]
    o = att(wl.q.reshape(t, -1), wl.k_new.reshape(t, -1), wl.v_new.reshape(t, -1))
    torch.cuda.synchronize()
    assert max_abs_err(o.view(t, wl.num_q_heads, wl.head_dim), want) <= ATOL_BF16
    # the block was stored where the slot mapping says
    ku = att.k_cache.permute(0, 3, 1, 2, 4).reshape(wl.k_cache.shape)
    vu = att.v_cache.permute(0, 3, 1, 2)
    slots = wl.slot_mapping.long()
    assert torch.equal(ku.reshape(-1, wl.num_kv_heads, wl.head_dim)[slots], wl.k_new)
    assert torch.equal(vu.reshape(-1, wl.num_kv_heads, wl.head_dim)[slots], wl.v_new)


def test_invariants_at_full_c3_size(dev):
    """Properties that need no oracle at the full Dream-7B shape, plus the oracle on a few sequences."""
    wl = make_workload("c3", device=dev)
    out = _run(wl)
    assert torch.isfinite(out.float()).all()
    want = oracle_fp32(wl, seqs=[0, 17, 63])
    cu = wl.cu_seqlens_q.tolist()
    for s, w in zip([0, 17, 63], want):
        assert max_abs_err(out[cu[s]:cu[s + 1]], w) <= ATOL_BF16
    # V == 1 gives O == 1 (softmax rows sum to one) for every query of every sequence
    ones = dfx.paged_attention(
        wl.q, wl.k_new, torch.ones_like(wl.v_new), wl.k_cache, torch.ones_like(wl.v_cache), wl.scale,
        block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
        cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len)
    assert float((ones.float() - 1).abs().max()) <= 1e-2
    # permuting the physical pages together with the block table changes nothing
    n_pages = wl.k_cache.shape[0]
    perm = torch.randperm(n_pages, generator=torch.Generator("cpu").manual_seed(3)).to(dev)
    kc2, vc2 = torch.empty_like(wl.k_cache), torch.empty_like(wl.v_cache)
    kc2[perm] = wl.k_cache
    vc2[perm] = wl.v_cache
    bt2 = wl.block_tables.clone()
    valid = bt2 >= 0
    bt2[valid] = perm[bt2[valid].long()].to(torch.int32)
    out2 = dfx.paged_attention(
        wl.q, wl.k_new, wl.v_new, kc2, vc2, wl.scale, block_tables=bt2, context_lens=wl.context_lens,
        cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len)
    assert torch.equal(out2, out)
    # neither the partition nor the tile path changes the result beyond rounding
    out3 = _run(wl, max_workgroups=97)
    assert max_abs_err(out3, out) <= 1e-2
    out4 = _run(wl, flags=GENERIC)
    assert max_abs_err(out4, out) <= 1e-2


def test_result_bits_do_not_depend_on_which_piece_merges(dev):
    """Items cut between workgroups are merged by whichever workgroup finishes last, which varies
    from launch to launch; the merge must be commutative to the last bit.  (A fused multiply-add
    in the merge breaks this about once in 200 launches at this size.)"""
    wl = make_workload("c3", device=dev)
    ref = _run(wl)
    n_pages = wl.k_cache.shape[0]
    gen = torch.Generator("cpu").manual_seed(11)
    for it in range(150):
        perm = torch.randperm(n_pages, generator=gen).to(dev)    # fresh allocations: other addresses, other timing
        kc2, vc2 = torch.empty_like(wl.k_cache), torch.empty_like(wl.v_cache)
        kc2[perm] = wl.k_cache
        vc2[perm] = wl.v_cache
        bt2 = wl.block_tables.clone()
        valid = bt2 >= 0
        bt2[valid] = perm[bt2[valid].long()].to(torch.int32)
        out = dfx.paged_attention(
            wl.q, wl.k_new, wl.v_new, kc2, vc2, wl.scale, block_tables=bt2, context_lens=wl.context_lens,
            cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len)
        assert torch.equal(out, ref), f"launch {it}"


def test_full_size_c4_and_c5_on_sampled_sequences(dev):
    """Full C4 and C5, without a plan and with the default plan (the launch bench.py times), each against
    the oracle on sampled sequences."""
    for name, seqs, tol in (("c4", [0, 13, 31], ATOL_BF16), ("c5", [3, 64, 100], ATOL_FP8)):
        wl = make_workload(name, device=dev)
        want = oracle_fp32(wl, seqs=seqs)
        cu = wl.cu_seqlens_q.tolist()
        cache = {}
        for kw in ({}, dict(plan_cache=cache), dict(plan_cache=cache)):
            out = _run(wl, **kw)
            assert torch.isfinite(out.float()).all()
            for s, w in zip(seqs, want):
                assert max_abs_err(out[cu[s]:cu[s + 1]], w) <= tol, (name, s, bool(kw))
        assert len(cache) == 1 and next(iter(cache.values())) is not None
        del wl, out, cache
        torch.cuda.empty_cache()


def test_full_size_c3_with_head_dim_64_on_sampled_sequences(dev):
    """The C3 shape with the head size of the reference's kernel tests (224 rows per item: the pipelined kernel's
    head_dim 64 variant), without a plan and with the default one, against the oracle on sampled sequences and
    against the compiler-scheduled step."""
    wl = make_workload("c3", device=dev, hd=64)
    seqs = [0, 21, 40, 63]
    want = oracle_fp32(wl, seqs=seqs)
    cu = wl.cu_seqlens_q.tolist()
    cache = {}
    outs = [_run(wl), _run(wl, plan_cache=cache), _run(wl, plan_cache=cache), _run(wl, flags=_lib.DFX_ATTN_NO_PIPELINE)]
    for out in outs:
        assert torch.isfinite(out.float()).all()
        for s, w in zip(seqs, want):
            assert max_abs_err(out[cu[s]:cu[s + 1]], w) <= ATOL_BF16, s
    assert torch.equal(outs[1], outs[2])
    assert max_abs_err(outs[0], outs[3]) <= 1e-2


def test_the_planned_launch_the_benchmark_times_against_the_oracle(dev):
    """Full C3 with the default plan (cut points from the capacity sweep: plan mode 2), the launch the
    headline figure is measured on: against the oracle on sampled sequences, and the same bits from
    every launch that reads the plan."""
    wl = make_workload("c3", device=dev)
    cache = {}
    got = _run(wl, plan_cache=cache)
    plan = next(iter(cache.values()))
    n_wg = torch.cuda.get_device_properties(dev).multi_processor_count
    hdr, ranges, _ = _read_plan(plan, wl.num_seqs, n_wg)
    assert hdr["magic"] == 0x44465850 and hdr["mode"] == 2 and hdr["n_active"] == n_wg
    seqs = [0, 9, 17, 31, 44, 63]
    cu = wl.cu_seqlens_q.tolist()
    wants = oracle_fp32(wl, seqs=seqs)
    for s, want in zip(seqs, wants):
        assert max_abs_err(got[cu[s]:cu[s + 1]], want) <= ATOL_BF16, f"sequence {s}"
    for _ in range(3):
        assert torch.equal(_run(wl, plan_cache=cache), got)
    # The plan deals the sequences to the workgroups in an order of its own where that needs a smaller
    # capacity per workgroup (at this shape it does); in the batch's order other items are cut, so the
    # rows agree to rounding only.  Both orders tile the unit space.
    assert hdr["reordered"] == 1
    cache2 = {}
    got2 = _run(wl, plan_cache=cache2, flags=_lib.DFX_ATTN_BATCH_ORDER)
    hdr2, ranges2, _ = _read_plan(next(iter(cache2.values())), wl.num_seqs, n_wg)
    assert hdr2["mode"] == 2 and hdr2["reordered"] == 0 and hdr2["total"] == hdr["total"]
    assert max_abs_err(got2, got) <= 1e-2
    for s, want in zip(seqs, wants):
        assert max_abs_err(got2[cu[s]:cu[s + 1]], want) <= ATOL_BF16, f"sequence {s}"
    for r in (ranges, ranges2):
        spans = [(int(x[0]), int(x[1])) for x in r]
        assert spans[0][0] == 0 and spans[-1][1] == hdr["total"] and all(x[1] == y[0] for x, y in zip(spans, spans[1:]))


def test_decode_under_inference_mode_eager_and_captured(dev):
    """The reference's runners build the step's metadata and run the model under
    torch.inference_mode() (strategy/block_diffusion/engine/model_runner.py:206,
    strategy/d2f/engine/model_runner.py:291): such tensors carry no version counter.  The plan cache
    must work on them, eagerly and inside a capture."""
    with torch.inference_mode():
        wl = make_workload("c3", num_seqs=6, ctx=(300, 900), seed=43).to(dev)
        assert wl.context_lens.is_inference()
        att = dfx.Attention(wl.num_q_heads, wl.head_dim, wl.scale, wl.num_kv_heads)
        att.k_cache, att.v_cache = wl.k_cache, wl.v_cache
        md = metadata_for(wl, "static")
        dfx.set_fetch_fn_for_attn_metadata(lambda: md)
        t = wl.q.shape[0]
        q, k, v = (x.reshape(t, -1).clone() for x in (wl.q, wl.k_new, wl.v_new))
        want = oracle_fp32(wl)
        eager = att(q, k, v)
        again = att(q, k, v)          # the second layer of the step: same metadata object, same plan
        torch.cuda.synchronize()
        assert len(md.dfx_plan_cache) == 1
        assert torch.equal(eager, again)
        assert max_abs_err(eager.view(t, wl.num_q_heads, wl.head_dim), want) <= ATOL_BF16
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            o_static = att(q, k, v)
        assert len(md.dfx_plan_cache) == 2   # a plan of its own inside the capture
        for _ in range(2):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(o_static, eager)


def test_static_decode_in_a_captured_graph(dev):
    """The block-diffusion runner replays the decode step from a captured graph
    (strategy/block_diffusion/engine/model_runner.py:206-274): store + attention are captured once,
    then replayed with new contents in the same tensors.  Every replay is compared with the eager
    result on the same inputs, with eager launches and synchronisations in between."""
    wl = make_workload("c3", num_seqs=6, ctx=(300, 900), seed=41).to(dev)   # cut items: partials and counters in use
    att = dfx.Attention(wl.num_q_heads, wl.head_dim, wl.scale, wl.num_kv_heads)
    att.k_cache, att.v_cache = wl.k_cache, wl.v_cache
    md = metadata_for(wl, "static")
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    t = wl.q.shape[0]
    q, k, v = (x.reshape(t, -1).clone() for x in (wl.q, wl.k_new, wl.v_new))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream: its workspace exists before the capture
        att(q, k, v)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        o_static = att(q, k, v)
    gen = torch.Generator(device=dev).manual_seed(7)
    for rep in range(4):
        for x in (q, k, v):
            x.copy_(torch.randn(x.shape, generator=gen, device=dev, dtype=torch.float32).to(x.dtype))
        if rep == 2:   # other contexts, same shapes
            md.context_lens.copy_(torch.clamp(md.context_lens - 37 * (rep + 1), min=0))
        graph.replay()
        torch.cuda.synchronize()
        got = o_static.clone()
        eager = att(q, k, v)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {rep}"
    wl2 = wl.to("cpu")
    wl2.q, wl2.k_new, wl2.v_new = (x.view(t, -1, wl.head_dim).cpu() for x in (q, k, v))
    wl2.context_lens = md.context_lens.cpu()
    assert max_abs_err(got.view(t, wl.num_q_heads, wl.head_dim), oracle_fp32(wl2)) <= ATOL_BF16


def test_graphs_captured_as_the_reference_runner_does(dev):
    """strategy/block_diffusion/engine/model_runner.py:239-262: warm up on the current stream, then
    capture one graph per batch size, largest first, on the capture context's own side stream.
    Here the smaller graph is replayed first, and the eager warm-up uses a smaller batch than the
    first capture (so the capture needs a larger workspace than any eager call has made)."""
    sizes = (12, 5)
    wls = {n: make_workload("c3", num_seqs=n, ctx=(300, 1100), seed=50 + n).to(dev) for n in sizes}
    att = dfx.Attention(28, 128, wls[5].scale, 4)
    cur = {}
    dfx.set_fetch_fn_for_attn_metadata(lambda: cur["md"])

    def call(n):
        wl = wls[n]
        att.k_cache, att.v_cache = wl.k_cache, wl.v_cache
        cur["md"] = metadata_for(wl, "static")
        t = wl.q.shape[0]
        return att(wl.q.reshape(t, -1), wl.k_new.reshape(t, -1), wl.v_new.reshape(t, -1))

    call(5)                                   # warm-up on the current stream
    torch.cuda.synchronize()
    graphs, outs = {}, {}
    for n in sizes:
        graphs[n] = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graphs[n]):
            outs[n] = call(n)
    for n in reversed(sizes):
        graphs[n].replay()
        torch.cuda.synchronize()
        got = outs[n].clone()
        want = call(n)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"batch {n}"
        assert max_abs_err(got.view(-1, 28, 128), oracle_fp32(wls[n])) <= ATOL_BF16


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("name,over,n_real", [
    ("c3", dict(num_seqs=8, ctx=(200, 900)), 5),
    ("c3", dict(num_seqs=16, ctx=(100, 2000), page=32), 9),
    ("c5", dict(num_seqs=8, ctx=(300, 1200)), 3),
])
def test_graph_buffers_padded_the_way_the_reference_pads_them(dev, name, over, n_real, flags):
    """The reference replays a graph captured for a larger batch on zero-filled buffers with the
    step's values in front (strategy/block_diffusion/engine/model_runner.py:176-197): behind the
    real sequences cu_seqlens drop back to 0 (the first padded sequence has a negative length),
    context_lens are 0 and the block-table rows are all page 0.  The real sequences' rows come out
    as without the padding; at capture time cu_seqlens_k counts in steps of max_model_len (:221-223),
    offsets far beyond the fresh rows, which must not be followed."""
    wl = make_workload(name, seed=97, **over).to(dev)
    n_pad, dbs = wl.num_seqs, wl.q_len
    cu = wl.cu_seqlens_q.clone()
    cu[n_real + 1:] = 0
    ctx = wl.context_lens.clone()
    ctx[n_real:] = 0
    bt = wl.block_tables.clone()
    bt[n_real:] = 0
    common = dict(max_seqlen_q=dbs, mask_mode=wl.mask_mode, diffusion_block_size=wl.diffusion_block_size,
                  k_scale=wl.k_scale, v_scale=wl.v_scale, flags=flags)
    t = n_real * dbs
    want = dfx.paged_attention(wl.q[:t], wl.k_new[:t], wl.v_new[:t], wl.k_cache, wl.v_cache, wl.scale,
                               block_tables=wl.block_tables[:n_real], context_lens=wl.context_lens[:n_real],
                               cu_seqlens_q=wl.cu_seqlens_q[:n_real + 1], cu_seqlens_new=wl.cu_seqlens_q[:n_real + 1],
                               **common)
    out = torch.full_like(wl.q, 3.0)
    dfx.paged_attention(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, block_tables=bt, context_lens=ctx,
                        cu_seqlens_q=cu, cu_seqlens_new=cu, out=out, **common)
    torch.cuda.synchronize()
    assert torch.equal(out[:t], want)
    assert (out[t:] == 3.0).all()                       # rows of the padding are not touched
    assert max_abs_err(want, oracle_fp32(wl)[:t]) <= (ATOL_FP8 if name == "c5" else ATOL_BF16)
    # capture-time metadata: zero lengths and tables, fresh-row offsets in steps of max_model_len
    far = (torch.arange(n_pad + 1, device=dev, dtype=torch.int32) * 4096)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    slots = torch.zeros(n_pad * dbs, dtype=torch.int32, device=dev)
    got = dfx.paged_attention(wl.q, wl.k_new, wl.v_new, kc, vc, wl.scale, block_tables=torch.zeros_like(bt),
                              context_lens=torch.zeros_like(ctx), cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=far,
                              store_slot_mapping=slots, **common)
    torch.cuda.synchronize()
    # only sequence 0 has fresh rows inside k_new: offsets 0 .. 4096 are cut to the rows there are
    clamped = torch.clamp(far, max=n_pad * dbs).cpu()
    ref = oracle_fp32(wl, context_lens=torch.zeros_like(ctx).cpu(), cu_seqlens_new=clamped)
    assert max_abs_err(got[:dbs], ref[:dbs]) <= (ATOL_FP8 if name == "c5" else ATOL_BF16)


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("name,over", [
    ("c1", {}),
    ("c3", dict(num_seqs=5, ctx=(200, 700))),
    ("c4", dict(num_seqs=3, ctx=(100, 500))),
    ("c5", dict(num_seqs=4, ctx=(200, 900))),
    ("c5", dict(num_seqs=3, ctx=[256, 0, 511], h_q=8, h_kv=2, hd=64, page=32)),
    ("c3", dict(num_seqs=5, ctx=(100, 800), hd=64)),     # 224 rows, head_dim 64: the pipelined kernel's narrow variant
])
def test_store_fused_into_the_attention_launch(dev, name, over, flags):
    """One launch that stores the fresh block and attends == the store launch followed by the
    attention launch (diffulex/attention/attn_impl.py:54-69): same cache bits, same output bits."""
    wl = make_workload(name, seed=53, **over).to(dev)
    md = metadata_for(wl, "static")
    for slot_dtype in (torch.int32, torch.int64):
        slots = wl.slot_mapping.to(slot_dtype).clone()
        slots[1::7] = -1                                   # rows that are not stored
        slots[3] = wl.k_cache.shape[0] * wl.k_cache.shape[1] + 5   # out of range: skipped
        for max_wg in (0, 3, 1000):                        # 1000: more workgroups than units
            kc_a, vc_a = wl.k_cache.clone(), wl.v_cache.clone()
            dfx.store_kvcache_unified_layout(wl.k_new, wl.v_new, kc_a, vc_a, slots, md)
            want = _run(wl, max_wg, flags=flags)
            kc_b, vc_b = wl.k_cache.clone(), wl.v_cache.clone()
            args = dict(block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
                        cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode,
                        diffusion_block_size=wl.diffusion_block_size, k_scale=wl.k_scale, v_scale=wl.v_scale,
                        max_workgroups=max_wg, flags=flags, store_slot_mapping=slots)
            got = dfx.paged_attention(wl.q, wl.k_new, wl.v_new, kc_b, vc_b, wl.scale, **args)
            torch.cuda.synchronize()
            assert torch.equal(got, want)
            assert torch.equal(kc_b.view(torch.uint8), kc_a.view(torch.uint8))
            assert torch.equal(vc_b.view(torch.uint8), vc_a.view(torch.uint8))
            assert not torch.equal(kc_b.view(torch.uint8), wl.k_cache.view(torch.uint8))  # something was stored


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("name,over", [
    ("c1", dict(num_seqs=3, ctx=[100, 64, 37])),                       # page 16: four pages per tile
    ("c3", dict(num_seqs=4, ctx=[700, 256, 1000, 90], page=32)),
    ("c3", dict(num_seqs=3, ctx=[700, 513, 1000])),                    # page 256: whole tiles vanish
    ("c5", dict(num_seqs=3, ctx=[700, 513, 1000])),
    ("c5", dict(num_seqs=3, ctx=[700, 513, 1000], page=32)),           # FP8: bands of a tile missing, masked per band
    ("c4", dict(num_seqs=2, ctx=[300, 95], page=48)),
])
def test_pages_with_negative_table_entries_are_skipped(dev, name, over, flags):
    """The reference skips a page whose block-table entry is negative: its tokens take no part
    (diffulex_kernel/python/dllm_flash_attn.py:260-261; the oracle follows
    tests/python/kernel/test_dllm_flash_attn_decode_kernel.py:63-76)."""
    wl = make_workload(name, seed=61, **over)
    bt = wl.block_tables.clone()
    page = wl.page_size
    for s in range(wl.num_seqs):
        n_ctx_pages = -(-int(wl.context_lens[s]) // page)
        for p in range(n_ctx_pages):
            if (p + s) % 3 == 1:
                bt[s, p] = -1
    bt[0, 0] = wl.k_cache.shape[0] + 7        # out of range counts as missing too
    wl.block_tables = bt
    want = oracle_fp32(wl, block_tables=torch.where(bt >= wl.k_cache.shape[0], torch.full_like(bt, -1), bt))
    g = wl.to(dev)
    tol = ATOL_FP8 if name == "c5" else ATOL_BF16
    for max_wg in (0, 3):
        got = _run(g, max_wg, flags=flags)
        assert max_abs_err(got, want) <= tol


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("name,over", [
    ("c3", dict(num_seqs=4, ctx=[300, 513, 64, 700], page=32)),
    ("c5", dict(num_seqs=3, ctx=[300, 513, 200])),
    ("c4", dict(num_seqs=3, ctx=[100, 300, 95], page=48)),
])
def test_rows_with_no_visible_key_get_zeros(dev, name, over, flags):
    """A sequence all of whose context pages are skipped and that brings no fresh rows has nothing
    to attend to: its rows are zeros (finite), the other sequences are unaffected."""
    wl = make_workload(name, seed=67, **over)
    bt = wl.block_tables.clone()
    bt[1, :] = -1
    wl.block_tables = bt
    cu_q = wl.cu_seqlens_q.tolist()
    lens_new = [cu_q[i + 1] - cu_q[i] for i in range(wl.num_seqs)]
    lens_new[1] = 0                                    # sequence 1: no fresh rows either
    cu_new = torch.tensor([0] + np.cumsum(lens_new).tolist(), dtype=torch.int32)
    keep = torch.cat([torch.arange(cu_q[i], cu_q[i + 1]) for i in range(wl.num_seqs) if i != 1])
    wl.k_new, wl.v_new = wl.k_new[keep].contiguous(), wl.v_new[keep].contiguous()
    want = oracle_fp32(wl, cu_seqlens_new=cu_new)
    assert float(want[cu_q[1]:cu_q[2]].abs().max()) == 0.0
    g = wl.to(dev)
    tol = ATOL_FP8 if name == "c5" else ATOL_BF16
    for max_wg in (0, 3):
        got = _run(g, max_wg, flags=flags, cu_seqlens_new=cu_new.to(dev))
        assert torch.isfinite(got.float()).all()
        assert float(got[cu_q[1]:cu_q[2]].float().abs().max()) == 0.0
        assert max_abs_err(got, want) <= tol


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("name,over", [
    ("c3", dict(num_seqs=5, ctx=(200, 700))),
    ("c5", dict(num_seqs=4, ctx=(200, 900))),
    ("c4", dict(num_seqs=3, ctx=(100, 500))),
])
def test_fresh_rows_are_bounded_by_the_rows_passed(dev, name, over, flags):
    """Offsets in cu_seqlens_new that point beyond the rows of k_new / v_new (padded batches) are
    cut to the rows there are, for the attention and for the fused store: the result equals the one
    with the offsets clamped, and the cache rows of the missing tokens stay as they were."""
    wl = make_workload(name, seed=71, **over).to(dev)
    cu = wl.cu_seqlens_q
    t_all = int(cu[-1])
    t_have = int(cu[-2]) + (t_all - int(cu[-2])) // 2          # the last sequence lost half its fresh rows
    k_new, v_new = wl.k_new[:t_have].contiguous(), wl.v_new[:t_have].contiguous()
    slots = wl.slot_mapping[:t_have].contiguous()
    cu_clamped = torch.clamp(cu, max=t_have)
    common = dict(block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=cu,
                  max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode, diffusion_block_size=wl.diffusion_block_size,
                  k_scale=wl.k_scale, v_scale=wl.v_scale, flags=flags)
    for max_wg in (0, 3):
        kc_a, vc_a = wl.k_cache.clone(), wl.v_cache.clone()
        want = dfx.paged_attention(wl.q, k_new, v_new, kc_a, vc_a, wl.scale, cu_seqlens_new=cu_clamped,
                                   store_slot_mapping=slots, max_workgroups=max_wg, **common)
        kc_b, vc_b = wl.k_cache.clone(), wl.v_cache.clone()
        got = dfx.paged_attention(wl.q, k_new, v_new, kc_b, vc_b, wl.scale, cu_seqlens_new=cu,
                                  store_slot_mapping=slots, max_workgroups=max_wg, **common)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(kc_b.view(torch.uint8), kc_a.view(torch.uint8))
        assert torch.equal(vc_b.view(torch.uint8), vc_a.view(torch.uint8))
    c = wl.to("cpu")
    ref = oracle_fp32(c, k_new=c.k_new[:t_have], v_new=c.v_new[:t_have], cu_seqlens_new=cu_clamped.cpu())
    assert max_abs_err(got, ref) <= (ATOL_FP8 if name == "c5" else ATOL_BF16)


@pytest.mark.parametrize("name,over,tol", [
    # more sequences than the two-workgroups-per-CU variant plans for (1023): the one-per-CU variants
    ("c3", dict(num_seqs=1500, ctx=(0, 150), h_q=8, h_kv=2), ATOL_BF16),
    ("c1", dict(num_seqs=1100, ctx=(0, 90), h_q=4, h_kv=4), ATOL_BF16),
    ("c5", dict(num_seqs=1200, ctx=(0, 200), h_q=8, h_kv=2), ATOL_FP8),
    # the largest batch the kernels take
    ("c3", dict(num_seqs=4095, ctx=(0, 40), h_q=4, h_kv=1, q_len=32), ATOL_BF16),
])
def test_many_short_sequences(dev, name, over, tol):
    wl = make_workload(name, seed=71, **over)
    g = wl.to(dev)
    seqs = [0, 1, wl.num_seqs // 2, wl.num_seqs - 2, wl.num_seqs - 1]
    want = oracle_fp32(wl, seqs=seqs)
    cu = wl.cu_seqlens_q.tolist()
    for flags in PATHS:
        got = _run(g, flags=flags)
        assert torch.isfinite(got.float()).all()
        for s, w in zip(seqs, want):
            assert max_abs_err(got[cu[s]:cu[s + 1]], w) <= tol
    assert max_abs_err(_run(g), _run(g, max_workgroups=64)) <= 1e-2   # another partition: rounding differences only


def test_batch_above_the_limit_is_refused(dev):
    wl = make_workload("c1", num_seqs=4096, ctx=(0, 20), seed=3).to(dev)
    with pytest.raises(Exception):
        _run(wl)


@pytest.mark.parametrize("over", [
    dict(num_seqs=3, h_q=7, h_kv=1, q_len=512, ctx=[0, 0, 0]),              # prefill shape: 2 row tiles per head
    dict(num_seqs=2, h_q=2, h_kv=2, q_len=512, ctx=[200, 0]),               # one head per KV head, cached prefix
    dict(num_seqs=2, h_q=14, h_kv=2, q_len=1024, ctx=[0, 333], hd=64),      # 4 row tiles per head, head_dim 64
    dict(num_seqs=2, h_q=4, h_kv=4, q_len=256, ctx=[300, 70]),              # one row tile per head: nothing to skip
    dict(num_seqs=2, h_q=6, h_kv=2, q_len=200, ctx=[0, 90]),                # row tiles straddle heads: every tile kept
])
@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("max_wg", [0, 5])
def test_block_causal_row_tiles_skip_the_fresh_tiles_they_cannot_see(dev, over, flags, max_wg):
    """Row tiles of long block-causal sequences own only the fresh tiles some of their rows can
    see; the result is the oracle's, whatever the partition."""
    wl = make_workload("c4", seed=31, page=64, **over)
    want = oracle_fp32(wl)
    got = _run(wl.to(dev), max_workgroups=max_wg, flags=flags)
    assert torch.isfinite(got.float()).all()
    assert max_abs_err(got, want) <= ATOL_BF16


def test_block_causal_prefill_without_a_cache(dev):
    B, L, hq, hkv, hd = 2, 768, 8, 2, 128
    g = torch.Generator().manual_seed(17)
    q = torch.randn(B * L, hq, hd, generator=g).to(torch.bfloat16)
    k = torch.randn(B * L, hkv, hd, generator=g).to(torch.bfloat16)
    v = torch.randn(B * L, hkv, hd, generator=g).to(torch.bfloat16)
    cu = torch.arange(0, B * L + 1, L, dtype=torch.int32)
    from oracle import attention as oat
    want = oat.paged_attention_fp32(q, k, v, None, None, None, None, cu, cu, hd ** -0.5,
                                    mask_mode=MASK_BLOCK_CAUSAL, dbs=32)
    for flags in PATHS:
        got = dfx.paged_attention(q.to(dev), k.to(dev), v.to(dev), None, None, hd ** -0.5, block_tables=None,
                                  context_lens=None, cu_seqlens_q=cu.to(dev), cu_seqlens_new=cu.to(dev),
                                  max_seqlen_q=L, mask_mode=MASK_BLOCK_CAUSAL, diffusion_block_size=32, flags=flags)
        torch.cuda.synchronize()
        assert max_abs_err(got, want) <= ATOL_BF16


@pytest.mark.parametrize("case", [
    # (lengths, query heads, KV heads, head_dim, diffusion block size)
    ((40, 100, 333), 14, 2, 128, 8),      # lengths that are no multiple of a wave's 32 rows: waves whose rows span two heads
    ((96, 200), 8, 2, 128, 48),           # blocks of 48 positions: waves whose rows span two blocks
    ((64, 512, 31), 8, 1, 128, 16),       # two blocks per wave
    ((300,), 28, 4, 128, 96),
    ((640, 1024), 14, 2, 128, 32),        # a block per wave, row tiles of eight blocks: waves that see nothing of a tile
    ((640, 130), 8, 2, 128, 64),          # two waves per block
    ((200, 577), 16, 2, 64, 32),
    ((100, 72), 8, 2, 64, 24),
])
def test_block_causal_prefill_where_the_waves_of_a_row_tile_see_different_keys(dev, case):
    """The pipelined kernel decides per wave whether a tile needs the block-causal mask, masks with one threshold
    where all of a wave's rows see the same keys and row by row where they do not: block sizes below, at and
    above a wave's 32 rows, lengths that put the rows of two heads or two blocks into one wave."""
    from oracle import attention as oat
    lengths, hq, hkv, hd, dbs = case
    T = sum(lengths)
    g = torch.Generator().manual_seed(T + dbs)
    q = torch.randn(T, hq, hd, generator=g).to(torch.bfloat16)
    k = torch.randn(T, hkv, hd, generator=g).to(torch.bfloat16)
    v = torch.randn(T, hkv, hd, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + list(np.cumsum(lengths)), dtype=torch.int32)
    want = oat.paged_attention_fp32(q, k, v, None, None, None, None, cu, cu, hd ** -0.5, mask_mode=MASK_BLOCK_CAUSAL, dbs=dbs)
    for max_wg in (0, 5):
        got = dfx.paged_attention(q.to(dev), k.to(dev), v.to(dev), None, None, hd ** -0.5, block_tables=None, context_lens=None,
                                  cu_seqlens_q=cu.to(dev), cu_seqlens_new=cu.to(dev), max_seqlen_q=max(lengths),
                                  mask_mode=MASK_BLOCK_CAUSAL, diffusion_block_size=dbs, max_workgroups=max_wg)
        torch.cuda.synchronize()
        assert torch.isfinite(got.float()).all()
        assert max_abs_err(got, want) <= ATOL_BF16


@pytest.mark.parametrize("mask", [MASK_FULL, MASK_BLOCK_CAUSAL])
def test_prefill_with_v_sliced_out_of_the_projection(dev, mask):
    """A prefill as a decoder layer issues it: K rotated into a buffer of its own, V still a column slice of the
    fused QKV projection (another token stride, the same head stride).  Long enough for the plain steps of the
    kernel variant without a cache; the same bits as with a contiguous V, within tolerance of the oracle."""
    from oracle import attention as oat
    B, L, hq, hkv, hd = 2, 1280, 14, 2, 128
    g = torch.Generator().manual_seed(23)
    q = torch.randn(B * L, hq, hd, generator=g).to(torch.bfloat16)
    k = torch.randn(B * L, hkv, hd, generator=g).to(torch.bfloat16)
    v = torch.randn(B * L, hkv, hd, generator=g).to(torch.bfloat16)
    cu = torch.arange(0, B * L + 1, L, dtype=torch.int32)
    want = oat.paged_attention_fp32(q, k, v, None, None, None, None, cu, cu, hd ** -0.5, mask_mode=mask, dbs=32)
    qkv = torch.zeros(B * L, (hq + 2 * hkv) * hd, dtype=torch.bfloat16, device=dev)
    v_view = qkv[:, (hq + hkv) * hd:].view(B * L, hkv, hd)
    v_view.copy_(v)
    assert v_view.stride(0) != k.stride(0) and v_view.stride(1) == k.stride(1)
    kw = dict(block_tables=None, context_lens=None, cu_seqlens_q=cu.to(dev), cu_seqlens_new=cu.to(dev), max_seqlen_q=L,
              mask_mode=mask, diffusion_block_size=32)
    for max_wg in (0, 3):
        ref = dfx.paged_attention(q.to(dev), k.to(dev), v.to(dev), None, None, hd ** -0.5, max_workgroups=max_wg, **kw)
        got = dfx.paged_attention(q.to(dev), k.to(dev), v_view, None, None, hd ** -0.5, max_workgroups=max_wg, **kw)
        torch.cuda.synchronize()
        assert torch.equal(got, ref)
        assert max_abs_err(got, want) <= ATOL_BF16


# the shapes of the reference's prefill kernel tests (tests/python/kernel/test_dllm_flash_attn_prefill_kernel.py
# :162-310): (sequences, query heads, KV heads, head_dim, length, block attention, diffusion block size)
REF_PREFILL_CASES = [
    (1, 32, 8, 128, 192, False, 32), (4, 32, 8, 128, 256, False, 32), (2, 32, 8, 128, 256, True, 32),
    (3, 32, 8, 128, 320, True, 32), (2, 32, 8, 128, 256, True, 64), (2, 32, 4, 128, 192, False, 32),
    (2, 32, 4, 128, 256, True, 32), (2, 32, 8, 64, 192, False, 32),
]


@pytest.mark.parametrize("case", REF_PREFILL_CASES)
def test_reference_prefill_test_shapes(dev, case):
    """Through the operator, against the fp32 oracle; the reference compares with atol = rtol = 1e-2."""
    from oracle import attention as oat
    B, hq, hkv, hd, L, block_attn, dbs = case
    g = torch.Generator().manual_seed(B * 1000 + L + dbs)
    q = torch.randn(B * L, hq, hd, generator=g).to(torch.bfloat16)
    k = torch.randn(B * L, hkv, hd, generator=g).to(torch.bfloat16)
    v = torch.randn(B * L, hkv, hd, generator=g).to(torch.bfloat16)
    cu = torch.arange(0, (B + 1) * L, L, dtype=torch.int32)
    scale = 1.0 / (hd ** 0.5)
    mask = MASK_BLOCK_CAUSAL if block_attn else MASK_FULL
    want = oat.paged_attention_fp32(q, k, v, None, None, None, None, cu, cu, scale, mask_mode=mask, dbs=dbs)
    md = dfx.PagedAttnMetaData(is_prefill=True, cu_seqlens_q=cu.to(dev), cu_seqlens_k=cu.to(dev), max_seqlen_q=L,
                               max_seqlen_k=L, attn_type="block_attention" if block_attn else "full_attention",
                               diffusion_block_size=dbs)
    got = dfx.dllm_flash_attn_prefill(q.to(dev), k.to(dev), v.to(dev), scale, md)
    torch.cuda.synchronize()
    assert got.shape == q.shape and got.dtype == torch.bfloat16
    assert max_abs_err(got, want) <= 1e-2


@pytest.mark.parametrize("flags", PATHS)
def test_block_causal_long_queries_on_an_fp8_cache(dev, flags):
    wl = make_workload("c5", seed=33, num_seqs=2, h_q=8, h_kv=2, q_len=512, ctx=[700, 130], mask=MASK_BLOCK_CAUSAL)
    want = oracle_fp32(wl)
    for max_wg in (0, 7):
        got = _run(wl.to(dev), max_workgroups=max_wg, flags=flags)
        assert max_abs_err(got, want) <= ATOL_FP8


def _random_case(rng):
    """A random but valid attention problem: shapes the operators accept, drawn from a seeded generator."""
    hd = int(rng.choice([64, 128]))
    h_kv = int(rng.choice([1, 2, 4, 8]))
    group = int(rng.choice([1, 2, 4, 7, 8]))
    page = int(rng.choice([16, 32, 48, 64, 256, 24, 1]))     # 24 and 1: pages the streaming path does not take
    dbs = int(rng.choice([16, 32, 64]))
    q_len = int(rng.choice([dbs, 2 * dbs, 3 * dbs, 8 * dbs]))
    b = int(rng.integers(1, 7))
    ctx = [int(x) for x in rng.choice([0, 1, 15, 63, 64, 65, 200, 511, 777], b)]
    mask = MASK_BLOCK_CAUSAL if rng.random() < 0.5 else MASK_FULL
    fp8 = bool(rng.random() < 0.3)
    return dict(num_seqs=b, h_q=h_kv * group, h_kv=h_kv, hd=hd, page=page, ctx=ctx, q_len=q_len, dbs=dbs, mask=mask), fp8


@pytest.mark.parametrize("seed", range(40))
def test_random_shapes_against_oracle(dev, seed):
    rng = np.random.default_rng(1000 + seed)
    over, fp8 = _random_case(rng)
    wl = make_workload("c5" if fp8 else "c1", seed=seed, **over)
    want = oracle_fp32(wl)
    tol = ATOL_FP8 if fp8 else ATOL_BF16
    g = wl.to(dev)
    for max_wg in (0, int(rng.integers(1, 40))):
        for flags in PATHS:
            got = _run(g, max_workgroups=max_wg, flags=flags)
            assert torch.isfinite(got.float()).all(), (over, fp8, max_wg, flags)
            assert max_abs_err(got, want) <= tol, (over, fp8, max_wg, flags)


@pytest.mark.parametrize("flags", PATHS)
def test_non_finite_inputs_stay_inside_their_sequence(dev, flags):
    """A NaN in one sequence's cached V and an infinity in another's fresh K make those sequences'
    rows non-finite (as in the oracle) and leave every other sequence exactly as without them,
    whatever the partition."""
    wl = make_workload("c3", seed=51, num_seqs=5, ctx=(300, 900))
    g = wl.to(dev)
    clean = {mw: _run(g, max_workgroups=mw, flags=flags) for mw in (0, 9)}
    page = int(wl.block_tables[1, 0])
    g.v_cache[page, 3, 1, 17] = float("nan")                   # sequence 1, context token 3
    t3 = int(wl.cu_seqlens_q[3])
    g.k_new[t3 + 5, 2, 40] = float("inf")                      # sequence 3, fresh token 5
    cu = wl.cu_seqlens_q.tolist()
    for mw in (0, 9):
        got = _run(g, max_workgroups=mw, flags=flags)
        for s in range(wl.num_seqs):
            rows = slice(cu[s], cu[s + 1])
            if s in (1, 3):
                assert not torch.isfinite(got[rows].float()).all()
            else:
                assert torch.equal(got[rows], clean[mw][rows])


# ---- launch plans (dfx_paged_attn_plan) ---------------------------------------------------------------
PLAN_CASES = [
    ("c3", {}),                                              # 256 items on 256 workgroups: pairing applies
    ("c3", dict(num_seqs=5, ctx=(200, 700))),                # fewer items than workgroups
    ("c3", dict(num_seqs=9, ctx=[64, 3000, 100, 2500, 700, 650, 1, 0, 4096])),
    ("c3", dict(num_seqs=70, ctx=(100, 900))),               # more items than workgroups: equal ranges
    ("c4", dict(num_seqs=3, ctx=(100, 500))),                # compact kernel, block-causal
    ("c5", dict(num_seqs=4, ctx=(200, 900))),                # FP8 streaming kernel
    ("c1", {}),                                              # head_dim 64
    ("c3", dict(num_seqs=12, ctx=(50, 1200), hd=64)),        # head_dim 64 with 224 rows: the pipelined kernel's narrow variant, cut items
    ("c3", dict(num_seqs=5, ctx=[0, 1, 63, 64, 700], hd=64, page=16)),
]


def _read_plan(plan, num_seqs, n_wg):
    """Header and per-workgroup work of a plan buffer (layout: csrc/plan.h)."""
    raw = plan.cpu().numpy()
    hdr = raw[:64].view(np.int32)
    bounds_off = (64 + (num_seqs + 1) * 4 + 63) // 64 * 64
    work_off = (bounds_off + (n_wg + 1) * 4 + 63) // 64 * 64
    work = raw[work_off:work_off + n_wg * 64].reshape(n_wg, 64)   # WgWork: 64-byte records
    ranges = work[:, :32].copy().view(np.int64).reshape(n_wg, 4)
    partner = work[:, 32:36].copy().view(np.int32).reshape(n_wg)
    bounds = raw[bounds_off:bounds_off + (n_wg + 1) * 4].copy().view(np.int32)
    return dict(magic=int(hdr[0]) & 0xffffffff, n_active=int(hdr[2]), mode=int(hdr[3]), per_head=int(hdr[4]),
                total=int(hdr[5]), critical=int(hdr[7]), reordered=int(hdr[8]), bounds=bounds), ranges, partner


@pytest.mark.parametrize("name,over", PLAN_CASES)
@pytest.mark.parametrize("max_wg", [0, 7])
def test_planned_launch_with_equal_ranges_gives_the_same_bits(dev, name, over, max_wg, monkeypatch):
    """With equal ranges the plan describes the partition the kernels work out for themselves:
    reading it must not change a bit."""
    monkeypatch.setattr(dfa, "PLAN_MIN_UNITS_PER_WORKGROUP", 0)   # (plan the tiny cases too)
    wl = make_workload(name, device=dev, **over)
    want = _run(wl, max_wg)
    cache = {}
    for _ in range(2):   # the second call reuses the plan
        got = _run(wl, max_wg, plan_cache=cache, flags=_lib.DFX_ATTN_EQUAL_RANGES)
        assert torch.equal(got, want)
    assert len(cache) == 1 and next(iter(cache.values())) is not None


@pytest.mark.parametrize("name,over", PLAN_CASES + [("c3", dict(num_seqs=40, ctx=(64, 1500))),
                                                    ("c3", dict(num_seqs=24, ctx=[70] * 12 + [2900] * 12))])
@pytest.mark.parametrize("max_wg", [0, 7, 40])
def test_planned_launch_with_cut_points_placed_by_cost(dev, name, over, max_wg, monkeypatch):
    """The default plan: ranges of equal cost, cut points moved onto a sequence's first unit where one is
    near.  Other pieces are merged than without a plan, so the rows differ in the last bits only;
    every launch with the plan gives the same bits; the ranges tile the unit space."""
    monkeypatch.setattr(dfa, "PLAN_MIN_UNITS_PER_WORKGROUP", 0)   # (plan the tiny cases too)
    wl = make_workload(name, device=dev, **over)
    cache = {}
    got = _run(wl, max_wg, plan_cache=cache)
    tol = ATOL_FP8 if wl.kv_fp8 else ATOL_BF16
    if wl.num_seqs <= 16:
        assert max_abs_err(got, oracle_fp32(wl)) <= tol
    else:   # the oracle on a sample: first, last and two sequences in between
        seqs = sorted({0, wl.num_seqs // 3, 2 * wl.num_seqs // 3, wl.num_seqs - 1})
        cu = wl.cu_seqlens_q.tolist()
        for s, want in zip(seqs, oracle_fp32(wl, seqs=seqs)):
            assert max_abs_err(got[cu[s]:cu[s + 1]], want) <= tol, f"sequence {s}"
    assert max_abs_err(got, _run(wl, max_wg)) <= 1e-2
    assert torch.equal(_run(wl, max_wg, plan_cache=cache), got)
    plan = next(iter(cache.values()))
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    ok = False
    for n_wg in ([max_wg, 2 * max_wg] if max_wg else [cus, 2 * cus]):   # (two workgroups per compute unit for the small shapes)
        hdr, ranges, _ = _read_plan(plan, wl.num_seqs, n_wg)
        assert hdr["magic"] == 0x44465850 and hdr["mode"] in (0, 2)
        spans = [(int(r[0]), int(r[1])) for r in ranges[:hdr["n_active"]]]
        if not (spans and spans[0][0] == 0 and spans[-1][1] == hdr["total"]):
            continue
        ok = True
        assert all(x[1] == y[0] for x, y in zip(spans, spans[1:])), (hdr, spans)
        if hdr["mode"] == 2:
            assert all(b >= a for a, b in spans), (hdr, spans)   # (the sweep may leave a workgroup without units)
            assert [a for a, _ in spans] + [hdr["total"]] == hdr["bounds"][:hdr["n_active"] + 1].tolist()
            assert hdr["total"] >= 8 * hdr["n_active"]
        break
    assert ok


@pytest.mark.parametrize("name,over", PLAN_CASES)
def test_planned_launch_with_the_pairing_partition(dev, name, over):
    wl = make_workload(name, device=dev, **over)
    cache = {}
    got = _run(wl, plan_cache=cache, flags=_lib.DFX_ATTN_PAIRING)
    tol = ATOL_FP8 if wl.kv_fp8 else ATOL_BF16
    if wl.num_seqs <= 16:
        assert max_abs_err(got, oracle_fp32(wl)) <= tol
    assert max_abs_err(got, _run(wl)) <= 1e-2
    again = _run(wl, plan_cache=cache, flags=_lib.DFX_ATTN_PAIRING)
    assert torch.equal(again, got)


def test_pairing_plan_covers_every_unit_once_at_c3(dev):
    """The plan of the headline workload: pairing partition, every unit of the linear unit space in
    exactly one workgroup's ranges, donated pieces in front of the partner's own item."""
    wl = make_workload("c3", device=dev)
    cache = {}
    got = _run(wl, plan_cache=cache, flags=_lib.DFX_ATTN_PAIRING)
    torch.cuda.synchronize()
    n_wg = torch.cuda.get_device_properties(dev).multi_processor_count
    hdr, ranges, partner = _read_plan(next(iter(cache.values())), wl.num_seqs, n_wg)
    assert hdr["magic"] == 0x44465850 and hdr["mode"] == 1 and hdr["n_active"] == n_wg
    tiles = sum((int(c) + 63) // 64 + 1 for c in wl.context_lens.tolist())
    assert hdr["per_head"] == tiles and hdr["total"] == tiles * wl.num_kv_heads
    spans = sorted((int(a), int(b)) for r in ranges for a, b in ((r[0], r[1]), (r[2], r[3])) if b > a)
    assert spans[0][0] == 0 and spans[-1][1] == hdr["total"]
    assert all(x[1] == y[0] for x, y in zip(spans, spans[1:]))
    loads = [(r[1] - r[0]) + (r[3] - r[2]) for r in ranges]
    assert max(loads) <= hdr["critical"] and hdr["critical"] <= -(-hdr["total"] // n_wg) + 6
    cut = [w for w in range(n_wg) if partner[w] >= 0]
    assert all(partner[partner[w]] == w for w in cut) and 0 < len(cut) < n_wg
    cu = wl.cu_seqlens_q.tolist()
    for s, want in zip([0, 63], oracle_fp32(wl, seqs=[0, 63])):
        assert max_abs_err(got[cu[s]:cu[s + 1]], want) <= ATOL_BF16


def test_plan_with_1024_workgroups(dev):
    """The largest grid the plan places cut points for: its table of 1025 cut points fills the
    plan kernel's array to the last word."""
    wl = make_workload("c3", device=dev, num_seqs=128, ctx=(2048, 8192), seed=12)
    cache = {}
    got = _run(wl, 1024, plan_cache=cache)
    hdr, ranges, _ = _read_plan(next(iter(cache.values())), wl.num_seqs, 1024)
    assert hdr["magic"] == 0x44465850 and hdr["mode"] == 2 and hdr["n_active"] == 1024
    spans = [(int(r[0]), int(r[1])) for r in ranges]
    assert spans[0][0] == 0 and spans[-1][1] == hdr["total"]
    assert all(x[1] == y[0] for x, y in zip(spans, spans[1:])) and all(b >= a for a, b in spans)
    assert [a for a, _ in spans] + [hdr["total"]] == hdr["bounds"][:1025].tolist()
    assert torch.equal(_run(wl, 1024, plan_cache=cache), got)
    seqs = [0, 77, 127]
    cu = wl.cu_seqlens_q.tolist()
    for s, want in zip(seqs, oracle_fp32(wl, seqs=seqs)):
        assert max_abs_err(got[cu[s]:cu[s + 1]], want) <= ATOL_BF16


def test_stale_plan_after_offsets_shrank_in_place_stays_inside_the_tensors(dev):
    """A C-ABI caller that rewrites cu_seqlens in place and reuses the plan gets wrong rows (its
    contract), but nothing outside q / out is touched: rows the plan names beyond num_q_tokens are
    neither read nor written."""
    wl = make_workload("c3", device=dev, num_seqs=6, ctx=(300, 900), seed=5)
    cache = {}
    _run(wl, plan_cache=cache)
    plan = next(iter(cache.values()))
    t_small = 4 * wl.q_len                                   # the batch shrinks to 4 sequences' rows ...
    cu_small = wl.cu_seqlens_q.clone()
    cu_small[5:] = t_small                                   # ... in a tensor of the same size (the last two have none)
    wl.cu_seqlens_q.copy_(cu_small)                          # in place: same address, the plan's signature still matches
    guard = torch.full((wl.q.shape[0], wl.num_q_heads, wl.head_dim), 7.0, dtype=torch.bfloat16, device=dev)
    out = guard[:t_small]
    key = next(iter(cache))
    stale = {key: plan}
    import diffulex_amd.dllm_flash_attn as dfa
    orig = dfa.plan_key
    dfa.plan_key = lambda *a, **k: key                       # (what a caller that bypasses PyTorch's version counters sees)
    try:
        dfx.paged_attention(wl.q[:t_small], wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, out=out,
                            block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
                            cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len, plan_cache=stale)
        torch.cuda.synchronize()
    finally:
        dfa.plan_key = orig
    assert bool((guard[t_small:] == 7.0).all()), "rows beyond num_q_tokens were written"


def test_plan_made_for_another_configuration_is_ignored(dev):
    """A stale or foreign plan must never be followed: the kernels compare its signature with their
    own launch and plan for themselves."""
    wl = make_workload("c3", device=dev, num_seqs=6, ctx=(300, 900))
    other = make_workload("c3", device=dev, num_seqs=6, ctx=(1000, 1500), seed=9)
    cache = {}
    _run(other, plan_cache=cache)
    plan = next(iter(cache.values()))
    want = _run(wl)
    # hand the foreign plan to a launch with other metadata tensors (different signature)
    p_cache = {}
    out = _run(wl, plan_cache=p_cache)
    key = next(iter(p_cache))
    p_cache[key] = plan
    got2 = _run(wl, plan_cache=p_cache)
    assert max_abs_err(got2, want) <= 1e-2 and torch.equal(got2, want)
    assert max_abs_err(out, want) <= 1e-2


def test_a_launch_of_a_few_tiles_is_not_planned(dev):
    """The operators skip the plan where a launch has at most a tile or two per workgroup (the plan kernels
    would take longer than they save); the launch plans for itself then, as without a plan cache."""
    wl = make_workload("c1", device=dev)
    cache = {}
    got = _run(wl, plan_cache=cache)
    assert list(cache.values()) == [None]
    assert torch.equal(got, _run(wl))
    assert max_abs_err(got, oracle_fp32(wl)) <= ATOL_BF16


def test_distinct_layout_in_a_captured_graph_and_through_the_static_entry(dev):
    """The distinct layout's streaming kernel the ways a serving loop reaches it: Attention.forward captured in a
    graph and replayed (the plan built inside the capture, eager launches between the replays), and the entry point
    that allocates nothing."""
    wl = make_workload("c3", num_seqs=6, ctx=(300, 1200), seed=45).to(dev)
    want = oracle_fp32(wl)
    att = dfx.Attention(wl.num_q_heads, wl.head_dim, wl.scale, wl.num_kv_heads)
    att.k_cache, att.v_cache = _to_distinct(wl.k_cache)[0], _to_distinct(wl.v_cache)[1]
    md = metadata_for(wl, "static")
    md.kv_cache_layout = "distinct"
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    t = wl.q.shape[0]
    q, k, v = (x.reshape(t, -1).clone() for x in (wl.q, wl.k_new, wl.v_new))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        eager = att(q, k, v)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert max_abs_err(eager.view(t, wl.num_q_heads, wl.head_dim), want) <= ATOL_BF16
    kc0, vc0 = att.k_cache.clone(), att.v_cache.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        o_static = att(q, k, v)
    for _ in range(3):
        graph.replay()
        att(q, k, v)               # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(o_static, eager)
    assert torch.equal(att.k_cache, kc0) and torch.equal(att.v_cache, vc0)   # (the same block stored again)
    out = torch.empty_like(wl.q)
    got = dfx.paged_attention(wl.q, wl.k_new, wl.v_new, att.k_cache, att.v_cache, wl.scale, out=out, static_scratch=True,
                              cache_layout="distinct", block_tables=wl.block_tables, context_lens=wl.context_lens,
                              cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len,
                              mask_mode=wl.mask_mode, diffusion_block_size=wl.diffusion_block_size)
    torch.cuda.synchronize()
    assert max_abs_err(got, want) <= ATOL_BF16


@pytest.mark.parametrize("ctx", [[0, 0, 700, 0, 64], [900, 5, 5, 5, 900, 5], [64, 64]])
def test_reordered_plan_with_sequences_of_no_or_few_tiles(dev, ctx):
    """The plan's second order of the sequences (k-th longest, k-th shortest) on batches whose short sequences have
    no context at all, or are all alike, or are too few for a second order: the same rows as the batch's order up to
    the rounding of other merges, and as the oracle."""
    wl = make_workload("c3", num_seqs=len(ctx), ctx=ctx, seed=47).to(dev)
    want = oracle_fp32(wl)
    for max_wg in (0, 6):
        got = _run(wl, max_wg, plan_cache={})
        kept = _run(wl, max_wg, plan_cache={}, flags=_lib.DFX_ATTN_BATCH_ORDER)
        torch.cuda.synchronize()
        assert max_abs_err(got, want) <= ATOL_BF16
        assert max_abs_err(got, kept) <= 1e-2


def test_step_microbenchmark_runs(dev):
    """diffulex_amd/build/step_bench (csrc/step_bench.hip): the generated step on LDS-resident tiles.  A step holds
    2048 cycles of matrix instructions per SIMD; whatever the schedule, it cannot be faster, and a step beyond
    twice that would mean the blocks no longer overlap anything."""
    import re
    import subprocess
    from diffulex_amd import build as dbuild
    if not dbuild.STEP_BENCH_PATH.exists():
        pytest.skip("diffulex_amd/build/step_bench has not been built (python -m diffulex_amd.build): a measuring tool, not part of the library")
    out = subprocess.run([str(dbuild.STEP_BENCH_PATH), "200"], capture_output=True, text=True, timeout=100)
    assert out.returncode == 0, out.stdout + out.stderr
    rows = re.findall(r"^(.+?)\s+(\d+) workgroups\s+tile loads (\w+)\s+(\d+) cycles/step", out.stdout, re.M)
    assert len(rows) == 10, out.stdout
    for name, _, _, cycles in rows:
        lo, hi = {"the step": (2048, 4096), "matrix instructions only": (2048, 3000)}.get(name.strip(), (500, 2500))
        assert lo <= int(cycles) <= hi, (name, cycles)
