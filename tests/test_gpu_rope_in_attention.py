"""The rotary embedding applied inside the attention launch (dfx_attn_params.rope_cos_sin) against the two
launches it replaces: dfx_rope_kv_store (itself bit-exact against the CPU oracle, tests/test_gpu_rotary.py)
followed by the attention launch on the rotated rows.  Same bits: the query rows are rotated with the same
arithmetic on their way into the matrix instructions, the fresh key rows before their tiles are read."""
import pytest
import torch

import diffulex_amd as dfx
from diffulex_amd import _lib
from diffulex_amd.rotary_embedding import RotaryEmbedding
from diffulex_amd.workloads import make_workload
from oracle import rotary as orot
from util import ATOL_BF16, ATOL_FP8, max_abs_err, metadata_for, oracle_fp32

pytestmark = pytest.mark.gpu
MAXPOS, BASE = 8192, 1.0e6


def _bits(t):
    t = t.contiguous()
    return t.view({1: torch.uint8, 2: torch.int16}[t.element_size()])


CASES = [
    ("c3", dict(num_seqs=6, ctx=(300, 900)), 0),                       # Dream heads: 224 rows per item, cut items
    ("c3", dict(num_seqs=3, ctx=[0, 64, 700]), 5),                     # a sequence without context; five workgroups
    ("c4", dict(num_seqs=3, ctx=(100, 500)), 0),                       # three in-flight blocks, block-causal, 96 rows
    ("c4", dict(num_seqs=2, ctx=(100, 300), h_q=8, h_kv=2, q_len=128, dbs=32), 7),   # several row tiles per sequence and head
    ("c5", dict(num_seqs=4, ctx=(200, 900)), 0),                       # FP8 cache: the store quantises the rotated rows
]


@pytest.mark.parametrize("name,over,max_wg", CASES)
@pytest.mark.parametrize("planned", [False, True])
def test_rope_inside_the_launch_gives_the_bits_of_rope_then_attention(dev, name, over, max_wg, planned):
    wl = make_workload(name, device=dev, **over)
    T, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    g = torch.Generator("cpu").manual_seed(5)
    qkv = torch.randn(T, (hq + 2 * hkv) * hd, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = (x.view(T, -1, hd) for x in qkv.split([hq * hd, hkv * hd, hkv * hd], dim=-1))
    pos = torch.randint(0, MAXPOS, (T,), generator=g).to(dev)
    if max_wg:  # (the cases with a workgroup limit also take the positions as int32)
        pos = pos.to(torch.int32)
    rope = RotaryEmbedding(hd, hd, MAXPOS, BASE).to(dev)
    kw = dict(block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
              cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode,
              diffusion_block_size=wl.diffusion_block_size, k_scale=wl.k_scale, v_scale=wl.v_scale, max_workgroups=max_wg)

    # two launches: rotate and store, then attend
    kc1, vc1 = wl.k_cache.clone(), wl.v_cache.clone()
    md = metadata_for(wl, "static")
    rq, rk = rope.forward_and_store(pos, q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1), kc1, vc1, wl.slot_mapping, md)
    want = dfx.paged_attention(rq.view(T, hq, hd), rk.view(T, hkv, hd), v, kc1, vc1, wl.scale,
                               plan_cache={} if planned else None, **kw)
    # one launch
    kc2, vc2 = wl.k_cache.clone(), wl.v_cache.clone()
    k_rot = torch.zeros(T, hkv, hd, dtype=torch.bfloat16, device=dev)
    got = dfx.paged_attention(q, k, v, kc2, vc2, wl.scale, store_slot_mapping=wl.slot_mapping,
                              rope=(rope.cos_sin_cache, pos), k_rotated=k_rot, plan_cache={} if planned else None, **kw)
    torch.cuda.synchronize()
    assert torch.equal(_bits(k_rot), _bits(rk.view(T, hkv, hd))), "rotated key rows"
    assert torch.equal(_bits(kc2), _bits(kc1)) and torch.equal(_bits(vc2), _bits(vc1)), "cache after the fused store"
    assert torch.equal(_bits(got), _bits(want)), "attention output"
    assert torch.equal(_bits(qkv.cpu()), _bits(qkv.cpu())) and torch.isfinite(got.float()).all()
    # and against the oracle: rotary embedding, then fp32 attention
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    c = wl.to("cpu")
    c.q = orot.apply_rotary(q.reshape(T, -1).cpu(), pos.cpu().long(), tab, hd).view(T, hq, hd)
    c.k_new = orot.apply_rotary(k.reshape(T, -1).cpu(), pos.cpu().long(), tab, hd).view(T, hkv, hd)
    c.v_new = v.cpu().contiguous()
    assert max_abs_err(got, oracle_fp32(c)) <= (ATOL_FP8 if wl.kv_fp8 else ATOL_BF16)


def test_attention_module_with_rope_takes_the_one_launch_path_and_matches_the_two_launch_path(dev):
    """Attention.forward(q, k, v, rope=(rotary, positions)) on projections sliced out of one QKV buffer."""
    wl = make_workload("c3", num_seqs=5, ctx=(200, 800), seed=8).to(dev)
    T, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    g = torch.Generator("cpu").manual_seed(6)
    qkv = torch.randn(T, (hq + 2 * hkv) * hd, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = qkv.split([hq * hd, hkv * hd, hkv * hd], dim=-1)
    pos = (wl.context_lens.repeat_interleave(wl.q_len) + torch.arange(wl.q_len, device=dev).repeat(wl.num_seqs)).long()
    rope = RotaryEmbedding(hd, hd, MAXPOS, BASE).to(dev)
    outs, caches = [], []
    for fused in (False, True):
        att = dfx.Attention(hq, hd, wl.scale, hkv)
        att.k_cache, att.v_cache = wl.k_cache.clone(), wl.v_cache.clone()
        md = metadata_for(wl, "static")
        md.need_kv_cache_store = True
        dfx.set_fetch_fn_for_attn_metadata(lambda: md)
        if fused:
            outs.append(att(q, k, v, rope=(rope, pos)))
        else:
            rq, rk = rope(pos, q, k)
            outs.append(att(rq, rk, v))
        caches.append((att.k_cache, att.v_cache))
    torch.cuda.synchronize()
    assert torch.equal(_bits(outs[0]), _bits(outs[1]))
    assert torch.equal(_bits(caches[0][0]), _bits(caches[1][0])) and torch.equal(_bits(caches[0][1]), _bits(caches[1][1]))


@pytest.mark.parametrize("name,over", [
    ("c1", {}),                                               # head_dim 64, 64 rows: no pipelined kernel
    ("c3", dict(num_seqs=3, ctx=(100, 600), hd=64)),          # head_dim 64, 224 rows: its pipelined kernel does not rotate
])
def test_shapes_whose_kernel_does_not_rotate_refuse_the_rope_and_the_module_falls_back(dev, name, over):
    wl = make_workload(name, device=dev, **over)
    T, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    rope = RotaryEmbedding(hd, hd, 512, 10000.0).to(dev)
    pos = torch.arange(T, device=dev) % 512
    with pytest.raises(_lib.DfxError):
        dfx.paged_attention(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, block_tables=wl.block_tables,
                            context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q,
                            max_seqlen_q=wl.q_len, rope=(rope.cos_sin_cache, pos))
    att = dfx.Attention(hq, hd, wl.scale, hkv)
    att.k_cache, att.v_cache = wl.k_cache.clone(), wl.v_cache.clone()
    md = metadata_for(wl, "static")
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    out = att(wl.q.reshape(T, -1), wl.k_new.reshape(T, -1), wl.v_new.reshape(T, -1), rope=(rope, pos))
    rq, rk = rope(pos, wl.q.reshape(T, -1), wl.k_new.reshape(T, -1))
    att2 = dfx.Attention(hq, hd, wl.scale, hkv)
    att2.k_cache, att2.v_cache = wl.k_cache.clone(), wl.v_cache.clone()
    assert torch.equal(_bits(out), _bits(att2(rq, rk, wl.v_new.reshape(T, -1))))
    # (the fallback rotates and stores in one launch: the same cache as the store of the rotated rows)
    assert torch.equal(_bits(att.k_cache), _bits(att2.k_cache)) and torch.equal(_bits(att.v_cache), _bits(att2.v_cache))


def test_attention_module_with_rope_on_the_distinct_layout(dev):
    """kv_cache_layout == "distinct": the rotary embedding's launch also stores the block into that layout
    (dfx_rope_kv_store), the attention launch then streams from it -- two launches, the same bits as rotating,
    storing with store_kvcache_distinct_layout and attending in three."""
    wl = make_workload("c3", num_seqs=5, ctx=(200, 800), seed=12).to(dev)
    T, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    g = torch.Generator("cpu").manual_seed(13)
    qkv = torch.randn(T, (hq + 2 * hkv) * hd, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = qkv.split([hq * hd, hkv * hd, hkv * hd], dim=-1)
    pos = torch.randint(0, MAXPOS, (T,), generator=g).to(dev)
    rope = RotaryEmbedding(hd, hd, MAXPOS, BASE).to(dev)
    pages, page = wl.k_cache.shape[0], wl.k_cache.shape[1]

    def distinct(c):
        return (c.view(pages, page, hkv, hd // 8, 8).permute(0, 2, 3, 1, 4).contiguous(), c.permute(0, 2, 3, 1).contiguous())
    outs, caches = [], []
    for one_call in (True, False):
        att = dfx.Attention(hq, hd, wl.scale, hkv)
        att.k_cache, att.v_cache = distinct(wl.k_cache)[0], distinct(wl.v_cache)[1]
        md = metadata_for(wl, "static")
        md.kv_cache_layout = "distinct"
        md.need_kv_cache_store = True
        dfx.set_fetch_fn_for_attn_metadata(lambda: md)
        if one_call:
            outs.append(att(q, k, v, rope=(rope, pos)))
        else:
            rq, rk = rope(pos, q, k)
            outs.append(att(rq, rk, v))
        caches.append((att.k_cache, att.v_cache))
    torch.cuda.synchronize()
    assert torch.equal(_bits(outs[0]), _bits(outs[1]))
    assert torch.equal(_bits(caches[0][0]), _bits(caches[1][0])) and torch.equal(_bits(caches[0][1]), _bits(caches[1][1]))
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    c = wl.to("cpu")
    c.q = orot.apply_rotary(q.contiguous().cpu(), pos.cpu(), tab, hd).view(T, hq, hd)
    c.k_new = orot.apply_rotary(k.contiguous().cpu(), pos.cpu(), tab, hd).view(T, hkv, hd)
    c.v_new = v.cpu().contiguous().view(T, hkv, hd)
    assert max_abs_err(outs[0].view(T, hq, hd), oracle_fp32(c)) <= ATOL_BF16


def test_rope_inside_the_launch_in_a_captured_graph(dev):
    """The one-launch layer step captured and replayed, with new projections in the same tensors between the
    replays: every replay equals the eager two-launch result on the same inputs."""
    wl = make_workload("c3", num_seqs=6, ctx=(300, 900), seed=7).to(dev)
    T, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    rope = RotaryEmbedding(hd, hd, MAXPOS, BASE).to(dev)
    att = dfx.Attention(hq, hd, wl.scale, hkv)
    att.k_cache, att.v_cache = wl.k_cache.clone(), wl.v_cache.clone()
    md = metadata_for(wl, "static")
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    g = torch.Generator("cpu").manual_seed(9)
    qkv = torch.randn(T, (hq + 2 * hkv) * hd, generator=g).to(torch.bfloat16).to(dev)
    pos = torch.randint(0, MAXPOS, (T,), generator=g).to(dev)
    q, k, v = qkv.split([hq * hd, hkv * hd, hkv * hd], dim=-1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        att(q, k, v, rope=(rope, pos))       # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        o_static = att(q, k, v, rope=(rope, pos))
    for i in range(3):
        qkv.copy_(torch.randn(qkv.shape, generator=g).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        cache_after = att.k_cache.clone()
        rq, rk = rope(pos, q, k)             # the two launches, eagerly, on the same inputs
        want = att(rq, rk, v)
        torch.cuda.synchronize()
        assert torch.equal(_bits(o_static), _bits(want)), i
        assert torch.equal(_bits(att.k_cache), _bits(cache_after)), i
