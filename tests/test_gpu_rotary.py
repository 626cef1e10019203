"""GPU parity of the rotary-embedding kernel (and its fused KV-cache store) against the CPU
oracle: bit-exact, through the C ABI."""
import ctypes as C

import pytest
import torch

from diffulex_amd import _lib
from diffulex_amd.rotary_embedding import RotaryEmbedding, get_rope
from oracle import kv_cache as okv
from oracle import rotary as orot

pytestmark = pytest.mark.gpu
MAXPOS, BASE = 8192, 1.0e6


def _bits(t):
    t = t.cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16}[t.element_size()])


def _inputs(T, Hq, Hkv, hd, seed, pos_dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * hd, generator=g).to(torch.bfloat16)
    pos = torch.randint(0, MAXPOS, (T,), generator=g).to(pos_dtype)
    return qkv, pos


def _rope(hd, dev):
    rope = RotaryEmbedding(hd, hd, MAXPOS, BASE).to(dev)
    assert torch.equal(rope.cos_sin_cache.cpu(), orot.cos_sin_cache(hd, MAXPOS, BASE))
    return rope


@pytest.mark.parametrize("T,Hq,Hkv,hd", [(2048, 28, 4, 128), (96, 4, 2, 64), (1, 1, 1, 16), (77, 32, 32, 128)])
@pytest.mark.parametrize("pos_dtype", [torch.int64, torch.int32])
def test_forward_bit_exact_on_split_projection_views(dev, T, Hq, Hkv, hd, pos_dtype):
    """query / key are column slices of one projection output (row stride larger than the row)."""
    qkv, pos = _inputs(T, Hq, Hkv, hd, seed=T + hd, pos_dtype=pos_dtype)
    q, k = qkv[:, :Hq * hd], qkv[:, Hq * hd:(Hq + Hkv) * hd]
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    want_q, want_k = orot.apply_rotary(q, pos, tab, hd), orot.apply_rotary(k, pos, tab, hd)
    rope = _rope(hd, dev)
    gq = qkv.to(dev)
    got_q, got_k = rope(pos.to(dev), gq[:, :Hq * hd], gq[:, Hq * hd:(Hq + Hkv) * hd])
    torch.cuda.synchronize()
    assert got_q.shape == q.shape and got_k.shape == k.shape and got_q.is_contiguous()
    assert torch.equal(_bits(got_q), _bits(want_q))
    assert torch.equal(_bits(got_k), _bits(want_k))
    assert torch.equal(_bits(gq), _bits(qkv)), "inputs must stay untouched"


def test_three_dimensional_inputs_and_cached_constructor(dev):
    T, Hq, Hkv, hd = 40, 6, 2, 128
    qkv, pos = _inputs(T, Hq, Hkv, hd, seed=9)
    q = qkv[:, :Hq * hd].contiguous().view(T, Hq, hd)
    k = qkv[:, Hq * hd:(Hq + Hkv) * hd].contiguous().view(T, Hkv, hd)
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    rope = get_rope(hd, hd, MAXPOS, BASE).to(dev)
    assert get_rope(hd, hd, MAXPOS, BASE) is rope
    got_q, got_k = rope(pos.to(dev), q.to(dev), k.to(dev))
    torch.cuda.synchronize()
    assert got_q.shape == (T, Hq, hd)
    assert torch.equal(_bits(got_q), _bits(orot.apply_rotary(q, pos, tab, hd)))
    assert torch.equal(_bits(got_k), _bits(orot.apply_rotary(k, pos, tab, hd)))


def test_in_place_through_the_c_abi(dev):
    """q_out == q and k_out == k: every lane reads its two chunks before it writes them."""
    T, Hq, Hkv, hd = 64, 8, 2, 128
    qkv, pos = _inputs(T, Hq, Hkv, hd, seed=4)
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    want = qkv.clone()
    want[:, :Hq * hd] = orot.apply_rotary(qkv[:, :Hq * hd], pos, tab, hd)
    want[:, Hq * hd:(Hq + Hkv) * hd] = orot.apply_rotary(qkv[:, Hq * hd:(Hq + Hkv) * hd], pos, tab, hd)
    g, gp, gt = qkv.to(dev), pos.to(dev), tab.to(dev)
    p = _lib.RopeParams()
    p.q = p.q_out = g.data_ptr()
    p.k = p.k_out = g.data_ptr() + Hq * hd * 2
    p.q_stride_token = p.k_stride_token = p.q_out_stride_token = p.k_out_stride_token = g.stride(0)
    p.positions, p.position_index_type = gp.data_ptr(), _lib.DFX_INDEX_I64
    p.cos_sin_cache, p.max_position = gt.data_ptr(), MAXPOS
    p.n_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = T, Hq, Hkv, hd
    rc = _lib.load().dfx_rope_kv_store(C.byref(p), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(_bits(g), _bits(want))          # V columns untouched as well


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("slot_dtype", [torch.int32, torch.int64])
def test_fused_store_equals_rotate_then_store(dev, fp8, slot_dtype):
    T, Hq, Hkv, hd, pages, page = 2048, 28, 4, 128, 40, 64
    qkv, pos = _inputs(T, Hq, Hkv, hd, seed=13)
    q, k, v = qkv[:, :Hq * hd], qkv[:, Hq * hd:(Hq + Hkv) * hd], qkv[:, (Hq + Hkv) * hd:]
    g = torch.Generator().manual_seed(14)
    slots = torch.randperm(pages * page, generator=g)[:T].to(slot_dtype)
    slots[::7] = -1
    slots[5] = pages * page + 3                  # out of range: skipped
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    want_q, want_k = orot.apply_rotary(q, pos, tab, hd), orot.apply_rotary(k, pos, tab, hd)
    cdt = torch.uint8 if fp8 else torch.bfloat16
    n = pages * page * Hkv * hd
    sentinel = (torch.arange(n, dtype=torch.int32) % 251 + 3).to(torch.uint8 if fp8 else torch.int16)
    kc0 = sentinel.view(cdt).reshape(pages, page, Hkv, hd).clone()
    ks = vs = None
    if fp8:
        ks = want_k.float().view(T, Hkv, hd).abs().amax(dim=(0, 2)) / 448.0
        vs = v.float().reshape(T, Hkv, hd).abs().amax(dim=(0, 2)) / 448.0
    want_kc, want_vc = kc0.clone(), kc0.clone()
    ok_slots = slots.clone()
    ok_slots[ok_slots >= pages * page] = -1
    okv.store_unified(want_k.view(T, Hkv, hd), v.reshape(T, Hkv, hd), want_kc, want_vc, ok_slots, ks, vs)
    rope = _rope(hd, dev)
    gq = qkv.to(dev)
    kc, vc = kc0.to(dev), kc0.to(dev)
    got_q, got_k = rope.forward_and_store(
        pos.to(dev), gq[:, :Hq * hd], gq[:, Hq * hd:(Hq + Hkv) * hd], gq[:, (Hq + Hkv) * hd:], kc, vc,
        slots.to(dev), k_scale=None if ks is None else ks.to(dev), v_scale=None if vs is None else vs.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(_bits(got_q), _bits(want_q))
    assert torch.equal(_bits(got_k), _bits(want_k))
    assert torch.equal(_bits(kc), _bits(want_kc))
    assert torch.equal(_bits(vc), _bits(want_vc))


def test_empty_input_is_a_no_op(dev):
    rope = _rope(128, dev)
    q = torch.empty(0, 28 * 128, dtype=torch.bfloat16, device=dev)
    k = torch.empty(0, 4 * 128, dtype=torch.bfloat16, device=dev)
    got_q, got_k = rope(torch.empty(0, dtype=torch.int64, device=dev), q, k)
    assert got_q.shape == q.shape and got_k.shape == k.shape


def test_layer_step_rope_store_attention_eager_and_in_a_graph(dev):
    """One decode step of an attention layer as the reference's model runs it
    (diffulex/model/dream.py:94-99): rotate q and k, store the rotated k and v, attend.  The fused
    rope + store launch followed by attention without its own store, eagerly and replayed from a
    captured graph, against the oracle pipeline (rotary -> store -> attention)."""
    import diffulex_amd as dfx
    from diffulex_amd.workloads import make_workload
    from oracle import attention as oat
    wl = make_workload("c3", num_seqs=5, ctx=(200, 900), seed=23)
    t, hq, hkv, hd = wl.q.shape[0], wl.num_q_heads, wl.num_kv_heads, wl.head_dim
    gen = torch.Generator().manual_seed(24)
    # each fresh token sits right behind its sequence's context
    pos = torch.cat([wl.context_lens[s] + torch.arange(wl.q_len) for s in range(wl.num_seqs)]).long()
    tab = orot.cos_sin_cache(hd, MAXPOS, BASE)
    q2, k2, v2 = wl.q.reshape(t, -1), wl.k_new.reshape(t, -1), wl.v_new.reshape(t, -1)
    rq, rk = orot.apply_rotary(q2, pos, tab, hd), orot.apply_rotary(k2, pos, tab, hd)
    want_kc, want_vc = wl.k_cache.clone(), wl.v_cache.clone()
    okv.store_unified(rk.view(t, hkv, hd), wl.v_new, want_kc, want_vc, wl.slot_mapping)
    want = oat.paged_attention_fp32(rq.view(t, hq, hd), rk.view(t, hkv, hd), wl.v_new, wl.k_cache, wl.v_cache,
                                    wl.block_tables, wl.context_lens, wl.cu_seqlens_q, wl.cu_seqlens_q, wl.scale)

    g = wl.to(dev)
    rope = _rope(hd, dev)
    att = dfx.Attention(hq, hd, g.scale, hkv)
    att.k_cache, att.v_cache = g.k_cache, g.v_cache
    md = dfx.PagedAttnMetaData(cu_seqlens_q=g.cu_seqlens_q, cu_seqlens_k=g.cu_seqlens_q, max_seqlen_q=g.q_len,
                               slot_mapping=g.slot_mapping, context_lens=g.context_lens, block_tables=g.block_tables,
                               page_block_size=g.page_size, decode_mode="static", need_kv_cache_store=False)
    dfx.set_fetch_fn_for_attn_metadata(lambda: md)
    gq, gk, gv, gpos = q2.to(dev), k2.to(dev), v2.to(dev), pos.to(dev)

    def layer():
        q_r, k_r = rope.forward_and_store(gpos, gq, gk, gv, att.k_cache, att.v_cache, md.slot_mapping, md)
        return att(q_r, k_r, gv)

    out = layer()
    torch.cuda.synchronize()
    assert torch.equal(_bits(g.k_cache), _bits(want_kc)) and torch.equal(_bits(g.v_cache), _bits(want_vc))
    assert float((out.view(t, hq, hd).float().cpu() - want).abs().max()) <= 2e-2

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer()                                   # the capture stream's workspace exists before the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        o_static = layer()
    dgen = torch.Generator(device=dev).manual_seed(9)
    for rep in range(3):
        for x in (gq, gk, gv):
            x.copy_(torch.randn(x.shape, generator=dgen, device=dev, dtype=torch.float32).to(x.dtype))
        graph.replay()
        torch.cuda.synchronize()
        got = o_static.clone()
        eager = layer()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {rep}"


@pytest.mark.parametrize("hd,h_q,h_kv,page", [(128, 28, 4, 256), (64, 8, 2, 32), (128, 4, 4, 16)])
def test_rope_and_store_into_the_distinct_layout_bit_exact(dev, hd, h_q, h_kv, page):
    """dfx_rope_kv_store writing the distinct cache layout (K [pages, H, hd / 8, page, 8], V [pages, H, hd, page]):
    the rotated K and V land where the CPU restatement of the reference's distinct store puts them, bit for bit;
    negative and out-of-range slots are skipped; the rest of the caches is untouched."""
    from oracle import kv_cache as okv
    g = torch.Generator("cpu").manual_seed(17)
    pages = 7
    T = min(300, pages * page - 8)
    qkv = torch.randn(T, (h_q + 2 * h_kv) * hd, generator=g).to(torch.bfloat16)
    q, k, v = qkv.split([h_q * hd, h_kv * hd, h_kv * hd], dim=-1)
    pos = torch.randint(0, 4096, (T,), generator=g)
    slots = torch.randperm(pages * page, generator=g)[:T].to(torch.int32)
    slots[5] = -1
    slots[9] = pages * page + 3
    kd0 = torch.randn(pages, h_kv, hd // 8, page, 8, generator=g).to(torch.bfloat16)
    vd0 = torch.randn(pages, h_kv, hd, page, generator=g).to(torch.bfloat16)
    tab = orot.cos_sin_cache(hd, 4096, 1.0e6)
    rk = orot.apply_rotary(k.contiguous(), pos, tab, hd)
    want_k, want_v = kd0.clone(), vd0.clone()
    ok = (slots >= 0) & (slots < pages * page)
    okv.store_distinct(rk.view(T, h_kv, hd)[ok], v.reshape(T, h_kv, hd)[ok], want_k, want_v, slots[ok])
    rope = RotaryEmbedding(hd, hd, 4096, 1.0e6).to(dev)
    kd, vd = kd0.to(dev), vd0.to(dev)
    d = qkv.to(dev)
    dq, dk, dv = d.split([h_q * hd, h_kv * hd, h_kv * hd], dim=-1)
    rq_got, rk_got = rope.forward_and_store(pos.to(dev), dq, dk, dv, kd, vd, slots.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(rk_got.cpu().view(torch.int16), rk.view(torch.int16))
    assert torch.equal(rq_got.cpu().view(torch.int16), orot.apply_rotary(q.contiguous(), pos, tab, hd).view(torch.int16))
    assert torch.equal(kd.cpu().view(torch.int16), want_k.view(torch.int16))
    assert torch.equal(vd.cpu().view(torch.int16), want_v.view(torch.int16))
