"""Pins oracle/attention.py against the library SDPA, brute force and invariants."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from diffulex_amd.workloads import make_workload, MASK_FULL, MASK_BLOCK_CAUSAL
from oracle import attention as oat
from oracle import fp8_e4m3


def _run_fp32(wl, **kw):
    args = dict(q=wl.q, k_new=wl.k_new, v_new=wl.v_new, k_cache=wl.k_cache, v_cache=wl.v_cache,
                block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
                cu_seqlens_new=wl.cu_seqlens_q, scale=wl.scale, mask_mode=wl.mask_mode,
                dbs=wl.diffusion_block_size, k_scale=wl.k_scale, v_scale=wl.v_scale)
    args.update(kw)
    return oat.paged_attention_fp32(**args)


def test_c1_matches_library_sdpa_fp32_on_gathered_kv():
    """The reference's own oracle (test_dllm_flash_attn_decode_kernel.py:14-105) is the library SDPA on
    gathered K/V; in fp32 it must agree with the explicit softmax to rounding error."""
    wl = make_workload("c1")
    got = _run_fp32(wl)
    want = oat.paged_attention_sdpa(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.block_tables,
                                    wl.context_lens, wl.cu_seqlens_q, wl.cu_seqlens_q, wl.scale,
                                    compute_dtype=torch.float32)
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("mask", [MASK_FULL, MASK_BLOCK_CAUSAL])
def test_small_d2f_matches_library_sdpa_with_mask(mask):
    wl = make_workload("c4", num_seqs=3, h_q=4, h_kv=2, hd=64, page=16, ctx=[40, 0, 97], mask=mask)
    got = _run_fp32(wl)
    want = oat.paged_attention_sdpa(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.block_tables,
                                    wl.context_lens, wl.cu_seqlens_q, wl.cu_seqlens_q, wl.scale,
                                    mask_mode=mask, dbs=32, compute_dtype=torch.float32)
    assert torch.allclose(got, want, atol=2e-6, rtol=1e-5)


def test_triple_loop_on_a_tiny_case():
    wl = make_workload("c1", num_seqs=2, h_q=2, h_kv=1, hd=8, page=4, ctx=[5, 9], q_len=6, dbs=2,
                       mask=MASK_BLOCK_CAUSAL)
    got = _run_fp32(wl)
    page = 4
    for s in range(2):
        ctx = int(wl.context_lens[s])
        for i in range(6):
            for h in range(2):
                qv = wl.q[s * 6 + i, h].double()
                keys, vals = [], []
                for t in range(ctx):
                    pg = int(wl.block_tables[s, t // page])
                    keys.append(wl.k_cache[pg, t % page, 0].double())
                    vals.append(wl.v_cache[pg, t % page, 0].double())
                for j in range(6):
                    if j < (i // 2 + 1) * 2:
                        keys.append(wl.k_new[s * 6 + j, 0].double())
                        vals.append(wl.v_new[s * 6 + j, 0].double())
                logits = torch.stack([(qv * k).sum() * wl.scale for k in keys])
                w = torch.softmax(logits, 0)
                o = sum(wi * v for wi, v in zip(w, vals))
                assert torch.allclose(got[s * 6 + i, h].double(), o, atol=1e-5)


def test_rows_of_ones_in_v_give_ones():
    wl = make_workload("c1")
    wl.v_new.fill_(1.0)
    wl.v_cache.fill_(1.0)
    got = _run_fp32(wl)
    assert torch.allclose(got, torch.ones_like(got), atol=1e-6)


def test_permuting_physical_pages_with_the_table_is_a_no_op():
    wl = make_workload("c1")
    base = _run_fp32(wl)
    g = torch.Generator().manual_seed(9)
    n_pages = wl.k_cache.shape[0]
    perm = torch.randperm(n_pages, generator=g)            # new_id = perm[old_id]
    kc2, vc2 = torch.empty_like(wl.k_cache), torch.empty_like(wl.v_cache)
    kc2[perm] = wl.k_cache
    vc2[perm] = wl.v_cache
    bt2 = wl.block_tables.clone()
    valid = bt2 >= 0
    bt2[valid] = perm[bt2[valid].long()].to(torch.int32)
    got = _run_fp32(wl, k_cache=kc2, v_cache=vc2, block_tables=bt2)
    assert torch.equal(got, base)


@pytest.mark.parametrize("mask", [MASK_FULL, MASK_BLOCK_CAUSAL])
def test_a_skipped_page_is_the_same_as_a_shorter_context_without_it(mask):
    """Negative table entries drop their page's tokens (dllm_flash_attn.py:260-261): the result is
    that of a sequence whose context simply lacks those tokens (table compacted, length reduced)."""
    wl = make_workload("c4", num_seqs=2, ctx=[100, 70], page=16, mask=mask, seed=13)
    bt = wl.block_tables.clone()
    bt[0, 1] = -1
    bt[0, 4] = -1
    bt[1, 0] = -1
    holed = _run_fp32(wl, block_tables=bt)
    # the same thing spelled without holes: drop the entries, shorten the contexts by whole pages
    bt2 = torch.full_like(bt, -1)
    ctx2 = wl.context_lens.clone()
    for s in range(2):
        n_ctx_pages = -(-int(wl.context_lens[s]) // 16)
        kept = [int(x) for x in bt[s, :n_ctx_pages] if x >= 0]
        assert int(wl.context_lens[s]) % 16 != 0 and bt[s, n_ctx_pages - 1] >= 0   # the partial last page stays last
        bt2[s, :len(kept)] = torch.tensor(kept, dtype=bt.dtype)
        ctx2[s] -= 16 * (n_ctx_pages - len(kept))
    plain = _run_fp32(wl, block_tables=bt2, context_lens=ctx2)
    assert torch.equal(holed, plain)
    assert not torch.equal(holed, _run_fp32(wl))
    lib = oat.paged_attention_sdpa(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, bt, wl.context_lens,
                                   wl.cu_seqlens_q, wl.cu_seqlens_q, wl.scale, mask_mode=mask,
                                   dbs=wl.diffusion_block_size, compute_dtype=torch.float32)
    assert float((lib - holed).abs().max()) < 2e-5


def test_repaging_the_same_context_is_a_no_op():
    wl = make_workload("c1")          # page 16
    base = _run_fp32(wl)
    # rebuild the same logical context in pages of 8 tokens
    page2 = 8
    ctx = wl.context_lens.tolist()
    rows_k = [oat.gather_context(wl.k_cache, wl.block_tables[s], ctx[s], 16) for s in range(2)]
    rows_v = [oat.gather_context(wl.v_cache, wl.block_tables[s], ctx[s], 16) for s in range(2)]
    n_pages = sum(-(-c // page2) for c in ctx)
    kc2 = torch.zeros(n_pages, page2, 2, 64, dtype=torch.bfloat16)
    vc2 = torch.zeros_like(kc2)
    bt2 = torch.full((2, max(-(-c // page2) for c in ctx)), -1, dtype=torch.int32)
    cur = 0
    for s in range(2):
        for p in range(-(-ctx[s] // page2)):
            m = min(page2, ctx[s] - p * page2)
            kc2[cur, :m] = rows_k[s][p * page2:p * page2 + m]
            vc2[cur, :m] = rows_v[s][p * page2:p * page2 + m]
            bt2[s, p] = cur
            cur += 1
    got = _run_fp32(wl, k_cache=kc2, v_cache=vc2, block_tables=bt2)
    assert torch.allclose(got, base, atol=1e-6)


def test_block_causal_with_one_block_equals_full_and_zero_context_is_in_block_attention():
    wl = make_workload("c1")
    assert torch.equal(_run_fp32(wl, mask_mode=MASK_BLOCK_CAUSAL, dbs=32), _run_fp32(wl, mask_mode=MASK_FULL))
    zero = torch.zeros_like(wl.context_lens)
    got = _run_fp32(wl, context_lens=zero)
    for s in range(2):
        q = wl.q[s * 32:(s + 1) * 32].float().permute(1, 0, 2)
        k = wl.k_new[s * 32:(s + 1) * 32].float().permute(1, 0, 2).repeat_interleave(2, 0)
        v = wl.v_new[s * 32:(s + 1) * 32].float().permute(1, 0, 2).repeat_interleave(2, 0)
        want = F.scaled_dot_product_attention(q, k, v, scale=wl.scale).permute(1, 0, 2)
        assert torch.allclose(got[s * 32:(s + 1) * 32], want, atol=2e-6, rtol=1e-5)


def test_fp8_cache_dequant_convention():
    """fp8.to(f32) * scale (diffulex_legacy/.../prefix_prefill.py:126-129): the fp8 oracle equals the
    bf16-free oracle run on explicitly dequantised fp32 caches."""
    wl = make_workload("c5", num_seqs=2, ctx=[70, 130], page=16, h_q=4, h_kv=2, hd=64)
    got = _run_fp32(wl)
    kd = torch.from_numpy(fp8_e4m3.dequantize_per_head(wl.k_cache.view(torch.uint8).numpy(), wl.k_scale.numpy()))
    vd = torch.from_numpy(fp8_e4m3.dequantize_per_head(wl.v_cache.view(torch.uint8).numpy(), wl.v_scale.numpy()))
    # library cast + multiply as the independent statement of the convention
    kd2 = wl.k_cache.to(torch.float32) * wl.k_scale.view(1, 1, -1, 1)
    assert torch.equal(kd, kd2)
    want = _run_fp32(wl, k_cache=kd, v_cache=vd, k_scale=None, v_scale=None)
    assert torch.allclose(got, want, atol=1e-6)
    # and it is close to attention on the unquantised source (sanity: quantisation error only)
    assert got.abs().max() < 10


def test_flop_and_byte_counts_closed_forms():
    ctx, ql = [100, 200], [32, 32]
    assert oat.algorithmic_flops(ctx, ql, ql, 28, 128) == 4 * 28 * 128 * (32 * 100 + 32 * 32 + 32 * 200 + 32 * 32)
    # three blocks, block-causal: rows of block b see 32*(b+1) fresh tokens
    assert oat.algorithmic_flops([10], [96], [96], 1, 64, MASK_BLOCK_CAUSAL, 32) == 4 * 64 * (96 * 10 + 32 * (32 + 64 + 96))
    assert oat.algorithmic_bytes(ctx, ql, ql, 28, 4, 128, 2) == 300 * 4 * 128 * 4 + 2 * 64 * 28 * 128 * 2 + 64 * 4 * 128 * 4


def test_golden_fixture_is_what_the_oracle_produces():
    import os
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_attention.npz"))
    wl = make_workload("c1")
    assert np.array_equal(fx["q_bits"], wl.q.view(torch.int16).numpy())
    assert np.array_equal(fx["k_cache_bits"], wl.k_cache.view(torch.int16).numpy())
    assert np.array_equal(fx["block_tables"], wl.block_tables.numpy())
    assert np.allclose(fx["out_fp32"], _run_fp32(wl).numpy(), atol=1e-6)
