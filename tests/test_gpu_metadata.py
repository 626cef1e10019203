"""GPU parity of dfx_build_decode_metadata against the CPU restatement of the reference's
prepare_decode loops: integer work, bit-exact."""
import numpy as np
import pytest
import torch

import diffulex_amd as dfx
from diffulex_amd.metadata import build_decode_metadata
from oracle import metadata as om
from test_oracle_metadata import random_d2f_batch, IN, TO, ACT

pytestmark = pytest.mark.gpu


def _padded(rows, width, fill=0, dtype=np.int32):
    out = np.full((len(rows), width), fill, dtype)
    for i, r in enumerate(rows):
        out[i, :len(r)] = r
    return out


def _dev(a, dev, dtype=torch.int32):
    return torch.as_tensor(np.asarray(a)).to(dtype).to(dev)


def _check(md, want, n_seqs):
    s = md.summary.tolist()
    n_tok, n_slot = len(want["positions"]), len(want["slot_mapping"])
    assert s[:7] == [n_tok, n_slot, want["max_seqlen_q"], want["max_seqlen_k"], int(want["need_kv_cache_store"]), 0, 0]
    assert s[7] == int(want["cu_seqlens_k"][-1])
    assert np.array_equal(md.positions[:n_tok].cpu().numpy(), want["positions"])
    assert np.array_equal(md.slot_mapping[:n_slot].cpu().numpy(), want["slot_mapping"])
    assert np.array_equal(md.cu_seqlens_q[:n_seqs + 1].cpu().numpy(), want["cu_seqlens_q"])
    assert np.array_equal(md.cu_seqlens_k[:n_seqs + 1].cpu().numpy(), want["cu_seqlens_k"])
    assert np.array_equal(md.context_lens[:n_seqs].cpu().numpy(), want["context_lens"])


def _bd_batch(rng, n_seqs, page, dbs):
    n_tokens = [dbs * int(rng.integers(1, 40)) for _ in range(n_seqs)]
    state = [[TO, ACT, IN][int(rng.integers(0, 3))] for _ in range(n_seqs)]
    # tables are as long as the sequence needs, sometimes with pages to spare (allocated ahead)
    tables = [rng.integers(0, 5000, size=-(-n // page) + int(rng.integers(0, 3))).tolist() for n in n_tokens]
    return n_tokens, state, tables


@pytest.mark.parametrize("n_seqs,page,dbs", [(1, 32, 32), (7, 16, 32), (64, 32, 32), (300, 8, 32), (1500, 32, 64),
                                             (5, 64, 32)])
def test_block_diffusion_metadata_bits(dev, n_seqs, page, dbs):
    rng = np.random.default_rng(n_seqs)
    n_tokens, state, tables = _bd_batch(rng, n_seqs, page, dbs)
    want = om.bd_prepare_decode(n_tokens, state, tables, page, dbs)
    width = max(len(t) for t in tables) + 1
    toks = [rng.integers(0, 150000, n).tolist() for n in n_tokens]
    md = build_decode_metadata(
        "block_diffusion", block_tables=_dev(_padded(tables, width, -1), dev), block_state=_dev(state, dev, torch.uint8),
        page_size=page, diffusion_block_size=dbs, num_tokens=_dev(n_tokens, dev),
        num_pages=_dev([len(t) for t in tables], dev), token_capacity=n_seqs * dbs,
        token_ids=_dev(_padded(toks, max(n_tokens) + 3, -7, np.int64), dev, torch.int64))
    _check(md, want, n_seqs)
    assert md.decode_mode == "static" and md.max_seqlen_q == dbs
    assert np.array_equal(md.input_ids.cpu().numpy(), om.input_ids_of(want, toks))


@pytest.mark.parametrize("n_seqs,page,dbs,short", [(1, 32, 32, False), (6, 16, 32, True), (64, 32, 32, False),
                                                   (200, 256, 32, True), (1100, 48, 16, False)])
def test_d2f_metadata_bits(dev, n_seqs, page, dbs, short):
    rng = np.random.default_rng(100 + n_seqs)
    prompt, states, tables, last, _ = random_d2f_batch(rng, n_seqs, page, dbs, allow_short_last=short)
    want = om.d2f_prepare_decode(prompt, states, tables, page, dbs, last_block_size=last)
    if not short:
        assert om.check_slot_mapping(states, dbs, want["slot_mapping"].tolist()) == len(want["slot_mapping"])
    totals = [p + (len(st) - 2) * dbs + l for p, st, l in zip(prompt, states, last)]
    toks = [rng.integers(0, 150000, n).tolist() for n in totals]
    md = build_decode_metadata(
        "d2f", block_tables=_dev(_padded(tables, max(len(t) for t in tables), -1), dev),
        block_state=_dev(_padded(states, 8, 3, np.uint8), dev, torch.uint8), page_size=page, diffusion_block_size=dbs,
        prompt_len=_dev(prompt, dev), num_diffusion_blocks=_dev([len(s) for s in states], dev),
        num_tokens=_dev(totals, dev) if short else None, token_capacity=n_seqs * 6 * dbs, sync_summary=True,
        token_ids=_dev(_padded(toks, max(totals), -7, np.int64), dev, torch.int64))
    _check(md, want, n_seqs)
    assert np.array_equal(md.input_ids.cpu().numpy(), om.input_ids_of(want, toks))
    assert np.array_equal(md.seq_lens_ts[:n_seqs].cpu().numpy(), want["seq_lens"])
    assert md.max_seqlen_q == want["max_seqlen_q"] and md.need_kv_cache_store == want["need_kv_cache_store"]


def test_graph_buffers_zero_padded_as_the_reference_leaves_them(dev):
    """The step's arrays written straight into buffers of a larger captured batch: what follows
    the step's own entries reads as zeros, whatever the buffers held before."""
    rng = np.random.default_rng(9)
    page, dbs, n_seqs, padded_seqs = 32, 32, 5, 16
    n_tokens, state, tables = _bd_batch(rng, n_seqs, page, dbs)
    want = om.pad_for_graph(om.bd_prepare_decode(n_tokens, state, tables, page, dbs), padded_seqs, padded_seqs * dbs)
    i32 = dict(dtype=torch.int32, device=dev)
    bufs = dict(positions=torch.full((padded_seqs * dbs,), 77, dtype=torch.int64, device=dev),
                slot_mapping=torch.full((padded_seqs * dbs,), 77, **i32),
                cu_seqlens_q=torch.full((padded_seqs + 1,), 77, **i32), cu_seqlens_k=torch.full((padded_seqs + 1,), 77, **i32),
                context_lens=torch.full((padded_seqs,), 77, **i32), seq_lens=torch.full((padded_seqs,), 77, **i32),
                summary=torch.zeros(8, **i32), input_ids=torch.full((padded_seqs * dbs,), 77, dtype=torch.int64, device=dev))
    toks = [rng.integers(1, 150000, n).tolist() for n in n_tokens]
    build_decode_metadata(
        "block_diffusion", block_tables=_dev(_padded(tables, 48, 0), dev), block_state=_dev(state, dev, torch.uint8),
        page_size=page, diffusion_block_size=dbs, num_tokens=_dev(n_tokens, dev),
        num_pages=_dev([len(t) for t in tables], dev), token_capacity=padded_seqs * dbs,
        padded_seqs=padded_seqs, padded_tokens=padded_seqs * dbs, out=bufs,
        token_ids=_dev(_padded(toks, max(n_tokens), 0, np.int64), dev, torch.int64))
    for name in ("positions", "cu_seqlens_q", "cu_seqlens_k", "context_lens"):
        assert np.array_equal(bufs[name].cpu().numpy(), want[name]), name
    ids = om.input_ids_of(om.bd_prepare_decode(n_tokens, state, tables, page, dbs), toks)
    assert np.array_equal(bufs["input_ids"].cpu().numpy(), np.concatenate([ids, np.zeros(padded_seqs * dbs - len(ids), np.int64)]))
    # a block that is neither active nor to be cached adds no slot entries: compare what was produced
    n_slot = int(bufs["summary"][1])
    assert np.array_equal(bufs["slot_mapping"].cpu().numpy(), want["slot_mapping"]) and n_slot <= n_seqs * dbs


def test_states_the_reference_would_raise_on_are_flagged(dev):
    page, dbs = 32, 32
    states = [[IN, TO, ACT], [IN, ACT, TO], [TO, ACT, ACT], [IN, IN, ACT]]   # 1: order broken, 2: nothing cached
    tables = [[1, 2, 3, 4]] * 4
    md = build_decode_metadata(
        "d2f", block_tables=_dev(tables, dev), block_state=_dev(states, dev, torch.uint8), page_size=page,
        diffusion_block_size=dbs, prompt_len=_dev([20] * 4, dev), num_diffusion_blocks=_dev([3] * 4, dev),
        token_capacity=512)
    s = md.summary.tolist()
    assert s[6] == 2                                    # the first offending sequence, 1-based
    want = om.d2f_prepare_decode([20, 20], [states[0], states[3]], [tables[0]] * 2, page, dbs)
    cu = md.cu_seqlens_q.tolist()
    assert cu == [0, 64, 64, 64, 96]                    # the flagged sequences contribute nothing
    got = torch.cat([md.slot_mapping[:64], md.slot_mapping[64:96]]).cpu().numpy()
    assert np.array_equal(got, want["slot_mapping"])
    with pytest.raises(ValueError):
        build_decode_metadata(
            "d2f", block_tables=_dev(tables, dev), block_state=_dev(states, dev, torch.uint8), page_size=page,
            diffusion_block_size=dbs, prompt_len=_dev([20] * 4, dev), num_diffusion_blocks=_dev([3] * 4, dev),
            token_capacity=512, sync_summary=True)


def test_capacity_too_small_is_flagged_and_nothing_is_written_beyond_it(dev):
    page, dbs = 32, 32
    bufs = dict(positions=torch.full((96,), 77, dtype=torch.int64, device=dev),
                slot_mapping=torch.full((96,), 77, dtype=torch.int32, device=dev))
    cap = 40
    build = lambda **kw: build_decode_metadata(
        "block_diffusion", block_tables=_dev([[1, 2], [3, 4], [5, 6]], dev), block_state=_dev([ACT, TO, ACT], dev, torch.uint8),
        page_size=page, diffusion_block_size=dbs, num_tokens=_dev([64] * 3, dev), num_pages=_dev([2] * 3, dev),
        token_capacity=cap, out=bufs, **kw)
    md = build()
    assert md.summary.tolist()[5] == 1
    assert (bufs["positions"][cap:] == 77).all() and (bufs["slot_mapping"][cap:] == 77).all()
    assert bufs["slot_mapping"][:cap].tolist() == [-1] * 32 + list(range(4 * 32, 4 * 32 + 8))
    with pytest.raises(ValueError):
        build(sync_summary=True)


def test_metadata_built_on_the_device_drives_the_attention(dev):
    """End to end: a block-diffusion step prepared by the device kernel gives the same attention
    output as the step prepared by the host loop."""
    from diffulex_amd.workloads import make_workload
    from util import metadata_for
    wl = make_workload("c3", seed=83, num_seqs=6, ctx=(200, 900), page=32).to(dev)
    n_tokens = (wl.context_lens + 32).to(torch.int32)
    n_pages = torch.div(n_tokens + 31, 32, rounding_mode="floor").to(torch.int32)
    md = build_decode_metadata(
        "block_diffusion", block_tables=wl.block_tables, block_state=torch.full((6,), ACT, dtype=torch.uint8, device=dev),
        page_size=32, diffusion_block_size=32, num_tokens=n_tokens, num_pages=n_pages, token_capacity=6 * 32)
    assert torch.equal(md.context_lens, wl.context_lens) and torch.equal(md.cu_seqlens_q, wl.cu_seqlens_q)
    want = dfx.dllm_flash_attn_decode(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, metadata_for(wl))
    got = dfx.dllm_flash_attn_decode(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, md)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
