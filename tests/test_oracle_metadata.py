"""The CPU restatement of the decode-step metadata loops, pinned by hand-worked cases, by the
layout the reference's own checker demands, and by a store -> gather round trip through a paged
cache (a slot mapping is right exactly when the gather by block table finds every token where the
store by slot mapping put it)."""
import numpy as np
import pytest
import torch

from oracle import metadata as om
from oracle import attention as oat

IN, TO, ACT = om.IN_CACHE, om.TO_CACHE, om.ACTIVE


def test_block_diffusion_hand_worked():
    # three sequences, 32-token blocks on 16-token pages: a block covers the last two pages of a table
    m = om.bd_prepare_decode(num_tokens=[96, 64, 160], last_state=[TO, ACT, IN],
                             block_tables=[[5, 2, 9, 4, 7, 1], [3, 8, 6, 0], list(range(10, 20))],
                             page_size=16, dbs=32)
    assert m["context_lens"].tolist() == [64, 32, 128]
    assert m["cu_seqlens_q"].tolist() == [0, 32, 64, 96] and m["cu_seqlens_k"].tolist() == [0, 32, 64, 96]
    assert m["positions"].tolist() == list(range(64, 96)) + list(range(32, 64)) + list(range(128, 160))
    # sequence 0 stores into pages 7 and 1, sequence 1 stores nothing (-1), sequence 2 adds no entries
    want = list(range(7 * 16, 8 * 16)) + list(range(16, 32)) + [-1] * 32
    assert m["slot_mapping"].tolist() == want
    assert (m["max_seqlen_q"], m["max_seqlen_k"], m["need_kv_cache_store"]) == (32, 32, True)
    only_active = om.bd_prepare_decode([64], [ACT], [[1, 2]], 32, 32)
    assert only_active["need_kv_cache_store"] is False and only_active["slot_mapping"].tolist() == [-1] * 32


def test_d2f_hand_worked_blocks_straddling_pages():
    # prompt of 40 tokens, 32-token blocks and pages: block 1 covers positions 40..71 (pages 1 and 2)
    m = om.d2f_prepare_decode(prompt_len=[40], states=[[IN, TO, ACT]], block_tables=[[6, 3, 11, 2]],
                              page_size=32, dbs=32)
    assert m["context_lens"].tolist() == [40] and m["seq_lens"].tolist() == [64]
    assert m["cu_seqlens_q"].tolist() == [0, 64] and m["cu_seqlens_k"].tolist() == [0, 104]
    assert m["positions"].tolist() == list(range(40, 104))
    want = list(range(3 * 32 + 8, 4 * 32)) + list(range(11 * 32, 11 * 32 + 8)) + [-1] * 32
    assert m["slot_mapping"].tolist() == want
    assert (m["max_seqlen_q"], m["max_seqlen_k"], m["need_kv_cache_store"]) == (64, 104, True)
    # two sequences: the second has everything after the prompt still active
    m2 = om.d2f_prepare_decode([40, 10], [[IN, TO, ACT], [IN, ACT, ACT]], [[6, 3, 11, 2], [9, 4, 5]], 32, 32)
    assert m2["slot_mapping"].tolist() == want + [-1] * 64
    assert m2["cu_seqlens_q"].tolist() == [0, 64, 128] and m2["cu_seqlens_k"].tolist() == [0, 104, 178]
    assert m2["context_lens"].tolist() == [40, 10] and m2["positions"].tolist()[64:] == list(range(10, 74))


def random_d2f_batch(rng, n_seqs, page, dbs, allow_short_last=False):
    prompt, states, tables, last = [], [], [], []
    next_page = 0
    for _ in range(n_seqs):
        p_len = int(rng.integers(1, 5 * page))
        n_blocks = int(rng.integers(2, 7))
        n_in = int(rng.integers(1, n_blocks))
        n_to = int(rng.integers(0, n_blocks - n_in + 1))
        st = [IN] * n_in + [TO] * n_to + [ACT] * (n_blocks - n_in - n_to)
        short = allow_short_last and st[-1] == TO and rng.integers(0, 2) == 1
        last_size = int(rng.integers(1, dbs)) if short else dbs
        total = p_len + (n_blocks - 2) * dbs + last_size
        n_pages = -(-total // page)
        ids = rng.permutation(np.arange(next_page, next_page + n_pages + 2))[:n_pages]   # disjoint page ids
        next_page += n_pages + 2
        prompt.append(p_len); states.append(st); tables.append(ids.tolist()); last.append(last_size)
    return prompt, states, tables, last, next_page


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("page,dbs", [(32, 32), (16, 32), (64, 32), (256, 32), (48, 16)])
def test_d2f_slots_are_where_the_gather_reads(seed, page, dbs):
    rng = np.random.default_rng(seed)
    prompt, states, tables, last, n_pages = random_d2f_batch(rng, 5, page, dbs, allow_short_last=True)
    m = om.d2f_prepare_decode(prompt, states, tables, page, dbs, last_block_size=last)
    if all(l == dbs for l in last):   # (the reference's checker assumes whole blocks)
        assert om.check_slot_mapping(states, dbs, m["slot_mapping"].tolist()) == len(m["slot_mapping"])
    # store the position of every fed token where the slot mapping says, then gather each
    # sequence's context + stored tokens by its block table: positions ctx .. ctx + stored come back
    cache = torch.full((n_pages, page, 1, 1), -7.0)
    slots, pos = m["slot_mapping"], m["positions"]
    for i, slot in enumerate(slots.tolist()):
        if slot >= 0:
            assert cache.view(-1)[slot] == -7.0, "two tokens in one slot"
            cache.view(-1)[slot] = float(pos[i])
    for s, st in enumerate(states):
        ctx = int(m["context_lens"][s])
        q0, q1 = int(m["cu_seqlens_q"][s]), int(m["cu_seqlens_q"][s + 1])
        stored = int((slots[q0:q1] >= 0).sum())
        sizes = [prompt[s]] + [dbs] * (len(st) - 2) + [last[s]]
        assert stored == sum(sz for sz, x in zip(sizes, st) if x == TO)
        assert (slots[q0 + stored:q1] == -1).all()
        got = oat.gather_context(cache, torch.tensor(tables[s]), ctx + stored, page).view(-1)
        assert got[ctx:].tolist() == [float(x) for x in range(ctx, ctx + stored)]
        assert (got[:ctx] == -7.0).all()                       # the cached prefix is not written again
        assert int(m["cu_seqlens_k"][s + 1] - m["cu_seqlens_k"][s]) == sum(sizes)
        assert q1 - q0 == sum(sizes) - ctx == int(m["seq_lens"][s])
        assert pos[q0:q1].tolist() == list(range(ctx, ctx + q1 - q0))


def test_checker_layout_holds_and_catches_a_wrong_mapping():
    rng = np.random.default_rng(3)
    prompt, states, tables, _, _ = random_d2f_batch(rng, 6, 32, 32)
    m = om.d2f_prepare_decode(prompt, states, tables, 32, 32)
    slots = m["slot_mapping"].tolist()
    assert om.check_slot_mapping(states, 32, slots) == len(slots)
    act = next(i for i, x in enumerate(slots) if x == -1)
    bad = list(slots); bad[act] = 5
    with pytest.raises(ValueError):
        om.check_slot_mapping(states, 32, bad)
    real = next(i for i, x in enumerate(slots) if x != -1)
    bad = list(slots); bad[real] = -1
    with pytest.raises(ValueError):
        om.check_slot_mapping(states, 32, bad)


def test_block_diffusion_round_trip():
    rng = np.random.default_rng(5)
    page, dbs = 16, 32
    n_tokens, st, tables = [], [], []
    nxt = 0
    for _ in range(7):
        n = dbs * int(rng.integers(1, 9))
        n_tokens.append(n); st.append([TO, ACT][int(rng.integers(0, 2))])
        k = n // page
        tables.append(rng.permutation(np.arange(nxt, nxt + k)).tolist()); nxt += k
    m = om.bd_prepare_decode(n_tokens, st, tables, page, dbs)
    cache = torch.full((nxt, page, 1, 1), -7.0)
    o = 0
    for s in range(7):
        q0 = int(m["cu_seqlens_q"][s])
        n_slots = dbs
        sl = m["slot_mapping"][o:o + n_slots]
        o += n_slots
        if st[s] == ACT:
            assert (sl == -1).all()
            continue
        for i, slot in enumerate(sl.tolist()):
            cache.view(-1)[slot] = float(m["positions"][q0 + i])
        got = oat.gather_context(cache, torch.tensor(tables[s]), n_tokens[s], page).view(-1)
        assert got[n_tokens[s] - dbs:].tolist() == [float(x) for x in range(n_tokens[s] - dbs, n_tokens[s])]
    assert o == len(m["slot_mapping"])


def test_graph_buffers_are_zero_filled_behind_the_step():
    m = om.bd_prepare_decode([64, 96], [TO, ACT], [[1, 2], [3, 4, 5]], 32, 32)
    g = om.pad_for_graph(m, padded_seqs=4, padded_tokens=128)
    assert g["cu_seqlens_q"].tolist() == [0, 32, 64, 0, 0] and g["context_lens"].tolist() == [32, 64, 0, 0]
    assert g["slot_mapping"][64:].tolist() == [0] * 64 and g["positions"][:64].tolist() == m["positions"].tolist()


def test_input_ids_are_the_sequences_tokens_at_the_fed_positions():
    """Hand-worked: the block-diffusion step feeds the last block of every sequence, the D2F step every
    block behind the cached ones; their token ids are the sequences' own at those positions."""
    toks = [list(range(1000, 1096)), list(range(2000, 2064))]
    m = om.bd_prepare_decode(num_tokens=[96, 64], last_state=[TO, ACT], block_tables=[[5, 2, 9], [3, 8]], page_size=32, dbs=32)
    assert om.input_ids_of(m, toks).tolist() == list(range(1064, 1096)) + list(range(2032, 2064))
    d = om.d2f_prepare_decode(prompt_len=[40, 10], states=[[IN, TO, ACT], [IN, ACT, ACT]], block_tables=[[6, 3, 11, 2], [9, 4, 5]],
                              page_size=32, dbs=32)
    toks = [list(range(5000, 5104)), list(range(7000, 7074))]
    assert om.input_ids_of(d, toks).tolist() == list(range(5040, 5104)) + list(range(7010, 7074))
    # with distinct random ids: position p of sequence s gives exactly token_ids[s][p]
    rng = np.random.default_rng(3)
    toks = [rng.integers(0, 50000, 104).tolist(), rng.integers(0, 50000, 74).tolist()]
    got = om.input_ids_of(d, toks)
    assert got.tolist() == toks[0][40:104] + toks[1][10:74]
