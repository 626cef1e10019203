"""Decode-step attention metadata restated on the CPU, on plain arrays.

Test infrastructure only (see ``oracle/__init__.py``).

The reference builds the metadata of a decode step in Python loops over its sequence objects
(``prepare_decode`` of the two strategies).  Here a sequence is reduced to the numbers those loops
read: its length, the size of its diffusion blocks, the state of every diffusion block
(``IN_CACHE`` / ``TO_CACHE`` / ``ACTIVE``), its row of the block table, and the page size.

* ``bd_prepare_decode``: diffulex/strategy/block_diffusion/engine/model_runner.py:114-173
  (with ``BDSequence.diffusion_decoding_inputs``, block_diffusion/engine/sequence.py:186-191).
* ``d2f_prepare_decode``: diffulex/strategy/d2f/engine/model_runner.py:137-262, the walk over
  memory blocks kept statement by statement (cursors included), with
  ``D2FSequence.diffusion_decoding_inputs`` (d2f/engine/sequence.py:357-370),
  ``mem_block_to_diffusion_blocks_map`` / ``token_to_diffusion_block_id`` (sequence.py:335-350).
* ``check_slot_mapping``: diffulex/utils/checker.py:1-27.
* ``pad_for_graph``: the graph-replay buffers of ``run_model``
  (block_diffusion/engine/model_runner.py:176-197): every buffer zeroed, then the step's values
  copied into its head.
"""
from __future__ import annotations

import numpy as np

IN_CACHE, TO_CACHE, ACTIVE = 0, 1, 2


def bd_prepare_decode(num_tokens, last_state, block_tables, page_size, dbs):
    """num_tokens[s]: len(seq) after ``next_diffusion_step``; last_state[s]: state of
    ``seq.diffusion_blocks[-1]``; block_tables[s]: ``seq.block_table`` (a list, its own length)."""
    positions, cu_q, cu_k, slots, ctx = [], [0], [0], [], []
    need_store = False
    max_q = max_k = 0
    for n, state, table in zip(num_tokens, last_state, block_tables):
        positions.extend(range(n - dbs, n))
        ctx.append(n - dbs)
        max_q, max_k = max(dbs, max_q), max(dbs, max_k)
        cu_q.append(cu_q[-1] + dbs)
        cu_k.append(cu_k[-1] + dbs)
        if state == ACTIVE:
            slots.extend([-1] * dbs)
        elif state == TO_CACHE:
            need_store = True
            n_storing = dbs // page_size
            total = len(table)
            for i in range(n_storing):
                start = table[total - n_storing + i] * page_size
                slots.extend(range(start, start + page_size))
    return dict(positions=np.asarray(positions, np.int64), cu_seqlens_q=np.asarray(cu_q, np.int32),
                cu_seqlens_k=np.asarray(cu_k, np.int32), slot_mapping=np.asarray(slots, np.int32),
                context_lens=np.asarray(ctx, np.int32), seq_lens=np.full(len(ctx), dbs, np.int32),
                max_seqlen_q=max_q, max_seqlen_k=max_k, need_kv_cache_store=need_store)


def d2f_prepare_decode(prompt_len, states, block_tables, page_size, dbs, last_block_size=None):
    """prompt_len[s]: ``seq.input_num_tokens`` (the size of diffusion block 0); states[s]: the
    state of every diffusion block; block_tables[s]: ``seq.block_table``.  Blocks after the first
    have ``dbs`` tokens, except that ``last_block_size[s]`` (optional) gives a shorter last one."""
    positions, cu_q, cu_k, slots, ctx_all, seq_lens = [], [0], [0], [], [], []
    need_store = False
    max_q = max_k = 0
    for s, (p_len, st, table) in enumerate(zip(prompt_len, states, block_tables)):
        n_blocks = len(st)
        sizes = [p_len] + [dbs] * (n_blocks - 1)
        if last_block_size is not None and n_blocks > 1:
            sizes[-1] = last_block_size[s]
        cursor = [0] * n_blocks
        total = sum(sizes)
        # diffusion_decoding_inputs
        cached_ids = [i for i, x in enumerate(st) if x == IN_CACHE]
        tail = list(range(cached_ids[-1] + 1, n_blocks))
        assert len(tail) == sum(x == ACTIVE for x in st) + sum(x == TO_CACHE for x in st)
        context_len = sum(sizes[i] for i in cached_ids)
        t = context_len
        n_in = 0
        for b in tail:
            positions.extend(range(t, t + sizes[b]))
            t += sizes[b]
            n_in += sizes[b]
        seq_lens.append(n_in)
        ctx_all.append(context_len)
        cached_num_tokens = context_len
        seqlen_q, seqlen_k = total - cached_num_tokens, total
        max_q, max_k = max(seqlen_q, max_q), max(seqlen_k, max_k)
        cu_q.append(cu_q[-1] + seqlen_q)
        cu_k.append(cu_k[-1] + seqlen_k)

        def block_of(token):
            return 0 if token < p_len else (token - p_len) // dbs + 1

        num_mem_blocks = (total + page_size - 1) // page_size
        n_slots_before = len(slots)
        for mem in range(num_mem_blocks):
            start_idx = mem * page_size
            end_idx = start_idx + page_size
            window = page_size if mem < num_mem_blocks - 1 else total - (num_mem_blocks - 1) * page_size
            cur_map = [block_of(tok) for tok in range(start_idx, start_idx + window)]
            is_last = meet_active = False
            while start_idx < end_idx and not is_last and not meet_active:
                local = start_idx % page_size
                b = cur_map[local]
                if b == 0 and cursor[b] != start_idx:
                    cursor[b] = start_idx
                if b == n_blocks - 1:
                    is_last = True
                remaining = sizes[b] - cursor[b]
                step = remaining if remaining + local <= page_size else page_size - local
                if st[b] == IN_CACHE:
                    cursor[b] += step
                    start_idx += step
                elif st[b] == TO_CACHE:
                    cursor[b] += step
                    start_idx += step
                    mem_start = table[mem] * page_size + context_len % page_size
                    context_len += step
                    slots.extend(range(mem_start, mem_start + step))
                    need_store = True
                elif st[b] == ACTIVE:
                    meet_active = True
            if meet_active:
                first_active = next((i for i, x in enumerate(st) if x == ACTIVE), None)
                if first_active is not None:
                    slots.extend([-1] * ((n_blocks - first_active) * dbs))
                break
        assert len(slots) - n_slots_before == n_in, "slot mapping length does not match the input length"
    return dict(positions=np.asarray(positions, np.int64), cu_seqlens_q=np.asarray(cu_q, np.int32),
                cu_seqlens_k=np.asarray(cu_k, np.int32), slot_mapping=np.asarray(slots, np.int32),
                context_lens=np.asarray(ctx_all, np.int32), seq_lens=np.asarray(seq_lens, np.int32),
                max_seqlen_q=max_q, max_seqlen_k=max_k, need_kv_cache_store=need_store)


def input_ids_of(meta, token_ids):
    """The step's ``input_ids``: the reference concatenates every sequence's ``cur_input_ids``
    (block_diffusion/engine/model_runner.py:126-130 with ``active_block_token_ids``, sequence.py:186-191;
    d2f/engine/model_runner.py:153-158 with the ``token_ids`` of every block behind the cached ones,
    sequence.py:369-382), which are the sequence's tokens at the positions the step feeds.
    ``token_ids[s]``: the token list of sequence s."""
    out = []
    pos = meta["positions"].tolist()
    lens = meta["seq_lens"].tolist()
    i = 0
    for s, n in enumerate(lens):
        for p in pos[i:i + n]:
            out.append(int(token_ids[s][p]))
        i += n
    return np.asarray(out, np.int64)


def check_slot_mapping(states, dbs, slot_mapping):
    """The layout ``CHECK_SLOT_MAPPING`` demands of a D2F slot mapping: per sequence, ``dbs``
    real slots for every block to be cached, then -1 from the first active block to the end."""
    start = 0
    for st in states:
        ref = []
        for idx, x in enumerate(st):
            if x == ACTIVE:
                ref.extend([-1] * ((len(st) - idx) * dbs))
                break
            if x == TO_CACHE:
                ref.extend([0] * dbs)
        cur = slot_mapping[start:start + len(ref)]
        if len(cur) != len(ref):
            raise ValueError("slot mapping too short")
        for slot, r in zip(cur, ref):
            if (r == -1 and slot != -1) or (r == 0 and slot == -1):
                raise ValueError(f"Slot mapping mismatch: {slot} != {r}")
        start += len(ref)
    return start


def pad_for_graph(meta, padded_seqs, padded_tokens):
    """The per-step arrays as the captured graph sees them: zero-filled buffers of the captured
    batch's size with the step's values in front."""
    def head(values, n, dtype):
        out = np.zeros(n, dtype)
        out[:len(values)] = values
        return out
    return dict(positions=head(meta["positions"], padded_tokens, np.int64),
                slot_mapping=head(meta["slot_mapping"], padded_tokens, np.int32),
                context_lens=head(meta["context_lens"], padded_seqs, np.int32),
                seq_lens=head(meta["seq_lens"], padded_seqs, np.int32),
                cu_seqlens_q=head(meta["cu_seqlens_q"], padded_seqs + 1, np.int32),
                cu_seqlens_k=head(meta["cu_seqlens_k"], padded_seqs + 1, np.int32))
