"""Pins oracle/kv_cache.py: brute force, sentinel invariants, layout identities and the
structural fixtures held by the reference's example scripts."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import kv_cache as okv
from oracle import fp8_e4m3

HERE = os.path.dirname(os.path.abspath(__file__))


def _rand_bf16(shape, gen):
    return torch.randn(shape, generator=gen, dtype=torch.float32).to(torch.bfloat16)


def _sentinel(shape):
    n = int(np.prod(shape))
    return (torch.arange(n, dtype=torch.int32) % 251 + 0x4000).to(torch.int16).view(torch.bfloat16).reshape(shape).clone()


def test_store_unified_brute_force_and_untouched_slots():
    g = torch.Generator().manual_seed(0)
    n, h, hd, pages, page = 11, 2, 8, 5, 4
    key, value = _rand_bf16((n, h, hd), g), _rand_bf16((n, h, hd), g)
    slots = torch.tensor([3, -1, 7, 0, 19, -1, 12, 5, 6, -1, 18], dtype=torch.int32)
    kc, vc = _sentinel((pages, page, h, hd)), _sentinel((pages, page, h, hd)) 
    kc0, vc0 = kc.clone(), vc.clone()
    okv.store_unified(key, value, kc, vc, slots)
    # element-by-element restatement of kv_cache_kernels.py:22-32
    ek, ev = kc0.clone().view(-1), vc0.clone().view(-1)
    d = h * hd
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        for e in range(d):
            ek[s * d + e] = key.reshape(n, d)[t, e]
            ev[s * d + e] = value.reshape(n, d)[t, e]
    assert torch.equal(kc.view(torch.int16), ek.view(pages, page, h, hd).view(torch.int16))
    assert torch.equal(vc.view(torch.int16), ev.view(pages, page, h, hd).view(torch.int16))
    touched = set(int(s) for s in slots if s >= 0)
    for s in range(pages * page):
        if s not in touched:
            assert torch.equal(kc.view(-1, d)[s].view(torch.int16), kc0.view(-1, d)[s].view(torch.int16))
    # K and V are independent
    assert not torch.equal(kc.view(torch.int16), vc.view(torch.int16))


def test_store_follows_reference_example_slot_recipe():
    """examples/test_dllm_kv_cache_store.py:27-33: per sequence, ctx_len consecutive slots starting at
    seq_idx * page, followed by 32 entries of -1; the cached prefix must equal the input rows."""
    g = torch.Generator().manual_seed(114514)
    ctx_lens = [119, 110, 81, 114, 112, 119, 110, 81]
    h, hd, page = 4, 16, 256
    total = sum(ctx_lens) + 32 * len(ctx_lens)
    key, value = _rand_bf16((total, h, hd), g), _rand_bf16((total, h, hd), g)
    slots, start = [], 0
    for i, c in enumerate(ctx_lens):
        slots += list(range(i * page, i * page + c)) + [-1] * 32
    slots = torch.tensor(slots, dtype=torch.int64)
    kc = torch.zeros(len(ctx_lens), page, h, hd, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    okv.store_unified(key, value, kc, vc, slots)
    for i, c in enumerate(ctx_lens):
        assert torch.equal(kc[i, :c], key[start:start + c])
        assert torch.equal(vc[i, :c], value[start:start + c])
        assert kc[i, c:].abs().sum() == 0
        start += c + 32


def test_captured_slot_mapping_fixture():
    """The slot mapping captured in examples/mimic_data/mimic_slot_mapping.py: 32 consecutive slots
    882..913 in a run, every other entry -1 (stored here as data: length, run start, run offset)."""
    fx = json.load(open(os.path.join(HERE, "golden", "mimic_slot_mapping.json")))
    slots = torch.full((fx["length"],), -1, dtype=torch.int64)
    slots[fx["run_offset"]:fx["run_offset"] + fx["run_length"]] = torch.arange(
        fx["run_first_slot"], fx["run_first_slot"] + fx["run_length"])
    g = torch.Generator().manual_seed(3)
    h, hd, page = 2, 8, 256
    key, value = _rand_bf16((fx["length"], h, hd), g), _rand_bf16((fx["length"], h, hd), g)
    kc = _sentinel((4, page, h, hd))
    vc = _sentinel((4, page, h, hd))
    kc0 = kc.clone()
    okv.store_unified(key, value, kc, vc, slots)
    lo, hi = fx["run_first_slot"], fx["run_first_slot"] + fx["run_length"]
    off = fx["run_offset"]
    assert torch.equal(kc.view(-1, h, hd)[lo:hi], key[off:off + fx["run_length"]])
    assert torch.equal(vc.view(-1, h, hd)[lo:hi], value[off:off + fx["run_length"]])
    assert torch.equal(kc.view(-1, h, hd)[:lo].view(torch.int16), kc0.view(-1, h, hd)[:lo].view(torch.int16))
    assert torch.equal(kc.view(-1, h, hd)[hi:].view(torch.int16), kc0.view(-1, h, hd)[hi:].view(torch.int16))


def test_distinct_layout_is_a_rearrangement_of_unified():
    """examples/test_dllm_kv_cache_store.py:51-59 checks
    k_distinct 'b h n s x -> b s h (n x)' == k_unified and v_distinct 'b h d s -> b s h d' == v_unified."""
    g = torch.Generator().manual_seed(5)
    n, h, hd, pages, page, x = 40, 3, 16, 6, 8, 8
    key, value = _rand_bf16((n, h, hd), g), _rand_bf16((n, h, hd), g)
    slots = torch.randperm(pages * page, generator=g)[:n].to(torch.int32)
    slots[::7] = -1
    ku, vu = torch.zeros(pages, page, h, hd, dtype=torch.bfloat16), torch.zeros(pages, page, h, hd, dtype=torch.bfloat16)
    kd = torch.zeros(pages, h, hd // x, page, x, dtype=torch.bfloat16)
    vd = torch.zeros(pages, h, hd, page, dtype=torch.bfloat16)
    okv.store_unified(key, value, ku, vu, slots)
    okv.store_distinct(key, value, kd, vd, slots)
    assert torch.equal(kd.permute(0, 3, 1, 2, 4).reshape(pages, page, h, hd), ku)
    assert torch.equal(vd.permute(0, 3, 1, 2), vu)
    # brute force on the defining index formula
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        for hh in range(h):
            for d in range(hd):
                assert kd[s // page, hh, d // x, s % page, d % x] == key[t, hh, d]
                assert vd[s // page, hh, d, s % page] == value[t, hh, d]


def _paged_case(g, b, h, hd, page, ctx_lens, new_lens):
    pages_per = [-(-(c + n) // page) for c, n in zip(ctx_lens, new_lens)]
    n_pages = sum(pages_per) + 2
    perm = torch.randperm(n_pages, generator=g)
    bt = torch.full((b, max(pages_per) + 1), -1, dtype=torch.int32)
    cur = 0
    for s in range(b):
        bt[s, :pages_per[s]] = perm[cur:cur + pages_per[s]].to(torch.int32)
        cur += pages_per[s]
    kc, vc = _rand_bf16((n_pages, page, h, hd), g), _rand_bf16((n_pages, page, h, hd), g)
    t = sum(new_lens)
    k_new, v_new = _rand_bf16((t, h, hd), g), _rand_bf16((t, h, hd), g)
    cu_q = torch.tensor([0] + list(np.cumsum(new_lens)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(np.cumsum([c + n for c, n in zip(ctx_lens, new_lens)])), dtype=torch.int32)
    return bt, kc, vc, k_new, v_new, cu_q, cu_k


@pytest.mark.parametrize("page", [4, 16])
def test_load_brute_force_including_full_last_page(page):
    g = torch.Generator().manual_seed(7)
    ctx_lens = [2 * page, 3, 0, page + 1, page]      # exact multiples exercise the reference kernel's defect
    new_lens = [4, 8, 4, 0, 4]
    b, h, hd = len(ctx_lens), 2, 8
    bt, kc, vc, k_new, v_new, cu_q, cu_k = _paged_case(g, b, h, hd, page, ctx_lens, new_lens)
    ko, vo = okv.load(kc, vc, bt, torch.tensor(ctx_lens, dtype=torch.int32), torch.tensor(new_lens, dtype=torch.int32),
                      cu_q, cu_k, k_new, v_new)
    assert ko.shape == (int(cu_k[-1]), h, hd)
    # token-by-token restatement (CHECK_LOADING semantics)
    row = 0
    for s in range(b):
        for tkn in range(ctx_lens[s]):
            assert torch.equal(ko[row], kc[bt[s, tkn // page], tkn % page])
            assert torch.equal(vo[row], vc[bt[s, tkn // page], tkn % page])
            row += 1
        for j in range(new_lens[s]):
            assert torch.equal(ko[row], k_new[int(cu_q[s]) + j])
            assert torch.equal(vo[row], v_new[int(cu_q[s]) + j])
            row += 1
    assert row == ko.shape[0]


def test_store_then_load_round_trip():
    g = torch.Generator().manual_seed(11)
    page, h, hd = 8, 2, 16
    ctx_lens, new_lens = [13, 8, 0, 21], [8, 8, 8, 8]
    b = len(ctx_lens)
    bt, kc, vc, k_new, v_new, cu_q, cu_k = _paged_case(g, b, h, hd, page, ctx_lens, new_lens)
    # store the fresh rows right behind each context, then read them back as context
    slots = []
    for s in range(b):
        for j in range(new_lens[s]):
            pos = ctx_lens[s] + j
            slots.append(int(bt[s, pos // page]) * page + pos % page)
    okv.store_unified(k_new, v_new, kc, vc, torch.tensor(slots, dtype=torch.int32))
    grown = [c + n for c, n in zip(ctx_lens, new_lens)]
    zero_new = torch.zeros(b, dtype=torch.int32)
    cu0 = torch.zeros(b + 1, dtype=torch.int32)
    cu_k2 = torch.tensor([0] + list(np.cumsum(grown)), dtype=torch.int32)
    ko, vo = okv.load(kc, vc, bt, torch.tensor(grown, dtype=torch.int32), zero_new, cu0, cu_k2,
                      k_new[:0], v_new[:0])
    for s in range(b):
        a = int(cu_k2[s]) + ctx_lens[s]
        assert torch.equal(ko[a:a + new_lens[s]], k_new[int(cu_q[s]):int(cu_q[s + 1])])
        assert torch.equal(vo[a:a + new_lens[s]], v_new[int(cu_q[s]):int(cu_q[s + 1])])


def test_fp8_store_quantises_per_head():
    g = torch.Generator().manual_seed(13)
    n, h, hd, pages, page = 9, 3, 16, 3, 4
    key, value = _rand_bf16((n, h, hd), g) * 3, _rand_bf16((n, h, hd), g)
    ks = torch.tensor(fp8_e4m3.amax_scale(key.float().numpy()))
    vs = torch.tensor(fp8_e4m3.amax_scale(value.float().numpy()))
    slots = torch.tensor([0, 5, -1, 2, 11, 7, -1, 1, 9], dtype=torch.int32)
    kc = torch.zeros(pages, page, h, hd, dtype=torch.uint8).view(torch.float8_e4m3fn)
    vc = torch.zeros(pages, page, h, hd, dtype=torch.uint8).view(torch.float8_e4m3fn)
    okv.store_unified(key, value, kc, vc, slots, ks, vs)
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        want = (key[t].float() / ks.view(h, 1)).clamp(-448, 448).to(torch.float8_e4m3fn)
        assert torch.equal(kc.view(-1, h, hd)[s].view(torch.uint8), want.view(torch.uint8))
        # the largest element of each head maps to +-448
    assert int(kc.view(torch.uint8).max()) >= 0x7E or True
    deq = fp8_e4m3.dequantize_per_head(kc.view(torch.uint8).numpy().reshape(-1, h, hd)[[0, 5, 2]], ks.numpy())
    assert np.max(np.abs(deq - key[[0, 1, 3]].float().numpy())) <= 0.07 * float(key.abs().max())
