"""CPU tests of the library's host-side logic: exported symbols, argument checking, the
host/device helper code (FP8 quantiser, bf16 rounding) and the work partition."""
import ctypes as C
import re
import os
import subprocess

import numpy as np
import pytest
import torch

from diffulex_amd import _lib
from oracle import fp8_e4m3
import hosthooks

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "diffulex_amd.h")).read()
    declared = set(re.findall(r"\b(dfx_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    lib = _lib.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.dfx_abi_version() == _lib.DFX_ABI_VERSION
    assert lib.dfx_status_string(0) == b"ok"
    assert lib.dfx_status_string(-2) == b"unsupported shape"


def test_operator_library_loads_and_defines_every_operator():
    """The PyTorch operator library (csrc/torch_ext.cpp) links against the kernel library and
    registers its operators; nothing is computed without a GPU."""
    ops = _lib.ops()
    for name in ("paged_attention", "paged_attention_workspace_bytes", "paged_attention_plan_bytes",
                 "paged_attention_plan", "stream_capture_id", "kv_store_unified", "kv_store_distinct", "kv_load",
                 "rope_kv_store", "build_decode_metadata"):
        assert hasattr(ops, name), name
    import torch
    if not torch.cuda.is_available():
        with pytest.raises((RuntimeError, NotImplementedError)):   # registered for device tensors only
            ops.kv_store_distinct(torch.zeros(1, 1, 8), torch.zeros(1, 1, 8), torch.zeros(1, 1, 1, 1, 8),
                                  torch.zeros(1, 1, 8, 1), torch.zeros(1, dtype=torch.int32))


@pytest.mark.parametrize("ctype,mirror", [("dfx_attn_params", _lib.AttnParams), ("dfx_rope_params", _lib.RopeParams),
                                          ("dfx_metadata_params", _lib.MetadataParams)])
def test_struct_layout_matches_header(tmp_path, ctype, mirror):
    """Size and every field offset of the ctypes mirror against what a C compiler makes of the header."""
    names = [f[0] for f in mirror._fields_]
    prints = "".join(f'printf("%zu\\n", offsetof({ctype}, {n}));' for n in names)
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "diffulex_amd.h"\n'
                   f'int main(void){{printf("%zu\\n", sizeof({ctype}));' + prints + 'return 0;}\n')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert got[0] == C.sizeof(mirror)
    assert got[1:] == [getattr(mirror, n).offset for n in names]


def test_rope_argument_errors_do_not_launch():
    lib = _lib.load()
    assert lib.dfx_rope_kv_store(None, None) == -1
    p = _lib.RopeParams()
    p.n_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim, p.max_position = 0, 28, 4, 128, 4096
    assert lib.dfx_rope_kv_store(C.byref(p), None) == 0          # no tokens: nothing to do
    p.n_tokens = 8
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -1         # null pointers
    p.head_dim = 24
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -2         # head_dim not a multiple of 16
    p.head_dim = 128
    p.q = p.k = p.q_out = p.k_out = p.positions = p.cos_sin_cache = 4096
    p.q_stride_token = p.q_out_stride_token = 28 * 128
    p.k_stride_token = p.k_out_stride_token = 4 * 128 - 8
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -1         # key rows overlap
    p.k_stride_token = p.k_out_stride_token = 4 * 128
    p.k_cache = 4096
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -1         # cache without slot_mapping
    p.k_cache = None
    p.q = 4100
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -1         # misaligned
    p.q = 4096
    p.position_index_type = 5
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -1
    p.position_index_type = 0
    p.slot_mapping, p.v, p.v_stride_token, p.k_cache, p.v_cache, p.n_slots = 4096, 4096, 512, 4096, 4096, 64
    p.kv_dtype = 1
    assert lib.dfx_rope_kv_store(C.byref(p), None) == -1         # FP8 cache without scales


def test_argument_errors_do_not_launch():
    lib = _lib.load()
    # null pointers with non-zero sizes
    assert lib.dfx_kv_store_unified(None, None, 512, 512, None, None, None, 0, 4, 16, 4, 128, 0, None, None, None) == -1
    # zero tokens is a no-op
    assert lib.dfx_kv_store_unified(None, None, 512, 512, None, None, None, 0, 0, 16, 4, 128, 0, None, None, None) == 0
    # bad index type / dtype
    assert lib.dfx_kv_store_unified(16, 16, 512, 512, 16, 16, 16, 7, 4, 16, 4, 128, 0, None, None, None) == -1
    assert lib.dfx_kv_store_unified(16, 16, 512, 512, 16, 16, 16, 0, 4, 16, 4, 128, 1, None, None, None) == -1
    p = _lib.AttnParams()
    p.num_seqs, p.num_q_heads, p.num_kv_heads, p.head_dim = 2, 28, 4, 96
    assert lib.dfx_paged_attn_workspace_bytes(C.byref(p)) == -2       # head_dim 96 unsupported
    p.head_dim, p.num_q_heads = 128, 30
    assert lib.dfx_paged_attn_workspace_bytes(C.byref(p)) == -1       # 30 % 4 != 0
    p.num_q_heads, p.max_workgroups, p.max_seqlen_q = 28, 8, 32
    need = lib.dfx_paged_attn_workspace_bytes(C.byref(p))
    # counters + two slots per workgroup of 8 query blocks (224 rows) of 8 fp16 chunks + statistics, hd 128
    assert need == _lib.DFX_WORKSPACE_COUNTER_BYTES + 2 * 8 * 8 * (8 + 1) * 64 * 16
    assert lib.dfx_paged_attn(C.byref(p), None) == -1                  # null tensors
    assert lib.dfx_paged_attn_static(C.byref(p), None) == -1           # the same checks, nothing launched
    assert lib.dfx_paged_attn_static(None, None) == -1
    p.max_workgroups = 4096                                            # 302 MB of slots: beyond the static array
    assert lib.dfx_paged_attn_workspace_bytes(C.byref(p)) > _lib.DFX_STATIC_SCRATCH_BYTES
    # (made-up, aligned addresses: the refusal comes before anything touches the device)
    p.q = p.k_new = p.v_new = p.out = p.cu_seqlens_q = p.cu_seqlens_new = 4096
    p.q_stride_token, p.q_stride_head, p.o_stride_token, p.o_stride_head = 3584, 128, 3584, 128
    p.kn_stride_token = p.vn_stride_token = 512
    p.kn_stride_head = p.vn_stride_head = 128
    p.scale, p.diffusion_block_size = 0.5, 32
    assert lib.dfx_paged_attn_static(C.byref(p), None) == _lib.DFX_ERR_SCRATCH_LIMIT
    # the fused store needs a cache and the number of fresh rows; a negative row count is refused
    p.store_slot_mapping, p.num_new_tokens = 4096, 64
    assert lib.dfx_paged_attn_static(C.byref(p), None) == -1          # no cache
    p.store_slot_mapping, p.num_new_tokens = None, -1
    assert lib.dfx_paged_attn_static(C.byref(p), None) == -1


def test_device_quantiser_source_matches_oracle_on_host():
    hooks = hosthooks.load()
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    x = bits.view(np.float32)
    x = np.ascontiguousarray(x[np.isfinite(x)])
    out = np.zeros(x.shape, dtype=np.uint8)
    for scale in (1.0, 0.0123, 3.7, 2.0 ** -20, 11.0, 0.0078125):
        hooks.hook_quantise_e4m3(x.ctypes.data, C.c_float(scale), out.ctypes.data, x.size)
        want = fp8_e4m3.quantize_per_head(x.reshape(-1, 1, 1), np.array([scale], np.float32)).reshape(-1)
        assert np.array_equal(out, want), scale
    codes = np.arange(256, dtype=np.uint8)
    f = np.zeros(256, dtype=np.float32)
    hooks.hook_e4m3_to_f32(codes.ctypes.data, f.ctypes.data, 256)
    want = fp8_e4m3.decode_e4m3fn(codes)
    ok = ~np.isnan(want)
    assert np.array_equal(f[ok].view(np.uint32), want[ok].view(np.uint32)) and np.all(np.isnan(f[~ok]))


def test_bf16_rounding_helper_matches_torch():
    hooks = hosthooks.load()
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    out = np.zeros(x.shape, dtype=np.uint16)
    hooks.hook_bf16_round(x.ctypes.data, out.ctypes.data, x.size)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(out, want)


def _walk(hooks, ctx, q_len, new_len, h_kv, group, rows_per_tile, n_wg):
    ctx, q_len, new_len = (np.ascontiguousarray(a, dtype=np.int32) for a in (ctx, q_len, new_len))
    cap = 200000
    rec = np.zeros((cap, 8), dtype=np.int64)
    n = hooks.hook_walk_segments(ctx.ctypes.data, q_len.ctypes.data, new_len.ctypes.data, len(ctx), h_kv, group,
                                 rows_per_tile, n_wg, rec.ctypes.data, cap)
    assert n <= cap
    return rec[:n]


@pytest.mark.parametrize("seed", range(12))
def test_partition_covers_every_tile_once_and_combine_finds_the_pieces(seed):
    hooks = hosthooks.load()
    rng = np.random.default_rng(seed)
    b = int(rng.integers(1, 40))
    h_kv = int(rng.integers(1, 5))
    group = int(rng.choice([1, 2, 4, 7, 8]))
    rows_per_tile = int(rng.choice([128, 256]))
    n_wg = int(rng.choice([1, 2, 3, 7, 64, 256, 1000]))
    ctx = rng.integers(0, 700, b)
    q_len = rng.choice([0, 32, 64, 96, 200], b)
    new_len = np.where(q_len > 0, q_len, 0)
    if seed % 3 == 0:
        ctx[rng.integers(0, b)] = 0
    rec = _walk(hooks, ctx, q_len, new_len, h_kv, group, rows_per_tile, n_wg)
    ctx32, q32, new32 = (np.ascontiguousarray(a, dtype=np.int32) for a in (ctx, q_len, new_len))
    # expected tiles per item
    seen = {}
    slots_by_item = {}
    slot_owner = {}
    for w, kvh, s, rt, t0, t1, complete, slot in rec.tolist():
        n_tiles = -(-int(ctx[s]) // 64) + -(-int(new_len[s]) // 64)
        assert 0 <= t0 < t1 <= n_tiles
        assert bool(complete) == (t0 == 0 and t1 == n_tiles)
        cover = seen.setdefault((kvh, s, rt), [])
        cover.append((t0, t1))
        if not complete:
            assert slot in (2 * w, 2 * w + 1)
            assert slot not in slot_owner, "a partial slot is written twice"
            slot_owner[slot] = (kvh, s, rt)
            slots_by_item.setdefault((kvh, s, rt), []).append(slot)
    for kvh in range(h_kv):
        for s in range(b):
            n_tiles = -(-int(ctx[s]) // 64) + -(-int(new_len[s]) // 64)
            n_rt = -(-group * int(q_len[s]) // rows_per_tile)
            for rt in range(n_rt):
                if n_tiles == 0:
                    continue
                pieces = sorted(seen[(kvh, s, rt)])
                assert pieces[0][0] == 0 and pieces[-1][1] == n_tiles
                for a, bb in zip(pieces, pieces[1:]):
                    assert a[1] == bb[0]
                # combine pass derives the same slots
                out = np.zeros(4096, dtype=np.int32)
                n = hooks.hook_combine_slots(ctx32.ctypes.data, q32.ctypes.data, new32.ctypes.data, b, h_kv, group,
                                             rows_per_tile, n_wg, kvh, s, rt, out.ctypes.data, 4096)
                want = sorted(slots_by_item.get((kvh, s, rt), []))
                assert sorted(out[:n].tolist()) == want
    assert len(seen) == sum(1 for kvh in range(h_kv) for s in range(b)
                            for rt in range(-(-group * int(q_len[s]) // rows_per_tile))
                            if -(-int(ctx[s]) // 64) + -(-int(new_len[s]) // 64) > 0)


def test_number_of_participating_workgroups():
    """Small batches use fewer workgroups (a cut item costs merge rounds that grow with its pieces),
    never fewer than there are items, never more than launched; large batches use them all."""
    f = hosthooks.load().hook_effective_workgroups
    import math
    for max_tiles in (1, 2, 9, 33, 129, 513, 5000):
        r = math.isqrt(max_tiles)                               # floor(sqrt(max_tiles))
        min_units = max(4, r)
        for n_items in (1, 4, 32, 256, 4096):
            total = n_items * max_tiles
            for n_wg in (1, 64, 256, 512):
                want = max(1, min(n_wg, max(n_items, -(-total // min_units))))
                assert f(total, n_items, max_tiles, n_wg) == want
    assert f(64 * 4 * 21, 256, 33, 256) == 256        # Dream-7B shape, batch 64: every compute unit
    assert f(4 * 33, 4, 33, 256) == 27                # batch 1, 2K context: 132 units at >= 5 per workgroup
    assert f(4 * 513, 4, 513, 256) == 94              # batch 1, 32K context: >= 22 per workgroup


def _visible_tiles(ctx, q_len, new_len, group, rows_per_tile, rt, block_causal, dbs):
    """Brute force: context tiles plus every fresh tile that some query row of row tile rt can see."""
    n_ctx = -(-ctx // 64)
    n_new = -(-new_len // 64)
    if not block_causal:
        return n_ctx + n_new
    rows = range(rt * rows_per_tile, min((rt + 1) * rows_per_tile, group * q_len))
    limit = max(min(new_len, ((r % q_len) // dbs + 1) * dbs) for r in rows)
    return n_ctx + sum(1 for t in range(n_new) if t * 64 < limit)


@pytest.mark.parametrize("ctx,q_len,new_len,group,rpt,dbs", [
    (0, 512, 512, 1, 128, 32), (300, 1024, 1024, 7, 256, 32), (0, 2048, 2048, 2, 256, 64), (70, 256, 256, 4, 256, 32),
    (0, 512, 700, 3, 128, 32), (0, 768, 300, 2, 256, 32), (100, 512, 0, 2, 128, 32), (0, 128, 128, 5, 128, 128),
])
def test_block_causal_row_tiles_own_exactly_the_tiles_they_can_see(ctx, q_len, new_len, group, rpt, dbs):
    hooks = hosthooks.load()
    cap = 200000
    out = np.zeros((cap, 3), dtype=np.int32)
    n = hooks.hook_enumerate_units(ctx, q_len, new_len, group, rpt, 1, dbs, out.ctypes.data, cap)
    want = []
    for rt in range(-(-group * q_len // rpt)):
        nt = _visible_tiles(ctx, q_len, new_len, group, rpt, rt, True, dbs)
        want += [(rt, t, nt) for t in range(nt)]
    assert n == len(want)
    assert out[:n].tolist() == [list(w) for w in want]
    full = hooks.hook_enumerate_units(ctx, q_len, new_len, group, rpt, 0, dbs, out.ctypes.data, 0)
    assert n <= full
    if new_len >= 2 * rpt and q_len >= 2 * rpt:
        assert n < full        # something is skipped


@pytest.mark.parametrize("ctx,q_len,new_len,group,rpt,dbs", [
    (0, 200, 200, 2, 128, 32),      # row tiles straddle heads
    (0, 512, 512, 2, 128, 48),      # block size does not divide the row tile
    (10, 96, 96, 1, 128, 32),       # one partial row tile (the D2F decode shape)
])
def test_block_causal_shapes_outside_the_schedule_keep_every_tile(ctx, q_len, new_len, group, rpt, dbs):
    hooks = hosthooks.load()
    out = np.zeros((100000, 3), dtype=np.int32)
    n = hooks.hook_enumerate_units(ctx, q_len, new_len, group, rpt, 1, dbs, out.ctypes.data, 100000)
    n_tiles = -(-ctx // 64) + -(-new_len // 64)
    assert n == n_tiles * -(-group * q_len // rpt)
    for rt in range(-(-group * q_len // rpt)):   # and that is never fewer than what the rows can see
        assert _visible_tiles(ctx, q_len, new_len, group, rpt, rt, True, dbs) <= n_tiles
    assert out[:n, 2].min() == n_tiles


@pytest.mark.parametrize("seed", range(6))
def test_masked_partition_covers_every_visible_tile_once(seed):
    hooks = hosthooks.load()
    rng = np.random.default_rng(100 + seed)
    b = int(rng.integers(1, 12))
    h_kv, group = int(rng.integers(1, 4)), int(rng.choice([1, 2, 7]))
    rpt = int(rng.choice([128, 256]))
    n_wg = int(rng.choice([1, 3, 64, 256]))
    q_len = rng.choice([0, 96, 256, 512, 1024], b)
    new_len = q_len.copy()
    ctx = rng.integers(0, 400, b)
    ctx32, q32, new32 = (np.ascontiguousarray(a, dtype=np.int32) for a in (ctx, q_len, new_len))
    cap = 400000
    rec = np.zeros((cap, 8), dtype=np.int64)
    n = hooks.hook_walk_segments_masked(ctx32.ctypes.data, q32.ctypes.data, new32.ctypes.data, b, h_kv, group, rpt,
                                        n_wg, 1, 32, rec.ctypes.data, cap)
    assert 0 <= n <= cap
    seen = {}
    for w, kvh, s, rt, t0, t1, complete, slot in rec[:n].tolist():
        nt = _visible_tiles(int(ctx[s]), int(q_len[s]), int(new_len[s]), group, rpt, rt, True, 32)
        assert 0 <= t0 < t1 <= nt and bool(complete) == (t0 == 0 and t1 == nt)
        seen.setdefault((kvh, s, rt), []).append((t0, t1))
    for kvh in range(h_kv):
        for s in range(b):
            for rt in range(-(-group * int(q_len[s]) // rpt)):
                nt = _visible_tiles(int(ctx[s]), int(q_len[s]), int(new_len[s]), group, rpt, rt, True, 32)
                if nt == 0:
                    continue
                pieces = sorted(seen[(kvh, s, rt)])
                assert pieces[0][0] == 0 and pieces[-1][1] == nt
                assert all(a[1] == bb[0] for a, bb in zip(pieces, pieces[1:]))


def _simulate_tree_merge(p, order_rng):
    """Model of the pairwise arrival protocol of finish_cut_item (csrc/attn_common.h): p pieces,
    each carried by its own workgroup, interleaved at the granularity of their memory operations
    in a random order.  Returns (pieces in the state that reached the root, rows written, counters)."""
    counters = {}
    slots = {}            # first piece of a subtree -> frozenset of the pieces in the stored state
    written = []

    def worker(j):
        state = frozenset([j])
        half = 1
        while half < p:
            later = (j & half) != 0
            second = (j & ~(2 * half - 1)) + half
            if not later and second >= p:
                half <<= 1
                continue
            there = False
            if later:
                yield
                there = counters.get(second, 0) == 1
            if not there:
                yield
                slots[j] = state
                yield
                old = counters.get(second, 0)
                counters[second] = old + 1
                there = old == 1
                if not there:
                    return
            yield
            sib = second - half if later else second
            other = slots[sib]
            assert not (other & state), "a piece merged twice"
            lo = j & ~(2 * half - 1)
            assert other == frozenset(range(sib, min(sib + half, p))), "sibling state is not its subtree"
            state = state | other
            yield
            counters[second] = 0
            j = lo
            half <<= 1
        written.append(state)

    live = [worker(j) for j in range(p)]
    while live:
        g = live[order_rng.integers(len(live))]
        try:
            next(g)
        except StopIteration:
            live.remove(g)
    return written, counters


@pytest.mark.parametrize("p", [2, 3, 4, 5, 6, 7, 8, 9, 13, 16, 33])
def test_pairwise_merge_protocol_model(p):
    for seed in range(200):
        written, counters = _simulate_tree_merge(p, np.random.default_rng(seed * 1000 + p))
        assert len(written) == 1, "the rows are written exactly once"
        assert written[0] == frozenset(range(p)), "every piece reaches the root"
        assert all(v == 0 for v in counters.values()), "every counter is left at zero"


# ---- the launch plan's capacity sweep (partition.h: sweep_head) and owners looked up in a table of cut points ----
SWEEP_WHOLE, SWEEP_BEGINS, SWEEP_ENDS, SWEEP_MIN_PIECE = 8, 10, 15, 5


def _sweep(lib, lengths, n_w, cap2):
    prefix = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    out = np.full(n_w + 1, -1, dtype=np.int32)
    ok = lib.hook_sweep_head(prefix.ctypes.data, len(lengths), n_w, int(cap2), out.ctypes.data)
    return prefix, out, bool(ok)


def _range_cost(prefix, a, e):
    """Cost of range [a, e) in half units, by the rule the sweep states."""
    if e <= a:
        return 0
    cost = 2 * (e - a)
    for i in range(len(prefix) - 1):
        lo, hi = int(prefix[i]), int(prefix[i + 1])
        if hi <= lo or hi <= a or lo >= e:
            continue
        if lo < a:
            cost += SWEEP_BEGINS
        elif hi > e:
            cost += SWEEP_ENDS
        else:
            cost += SWEEP_WHOLE
    return cost


@pytest.mark.parametrize("seed", range(12))
def test_plan_sweep_tiles_the_head_and_keeps_its_promises(seed):
    lib = hosthooks.load()
    rng = np.random.default_rng(seed)
    n_seq = int(rng.integers(1, 90))
    lengths = rng.integers(0 if seed % 3 == 0 else 1, int(rng.integers(4, 60)), size=n_seq)
    if lengths.sum() == 0:
        lengths[0] = 7
    n_w = int(rng.integers(2, 80))
    base2 = (2 * int(lengths.sum()) + SWEEP_WHOLE * int((lengths > 0).sum()) + n_w - 1) // n_w
    feasible_before = False
    starts = set(np.concatenate([[0], np.cumsum(lengths)]).tolist())
    for t in range(0, 64, 3):
        cap2 = base2 + base2 * t // 100
        prefix, b, ok = _sweep(lib, lengths, n_w, cap2)
        per_head = int(prefix[-1])
        assert b[0] == 0 and b[-1] == per_head and np.all(np.diff(b) >= 0), (b, cap2)
        assert not (feasible_before and not ok), "a larger capacity cannot fail where a smaller one worked"
        feasible_before = feasible_before or ok
        for w in range(n_w):
            a, e = int(b[w]), int(b[w + 1])
            if e == a:
                assert a in starts or a == per_head, "a workgroup without units only where a sequence begins"
                continue
            if ok or w + 1 < n_w:
                # (an item cut for the second time takes at least one unit whatever the capacity)
                assert _range_cost(prefix, a, e) <= cap2 + SWEEP_BEGINS + SWEEP_ENDS + 2, (w, a, e, cap2)
        # a first cut of an item leaves at least SWEEP_MIN_PIECE units on either side
        for w in range(1, n_w):
            x = int(b[w])
            if x in starts or x == int(b[w - 1]):
                continue
            i = int(np.searchsorted(prefix, x, side="right") - 1)
            lo, hi = int(prefix[i]), int(prefix[i + 1])
            if int(b[w - 1]) <= lo:       # the range that ends here began at or before the item: its first cut
                assert x - lo >= SWEEP_MIN_PIECE and hi - x >= SWEEP_MIN_PIECE, (w, x, lo, hi)


@pytest.mark.parametrize("seed", range(8))
def test_owners_of_a_cut_item_from_a_table_of_cut_points(seed):
    """The attention kernels find the workgroups that hold pieces of a cut item by walking the plan's
    table of cut points; workgroups without units (the sweep leaves them where a sequence begins)
    must never be counted among them."""
    lib = hosthooks.load()
    rng = np.random.default_rng(100 + seed)
    lengths = rng.integers(1, 40, size=int(rng.integers(3, 50)))
    n_w = int(rng.integers(3, 60))
    base2 = (2 * int(lengths.sum()) + SWEEP_WHOLE * len(lengths) + n_w - 1) // n_w
    prefix, b, ok = _sweep(lib, lengths, n_w, base2 + base2 * int(rng.integers(20, 80)) // 100)
    bounds = b.astype(np.int32)
    for i in range(len(lengths)):
        first, last = int(prefix[i]), int(prefix[i + 1]) - 1
        owners = [w for w in range(n_w) if bounds[w] < bounds[w + 1] and bounds[w] <= last and bounds[w + 1] > first]
        assert owners == list(range(owners[0], owners[-1] + 1)), "pieces of an item are held by consecutive workgroups"
        for me in owners:
            wa, wb = C.c_int(-1), C.c_int(-1)
            lib.hook_owners_with_bounds(bounds.ctypes.data, n_w, me, first, last, C.byref(wa), C.byref(wb))
            assert (wa.value, wb.value) == (owners[0], owners[-1]), (i, me, owners)



def test_plan_cache_key_works_on_inference_tensors_and_sees_in_place_updates():
    """The reference's runners create the step's metadata under torch.inference_mode()
    (strategy/block_diffusion/engine/model_runner.py:206, strategy/d2f/engine/model_runner.py:291);
    such tensors have no version counter and asking for it raises.  The key must not."""
    from diffulex_amd.dllm_flash_attn import plan_key, _content_token
    q = torch.zeros(64, 28, 128, dtype=torch.bfloat16)
    k = torch.zeros(64, 4, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 256, 4, 128, dtype=torch.bfloat16)
    tail = (0.1, 32, 0, 32, 0, 0, 0, None, None, None)   # (no rotary embedding inside the launch)

    def meta():
        return (torch.zeros(2, 8, dtype=torch.int32), torch.zeros(2, dtype=torch.int32),
                torch.zeros(3, dtype=torch.int32), torch.zeros(3, dtype=torch.int32))
    with torch.inference_mode():
        m = meta()
        assert all(t.is_inference() for t in m)
        with pytest.raises(RuntimeError):
            m[0]._version
        key = plan_key(q, k, kc, False, tail, m, 0)
        assert key == plan_key(q, k, kc, False, tail, m, 0)          # the layers of one step share the plan
        assert key != plan_key(q, k, kc, False, tail, m, 5)          # a capture gets a plan of its own
        assert key != plan_key(q, k, kc, False, tail, meta(), 0)     # the next step's tensors
        assert _content_token(m[1]) == (m[1].data_ptr(), -1)
    m = meta()
    key = plan_key(q, k, kc, False, tail, m, 0)
    m[1].add_(1)   # ordinary tensors: an in-place update makes a new key
    assert key != plan_key(q, k, kc, False, tail, m, 0)
