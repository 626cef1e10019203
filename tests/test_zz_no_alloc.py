"""dfx_paged_attn_static (scratch in a static device array of the library, no allocation) against
dfx_paged_attn (caller-provided workspace): same kernels, so the same bits.  Runs last: a failure
here must not hide the other GPU tests."""
import ctypes as C

import pytest
import torch

import diffulex_amd as dfx
from diffulex_amd import _lib
from diffulex_amd.workloads import make_workload
from util import ATOL_BF16, ATOL_FP8, max_abs_err, oracle_fp32

pytestmark = pytest.mark.gpu


def _args(wl, **kw):
    a = dict(block_tables=wl.block_tables, context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q,
             cu_seqlens_new=wl.cu_seqlens_q, max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode,
             diffusion_block_size=wl.diffusion_block_size, k_scale=wl.k_scale, v_scale=wl.v_scale)
    a.update(kw)
    return a


def _both(wl, **kw):
    out = torch.full_like(wl.q, float("nan"))
    dfx.paged_attention(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, out=out,
                        static_scratch=True, **_args(wl, **kw))
    torch.cuda.synchronize()
    want = dfx.paged_attention(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, **_args(wl, **kw))
    torch.cuda.synchronize()
    return out, want


def test_static_scratch_entry_point_two_calls_in_a_row(dev):
    """Two calls in a row on the same device array, the second with a smaller input; both cut
    items between workgroups, so counters and partial-result slots are in use."""
    big = make_workload("c3", num_seqs=24, seed=5, device=dev)
    small = make_workload("c3", num_seqs=3, ctx=(100, 700), seed=6, device=dev)
    for wl in (big, small):
        got, want = _both(wl)
        assert torch.equal(got, want)
    cu = big.cu_seqlens_q.tolist()
    got, _ = _both(big)
    for s, w in zip([0, 23], oracle_fp32(big, seqs=[0, 23])):
        assert max_abs_err(got[cu[s]:cu[s + 1]], w) <= ATOL_BF16


def test_static_scratch_other_kernels_and_limit(dev):
    """FP8 KV, the block-causal compact kernel and the generic path through the same array, then a
    shape whose scratch would exceed the static array is refused and launches nothing."""
    for name, over, tol in (("c5", dict(num_seqs=6, ctx=(300, 1500)), ATOL_FP8),
                            ("c4", dict(num_seqs=4, ctx=(200, 900)), ATOL_BF16),
                            ("c1", {}, ATOL_BF16)):
        wl = make_workload(name, device=dev, **over)
        got, want = _both(wl)
        assert torch.equal(got, want)
        assert max_abs_err(got, oracle_fp32(wl)) <= tol
        got, want = _both(wl, flags=_lib.DFX_ATTN_GENERIC_PATH, max_workgroups=7)
        assert torch.equal(got, want)
    wl = make_workload("c1", device=dev)
    out = torch.zeros_like(wl.q)
    with pytest.raises(_lib.DfxError, match="static scratch"):
        dfx.paged_attention(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.scale, out=out,
                            static_scratch=True, **_args(wl, max_workgroups=4096))
    torch.cuda.synchronize()
    assert not out.any()
