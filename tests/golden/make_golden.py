"""Writes the golden fixtures of the attention parity tests from the fp32 oracle.

    python tests/golden/make_golden.py

c1_attention.npz: the C1 workload's seeded inputs (bf16 bit patterns) and the fp32 oracle output.
No reference code is imported: the oracle restates the reference path and is pinned by
tests/test_oracle_attention.py.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from diffulex_amd.workloads import make_workload  # noqa: E402
from oracle import attention as oat  # noqa: E402


def main():
    wl = make_workload("c1")
    out = oat.paged_attention_fp32(wl.q, wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.block_tables,
                                   wl.context_lens, wl.cu_seqlens_q, wl.cu_seqlens_q, wl.scale)
    bits = lambda t: t.view(torch.int16).numpy()
    np.savez_compressed(
        os.path.join(HERE, "c1_attention.npz"),
        q_bits=bits(wl.q), k_new_bits=bits(wl.k_new), v_new_bits=bits(wl.v_new),
        k_cache_bits=bits(wl.k_cache), v_cache_bits=bits(wl.v_cache),
        block_tables=wl.block_tables.numpy(), context_lens=wl.context_lens.numpy(),
        cu_seqlens_q=wl.cu_seqlens_q.numpy(), scale=np.float32(wl.scale), out_fp32=out.numpy())


if __name__ == "__main__":
    main()
