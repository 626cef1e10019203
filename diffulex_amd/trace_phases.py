"""Per-workgroup phase times of the bf16 streaming attention kernel (development aid).

Needs a library built with the phase timers compiled in:

    DFX_EXTRA_FLAGS=-DDFX_TRACE python -m diffulex_amd.build
    python -m diffulex_amd.trace_phases [workload]          # c3 by default

In that build thread 0 of every workgroup accumulates clock readings (100 MHz) and leaves them in
the unused upper part of the workspace's counter area (see paged_attn_stream_kernel in
csrc/attn_stream.h for the slots).  Rebuild without the flag afterwards: the timers cost a few
percent.
"""
from __future__ import annotations

import sys

import numpy as np
import torch

import diffulex_amd as dfx
from diffulex_amd import dllm_flash_attn as dfa
from diffulex_amd.workloads import make_workload

TICK_US = 0.01
TRACE_OFF_INTS = 16384      # a.arrivals + 16384 in the kernel
SLOTS = 16


def main(name: str = "c3") -> None:
    wl = make_workload(name, device="cuda")
    caches = [(wl.k_cache, wl.v_cache)] + [(wl.k_cache.clone(), wl.v_cache.clone()) for _ in range(3)]
    out = torch.empty_like(wl.q)

    def step(i):
        kc, vc = caches[i % len(caches)]
        dfx.paged_attention(wl.q, wl.k_new, wl.v_new, kc, vc, wl.scale, out=out, block_tables=wl.block_tables,
                            context_lens=wl.context_lens, cu_seqlens_q=wl.cu_seqlens_q, cu_seqlens_new=wl.cu_seqlens_q,
                            max_seqlen_q=wl.q_len, mask_mode=wl.mask_mode, k_scale=wl.k_scale, v_scale=wl.v_scale)

    for i in range(2000):
        step(i)
    torch.cuda.synchronize()
    n_wg = torch.cuda.get_device_properties(0).multi_processor_count
    runs = []
    for i in range(20):
        step(i)
        torch.cuda.synchronize()
        ws = next(iter(dfa._workspaces.values()))
        raw = ws.view(torch.int32)[TRACE_OFF_INTS:TRACE_OFF_INTS + n_wg * SLOTS * 2].cpu().numpy()
        runs.append(raw.view(np.int64).reshape(n_wg, SLOTS).astype(np.float64))
    tr = np.mean(runs, axis=0)
    if not tr[:, 0].any():
        sys.exit("no timer values: build with DFX_EXTRA_FLAGS=-DDFX_TRACE (bf16 streaming kernel, 8 waves)")
    t0 = tr[:, 0].min()
    life = (tr[:, 4] - tr[:, 0]) * TICK_US
    print(f"launch span {((tr[:, 4].max() - t0) * TICK_US):.1f} us; workgroup lifetime mean {life.mean():.1f}, "
          f"min {life.min():.1f}, max {life.max():.1f} us")
    print(f"prefix {((tr[:, 1] - tr[:, 0]).mean() * TICK_US):.2f}  plan {((tr[:, 2] - tr[:, 1]).mean() * TICK_US):.2f}  "
          f"ring fill + first query rows {((tr[:, 3] - tr[:, 2]).mean() * TICK_US):.2f} us")
    print(f"tile loops {tr[:, 5].mean() * TICK_US:.2f} us for {tr[:, 6].mean():.2f} tiles per workgroup: "
          f"{tr[:, 5].sum() / tr[:, 6].sum() * TICK_US:.3f} us per tile")
    for k, what in ((1, "rows written"), (2, "piece stored"), (3, "pieces merged")):
        n = tr[:, 9 + k].sum()
        print(f"{what:14s}: {tr[:, 9 + k].mean():.2f} per workgroup, {tr[:, 6 + k].sum() / max(n, 1) * TICK_US:.2f} us each")
    print(f"further items opened: {tr[:, 13].mean() * TICK_US:.2f} us per workgroup")


if __name__ == "__main__":
    main(*sys.argv[1:2])
