"""CPU oracle for the dLLM decoding hot path: TEST INFRASTRUCTURE ONLY.

This package restates, in plain numpy / fp32 torch on the CPU, what the
reference's operators compute on this path.  It exists so that the HIP kernels
can be checked against it.  Nothing in ``diffulex_amd`` may import it; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and there only as the checker / the timed CPU baseline.

Every function cites the reference lines it follows.  How each one is pinned
(what independent fact a plausible mistake in it would violate):

* ``fp8_e4m3.encode_e4m3fn`` / ``decode_e4m3fn``: exhaustive comparison with
  the library cast ``torch.Tensor.to(torch.float8_e4m3fn)`` over all 65 536
  bf16 bit patterns, and all 256 codes for decoding
  (tests/test_oracle_fp8.py).
* ``kv_cache.store_unified`` / ``store_distinct`` / ``load``: brute-force
  pure-Python loops on tiny inputs, sentinel-fill invariants (untouched slots
  unchanged, negative slots ignored), the distinct<->unified rearrangement
  identity the reference's example script checks, the store->load round trip,
  and the slot-mapping recipe / captured slot mapping held by the reference's
  example scripts (tests/test_oracle_kv_cache.py).
* ``attention.paged_attention_fp32``: the library routine
  ``torch.nn.functional.scaled_dot_product_attention`` in fp32 on K/V gathered
  the way the reference's test oracle gathers them, a triple Python loop on
  tiny inputs, and invariants (V == 1 gives O == 1, permuting physical pages
  together with the block table is a no-op, re-paging the same context with a
  different page size is a no-op, block-causal with a single block equals
  bidirectional) (tests/test_oracle_attention.py).
* Parity unpinned: the bit-level rounding of the reference's TileLang /
  flash-attn kernels (bf16 P, exp2 fast-math).  The reference's own tests accept
  1e-2 against a naive SDPA, so nothing here depends on it.
"""
