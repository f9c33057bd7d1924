"""CPU oracle for the KV-cache hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, on the CPU and with plain torch / numpy, the semantics
of the reference's KV-cache path so that the HIP kernels can be checked against
it.  Nothing here is product code: only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import it, and only as the
checker.  The product package never imports ``oracle``.

Modules
-------
cache_ref      contiguous caches of the reference (``pace/llm/cache.py``)
attention_ref  attention semantics (``pace/ops/backends/native.py:32-47``,
               ``csrc/ops/kernels/attention_kernels.cpp:162-257``) and the
               4-D causal mask the models build (``pace/llm/models/llama.py:284-310``)
rope_ref       rotary embedding (``pace/ops/rotary_embedding.py``): tables, row
               selection and the rotation with its bf16 rounding sequence
speculative_ref  acceptance of speculated tokens and the rollback length for one
               sequence (``pace/llm/generator.py:669-713``)
paged_ref      contiguous-semantics model of the block-paged operations
               (append by slot, gather, truncate, evict, compact)

Pinning status (what independent evidence fixes each function):
  * cache_ref.*        shapes asserted by the reference's own
                       ``tests/llm_infra/test_cache.py`` + closed forms
                       (``torch.cat`` / prefix) -- pinned.
  * repeat_kv          ``torch.repeat_interleave`` -- pinned.
  * sdpa_native /      fp64 brute force on tiny inputs, row-sum / L=1 /
    sdpa_fp32          mask-shift invariants -- pinned.
  * sdpa_jit_emulated  only to the reference's own 1e-1 bf16 tolerance
                       (``tests/ops/test_sdpa.py:113-127``): the exact oneDNN
                       v3.8 bit pattern is **parity unpinned**.
  * causal_mask_4d     reference delegates to transformers==4.51.3
                       ``AttentionMaskConverter.to_4d``; checked here against
                       the installed transformers' class of the same name
                       (a different release) -- the 4.51.3 behaviour itself
                       is **parity unpinned** by any reference test.
  * rope_ref.*         no reference test exists; complex multiplication in fp64,
                       rotation invariants, integer-bit emulation of the bf16
                       roundings, transformers' inverse frequencies -- pinned.
                       The longrope row-selection rule agrees with the installed
                       transformers' rule on both sides of one point (largest id
                       == original length), where the two differ and the
                       reference is followed as written: that point is
                       **parity unpinned**.
  * speculative_ref.*  brute force against "1 + longest common prefix" -- pinned.
  * paged_ref.*        row permutations of the pinned contiguous cache; checked
                       against ``DynamicKVCacheRef`` replay of surviving tokens.
"""
