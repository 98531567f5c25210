"""CPU oracle for the decode-time cache hot path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package imports this directory; it is
used by `tests/`, by `__graft_entry__.smoke()` as the checker, and by the `cpu_baseline`
leg of `bench.py`. It restates, in numpy (and plain torch CPU ops for the timed baseline),
the algorithms of the reference's Python files for this path; every function cites the
reference lines it follows.

How each part is pinned (the reference ships no tests, golden vectors or fixtures for
this path, so nothing here is pinned by a reference fixture):

  hf_cache.OracleCache        closed form "last min(n, W) rows of the stream", an independent
                              list-of-rows model, and the worked traces of cache.py for
                              prompts 300/511/700/900 at W=512 (tests/test_oracle_hf_cache.py)
  attention.*                 torch.nn.functional.scaled_dot_product_attention (library
                              routine) on the gathered dense K/V; single-key and constant-V
                              special cases; block-table permutation invariance; split merge
                              == attention over the union (tests/test_oracle_attention.py)
  attention.* softcap / alibi_slopes   torch SDPA with the ALiBi term written out as an additive
                              mask; the cap's formula evaluated by torch on explicit scores and its
                              two limits (huge cap = none, vanishing cap = mean of the visible V
                              rows); varlen form == decode per query (tests/test_oracle_attention.py)
  gla.*                       closed form S_T = sum_t diag(exp(sum_{u>t} g_u)) k_t^T v_t in
                              float64; g=0, k=0 and q=e_i special cases; slot -1 no-op
                              (tests/test_oracle_gla.py)
  attention.metatoken_attention   the one-softmax statement equals window attention merged
                              with the meta-token attention by lse_merge, per head and query;
                              equal-score closed case (tests/test_oracle_attention.py)
  quant.*                     hand-computed rows (ties to even, scale exactly 1), both scale
                              clamps, code saturation, |x - code*scale| <= scale/2, symmetry and
                              power-of-two invariance; bf16 rounding against torch's conversion
                              (tests/test_oracle_quant.py)
  cpu_path.*                  (the torch-CPU restatement timed as bench.py's cpu_baseline) an independent
                              list-of-rows model for the window update, an explicit mask-and-softmax
                              loop for the attention, the float64 unrolled closed form for the GLA
                              step (tests/test_oracle_cpu_path.py)
  paged.*                     brute force over every position of small sequences: the set of
                              resident (block, offset) pairs equals the window; slots are
                              bt[pos//bs]*bs + pos%bs; dense<->paged equivalence
                              (tests/test_oracle_paged.py)

Parity unpinned against the reference's third-party kernels (flash_attn 2.7.3,
flash-linear-attention 0.1, vllm 0.10.0 custom ops, Triton 3.3.1): those packages are
absent here, so their internal rounding order (bf16 P in flash-attn, bf16 k*v product in
the Triton GLA kernel) and vLLM's block-manager free-list order are not reproduced; the
oracle is the fp32/fp64 mathematics those kernels approximate.
"""
