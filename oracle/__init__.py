"""CPU oracle: a numpy restatement of the reference's decode-step arithmetic.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the product:
only tests, the smoke check and the CPU-baseline leg of the benchmark may import
it, and only as the checker.  The product path (package ``tunix_amd``) never
imports it and fails loudly when its HIP library is missing.

Every function cites the reference file:line (relative to the reference tree)
whose arithmetic it restates.  Pinning status per function group:

* masks / positions / padding / eos finders ............ pinned by the golden
  arrays held in the reference's own tests (tests/generate/utils_test.py:91-179,
  tests/generate/sampler_test.py:1095-1132).
* dense Llama3 / Qwen3 / Qwen3-MoE forward, KV-cache decode == full forward ...
  pinned against ``transformers`` modelling code with random weights (fp32) and
  by closed forms / brute force in fp64.
* LoRA delta ............................................ pinned by the merged-
  weight identity  x W + (x A) B s == x (W + A B s).
* int4 unpack / dequantise .............................. pinned exhaustively
  (all 16 nibbles x all bf16 scales of a sampled set; pack o unpack = id).
* int4 QUANTISE calibration constant (absmax / 7.5) ..... parity unpinned: the
  arithmetic lives in the third-party module ``qwix`` (constraint qwix>=0.1.6,
  pyproject.toml:48, not vendored, not installed here).  It is a parameter.
* threefry2x32 block function ........................... pinned by the
  Random123 known-answer vectors.
* jax.random wiring around it (PRNGKey, fold_in, partitionable counters,
  bits->uniform->gumbel) ................................ parity unpinned: JAX
  is not installed; restated from the published algorithm.
"""
