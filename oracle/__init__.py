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
* JAX's key / counter word order, partitionable bit generation and the
  bits->[0, 1) map ....................................... pinned by the values
  JAX's documentation prints for split(PRNGKey(0)), normal(key(42)) and
  uniform(key(0)).
* fold_in's counter words, gumbel's clamp, categorical's use of them ... parity
  unpinned: JAX is not installed and no published value covers them; restated
  from the published algorithm.
* selective_log_softmax (scoring) ........................ pinned by closed forms
  (NaN / inf / clip cases, logsumexp form).
"""
