"""CPU oracle for the T5X autoregressive decode path.

TEST INFRASTRUCTURE ONLY.  Everything under this package is a NumPy restatement
of the reference algorithms, written to be read next to the reference source
and used as the checker for the HIP path.  Only the test-suite, the smoke check
and the ``cpu_baseline`` leg of the benchmark may import it; the product
package never does.

Pinned by (see tests/test_oracle_*.py): every literal known-answer vector the
reference's own tests hold for this path (t5x/decoding_test.py,
t5x/binary_search_test.py, t5x/examples/t5/layers_test.py attention/caching
cases, t5x/models_test.py predict_batch cases), closed forms (textbook
softmax-attention, stable sort for top-k, k-th order statistic for topk_mask)
and brute force (full-sequence decoder forward == step-by-step cached decode).

Parity unpinned (no reference vector exists and the library that defines the
behaviour is not vendored in the reference):
  * the GELU variant (assumed tanh-approximate = flax.linen.gelu default);
  * where XLA rounds to bfloat16 inside softmax / einsum / rsqrt;
  * lax.top_k / jnp.argmax tie rule (assumed: lower index wins);
  * jax.random.split / random.categorical key stream (replaced by a supplied
    Gumbel tensor; categorical == argmax(logits + gumbel)).
"""
