"""NumPy restatement of t5x/binary_search.py (test oracle, not product code).

Each function cites the reference lines it follows.  The 32-step bit-pattern
search is kept literally so that the HIP kernels' closed forms (k-th order
statistic) are checked against the reference *algorithm*, not against another
copy of the closed form.
"""

import numpy as np

_I32 = np.int32


def int32_bsearch(batch_shape, predicate):
  """Largest int32 for which `predicate` is False (t5x/binary_search.py:28-71)."""
  current_bits = np.zeros(batch_shape, dtype=_I32)
  # Sign bit first: it orders opposite to the other bits (:51-58).
  satisfied = np.asarray(predicate(current_bits), dtype=bool)
  sign = np.where(satisfied, np.uint32(1 << 31), np.uint32(0)).astype(np.uint32)
  current_bits = current_bits | sign.view(_I32).reshape(current_bits.shape)
  for i in range(31):  # :60-70
    bit = _I32(1 << (30 - i))
    midpoint = current_bits | bit
    satisfied = np.asarray(predicate(midpoint), dtype=bool)
    current_bits = current_bits | np.where(satisfied, _I32(0), bit)
  return current_bits.astype(_I32)


def _monotonic_int32_to_float32_bit_pattern(x):
  """int32 -> float32 bit pattern, order preserving (t5x/binary_search.py:74-101)."""
  x = np.asarray(x, dtype=_I32)
  non_sign_bits = _I32((1 << 31) - 1)
  return x ^ np.where(x < 0, non_sign_bits, _I32(0))


def _monotonic_int32_to_float32(x):
  """t5x/binary_search.py:104-118."""
  return _monotonic_int32_to_float32_bit_pattern(x).astype(_I32).view(np.float32)


def float32_bsearch(batch_shape, predicate):
  """Largest finite float32 for which `predicate` is False (:121-164)."""
  exponent_bits = _I32((1 << 31) - (1 << (31 - 8)))

  def int32_predicate(x):
    x = _monotonic_int32_to_float32_bit_pattern(x)
    is_finite = (x & exponent_bits) != exponent_bits
    predicate_on_nonfinite = x >= 0
    x_float32 = x.astype(_I32).view(np.float32)
    with np.errstate(invalid='ignore'):
      p = np.asarray(predicate(x_float32), dtype=bool)
    return np.where(is_finite, p, predicate_on_nonfinite)

  result = int32_bsearch(batch_shape, int32_predicate)
  return _monotonic_int32_to_float32(result)


def topk_mask(x, k, replace_val):
  """Everything but the top k per row becomes replace_val; ties at the cutoff
  all survive (t5x/binary_search.py:167-227)."""
  x = np.asarray(x)
  batch_shape = tuple(x.shape[:-1])

  def predicate(threshold):
    threshold = -threshold
    count_gt = np.sum(x > threshold[..., None], axis=-1)
    return count_gt >= k

  cutoff = -float32_bsearch(batch_shape, predicate)
  return np.where(x >= cutoff[..., None], x, np.full_like(x, replace_val))


def softmax(x, axis=-1):
  """jax.nn.softmax: exp(x - max) / sum(exp(x - max))."""
  x = np.asarray(x)
  m = np.max(x, axis=axis, keepdims=True)
  e = np.exp(x - m)
  return e / np.sum(e, axis=axis, keepdims=True)


def topp_mask(logits, p, replace_val):
  """Smallest set of logits with probability mass >= p (:230-299)."""
  logits = np.asarray(logits)
  batch_shape = tuple(logits.shape[:-1])
  probs = softmax(logits, axis=-1)

  def predicate(threshold):
    mass = np.sum(
        np.where(probs >= threshold[..., None], probs, probs.dtype.type(0)),
        axis=-1)
    return mass < p

  threshold = float32_bsearch(batch_shape, predicate)
  return np.where(probs >= threshold[..., None], logits,
                  np.full_like(logits, replace_val))
