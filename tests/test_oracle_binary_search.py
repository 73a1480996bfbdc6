"""Pins oracle/binary_search.py to t5x/binary_search_test.py's literal vectors
and to the closed form the HIP kernels use (k-th order statistic)."""

import numpy as np
import pytest

from oracle import binary_search

I32_MIN = np.iinfo(np.int32).min
I32_MAX = np.iinfo(np.int32).max


def test_int32_bsearch_identity():
  # binary_search_test.py:29-50
  a = np.asarray([1, 43, 79, 2048, 0, 2047, I32_MIN, I32_MIN + 1, I32_MAX,
                  I32_MAX - 1], dtype=np.int32)
  r = binary_search.int32_bsearch(a.shape, lambda x: x > a)
  np.testing.assert_array_equal(a, r)


def test_int32_bsearch_extreme_predicates():
  # binary_search_test.py:52-67
  np.testing.assert_array_equal(
      [I32_MAX],
      binary_search.int32_bsearch((1,), lambda x: np.full_like(x, False)))
  np.testing.assert_array_equal(
      [I32_MIN],
      binary_search.int32_bsearch((1,), lambda x: np.full_like(x, True)))


def test_float32_bsearch():
  # binary_search_test.py:69-82
  a = np.asarray([1.23, 0.0, -0.0, 105.4, -1024, 4.3], dtype=np.float32)
  c = binary_search.float32_bsearch(a.shape, lambda x: x > a)
  assert np.all(a == c), (a, c)


M = -1e10
X = np.asarray([[1.4, 7.9, -4.3, 100, 71, 6, -1e4],
                [8.3, 1.2, 1.3, 1.2, 1.2, 9.7, -100]], dtype=np.float32)
TOPK_TABLE = {  # binary_search_test.py:84-141
    1: [[M, M, M, 100, M, M, M], [M, M, M, M, M, 9.7, M]],
    2: [[M, M, M, 100, 71, M, M], [8.3, M, M, M, M, 9.7, M]],
    3: [[M, 7.9, M, 100, 71, M, M], [8.3, M, 1.3, M, M, 9.7, M]],
    4: [[M, 7.9, M, 100, 71, 6, M], [8.3, 1.2, 1.3, 1.2, 1.2, 9.7, M]],
    5: [[1.4, 7.9, M, 100, 71, 6, M], [8.3, 1.2, 1.3, 1.2, 1.2, 9.7, M]],
    6: [[1.4, 7.9, -4.3, 100, 71, 6, M], [8.3, 1.2, 1.3, 1.2, 1.2, 9.7, M]],
    7: [[1.4, 7.9, -4.3, 100, 71, 6, -1e4],
        [8.3, 1.2, 1.3, 1.2, 1.2, 9.7, -100]],
}


@pytest.mark.parametrize('k', sorted(TOPK_TABLE))
def test_topk_mask_table(k):
  want = np.asarray(TOPK_TABLE[k], dtype=np.float32)
  np.testing.assert_array_equal(want, binary_search.topk_mask(X, k, M))


def test_topk_mask_equals_kth_order_statistic():
  rs = np.random.RandomState(3)
  x = rs.randn(16, 997).astype(np.float32)
  x[:, ::7] = x[:, 1:2]  # plant ties
  for k in (1, 2, 40, 996, 997):
    kth = -np.sort(-x, axis=-1)[:, k - 1:k]
    want = np.where(x >= kth, x, np.float32(-1e7))
    np.testing.assert_array_equal(want,
                                  binary_search.topk_mask(x, k, -1e7))


PROBS = np.asarray([[0.0, 0.7, 0.04, 0.06, 0.2, 0.0],
                    [0.0, 0.2, 0.2, 0.2, 0.3, 0.1]])
TOPP_KEEP = {  # binary_search_test.py:143-209 (1 = kept)
    0.1: [[0, 1, 0, 0, 0, 0], [0, 0, 0, 0, 1, 0]],
    0.3: [[0, 1, 0, 0, 0, 0], [0, 0, 0, 0, 1, 0]],
    0.4: [[0, 1, 0, 0, 0, 0], [0, 1, 1, 1, 1, 0]],
    0.8: [[0, 1, 0, 0, 1, 0], [0, 1, 1, 1, 1, 0]],
    0.95: [[0, 1, 0, 1, 1, 0], [0, 1, 1, 1, 1, 1]],
}


@pytest.mark.parametrize('p', sorted(TOPP_KEEP))
def test_topp_mask_table(p):
  with np.errstate(divide='ignore'):
    logits = np.log(PROBS).astype(np.float32)
  np.testing.assert_allclose(binary_search.softmax(logits), PROBS, rtol=1e-6)
  keep = np.asarray(TOPP_KEEP[p], dtype=bool)
  want = np.where(keep, logits, np.float32(M))
  np.testing.assert_array_equal(want, binary_search.topp_mask(logits, p, M))
