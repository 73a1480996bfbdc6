"""Host-side layout helpers that run without a GPU: the cache layouts the
decode loops keep (t5x/examples/t5/layers.py:231-241 is the layout they are
converted from and back to), the validity bitmask of the encoder masks
(t5x/examples/t5/network.py:362-370) and the choice of layout."""

import numpy as np
import pytest
import torch

from t5x_amd import network, ops


@pytest.mark.parametrize('L,n', [(32, 0), (32, 31), (32, 32), (64, 33),
                                 (128, 64), (128, 127), (256, 200),
                                 (256, 256)])
def test_tail_layout_round_trip(L, n):
  """tail_cached_key / tail_cached_value and their inverses on a cache that
  holds n positions: the round trip returns the held positions, zero beyond,
  and the tail block holds exactly the positions of the unfinished block,
  position-major."""
  rs = np.random.RandomState(L + n)
  R, H, D = 3, 2, 64
  k = torch.as_tensor(rs.randn(R, H, D, L).astype(np.float32))
  v = torch.as_tensor(rs.randn(R, H, D, L).astype(np.float32))
  v[..., n:] = 0
  tk = ops.tail_cached_key(k)
  assert tk.shape == (R, H, L + 32, D)
  assert torch.equal(tk[:, :, 5 if L > 5 else 0], k[:, :, :, 5 if L > 5 else 0])
  assert torch.equal(ops.untail_cached_key(tk), k)
  tv = ops.tail_cached_value(v, n)
  assert tv.shape == (R, H, L // 32 + 1, D, 32)
  full, rest = n // 32, n % 32
  for b in range(full):   # finished blocks: [64, 32] slices of the cache
    assert torch.equal(tv[:, :, b], v[..., 32 * b:32 * b + 32])
  tail = tv[:, :, -1].reshape(R, H, 32, D)
  if rest and full < L // 32:
    assert torch.equal(tail[:, :, :rest],
                       v[..., 32 * full:n].transpose(2, 3))
  assert float(tail[:, :, rest:].abs().sum()) == 0
  assert torch.equal(ops.untail_cached_value(tv, n), v)


def test_decode_cache_layout_choice():
  bf, f32 = torch.bfloat16, torch.float32
  assert network.decode_cache_layout(bf, 4, 127) == (3, 128)
  assert network.decode_cache_layout(bf, 8, 256) == (3, 256)
  assert network.decode_cache_layout(bf, 1, 1) == (3, 32)
  assert network.decode_cache_layout(bf, 4, 257) == (2, 288)   # beyond the tail kernels
  assert network.decode_cache_layout(bf, 9, 64) == (2, 64)     # more than 8 beams
  assert network.decode_cache_layout(f32, 4, 127) == (0, 128)  # reference layout
  assert network.decode_cache_layout(f32, 4, 5) == (0, 8)


@pytest.mark.parametrize('E', [1, 31, 32, 33, 100, 512])
def test_valid_bits_packing(E):
  rs = np.random.RandomState(E)
  B = 3
  valid = rs.rand(B, E) > 0.3
  bits = ops.pack_valid_bits(torch.as_tensor(valid))
  assert bits.dtype == torch.int32 and tuple(bits.shape) == (B, (E + 31) // 32)
  words = bits.numpy().astype(np.int64) & 0xFFFFFFFF
  for b in range(B):
    for e in range(E):
      assert bool((words[b, e >> 5] >> (e & 31)) & 1) == bool(valid[b, e])
    for e in range(E, 32 * words.shape[1]):   # padding bits stay clear
      assert not (words[b, e >> 5] >> (e & 31)) & 1
