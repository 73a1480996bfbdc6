"""t5d_beam_topk_static (the entry point that allocates nothing: its per-row
candidates live in an array built into the library) against t5d_beam_topk on
the same inputs, bit for bit, through the C ABI: two calls in a row, the
second with a smaller input, so that what the first call left in the shared
array cannot leak into the second result."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(B, beams, V, k, seed):
  from t5x_amd import _lib
  gen = torch.Generator(device='cuda')
  gen.manual_seed(seed)
  R = B * beams
  logits = torch.randn((R, V), generator=gen, device='cuda') * 3.0
  # ties across rows and inside rows: both paths must break them the same way
  logits[:, 7] = logits[:, 3]
  logits[R // 2] = logits[0]
  live = torch.randn((B, beams), generator=gen, device='cuda')
  s = _lib.stream_handle()

  def outputs():
    return (torch.full((B, k), float('nan'), device='cuda'),
            torch.full((B, k), -1, dtype=torch.int32, device='cuda'),
            torch.full((R,), float('nan'), device='cuda'),
            torch.full((R,), float('nan'), device='cuda'))

  want = outputs()
  scratch = torch.empty((2 * R * k,), dtype=torch.int32, device='cuda')
  _lib.call('t5d_beam_topk', s, logits.data_ptr(), live.data_ptr(),
            want[0].data_ptr(), want[1].data_ptr(), want[2].data_ptr(),
            want[3].data_ptr(), scratch.data_ptr(), B, beams, V, k)
  got = outputs()

  def static_call():
    _lib.call('t5d_beam_topk_static', s, logits.data_ptr(), live.data_ptr(),
              got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(),
              got[3].data_ptr(), B, beams, V, k)
    torch.cuda.synchronize()

  torch.cuda.synchronize()
  static_call()   # the first call on a device looks the array's address up
  # What the driver reports as free device memory (the library calls HIP
  # directly, so torch's allocator statistics would not see a hipMalloc of
  # its own); nothing else runs between the two readings.
  free_before, _ = torch.cuda.mem_get_info()
  static_call()
  free_after, _ = torch.cuda.mem_get_info()
  assert free_after == free_before
  for g, w in zip(got, want):
    np.testing.assert_array_equal(g.cpu().numpy(), w.cpu().numpy())
  assert int(got[1].min()) >= 0


def test_static_workspace_matches_caller_workspace_twice():
  print('t5d_beam_topk_static: B=32 beams=4 V=32128 k=8', flush=True)
  _both(32, 4, 32128, 8, seed=0)
  print('t5d_beam_topk_static: B=5 beams=2 V=1000 k=4 (smaller)', flush=True)
  _both(5, 2, 1000, 4, seed=1)


def test_static_workspace_rejects_sizes_beyond_its_limit():
  from t5x_amd import _lib
  x = torch.zeros(16, device='cuda')
  with pytest.raises(_lib.T5DError, match='exceed the built-in workspace'):
    _lib.call('t5d_beam_topk_static', _lib.stream_handle(), x.data_ptr(),
              x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(),
              x.data_ptr(), 2048, 1, 32128, 16)
