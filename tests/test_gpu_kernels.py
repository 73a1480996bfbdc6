"""Per-kernel parity of the HIP path against the CPU oracle, through the C ABI.

Integer / index results (token ids, beam indices, top-k selections, cache
contents) must be bit-exact.  Floating point: float32 activations within 1e-4,
bfloat16 activations within 2e-2 absolute (one bf16 rounding of an O(1) value
is 4e-3), as stated by the parity rule for this path.
"""

import numpy as np
import pytest
import torch

from oracle import decoding as odec
from oracle import binary_search as obs
from oracle import t5 as ot5

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def dev(x, dtype=None):
  t = torch.as_tensor(np.ascontiguousarray(x), device='cuda')
  return t.to(dtype) if dtype is not None else t


def host(t):
  return t.detach().float().cpu().numpy() if t.is_floating_point() else \
      t.detach().cpu().numpy()


def oracle_dtype(dt):
  return 'bfloat16' if dt == torch.bfloat16 else 'float32'


@pytest.fixture(scope='module')
def ops():
  from t5x_amd import ops as _ops
  return _ops


@pytest.mark.parametrize('dt', [torch.float32, torch.bfloat16])
def test_embed_exact(ops, dt):
  rs = np.random.RandomState(0)
  table = dev(rs.randn(100, 64).astype(np.float32), dt)
  ids = dev(rs.randint(0, 100, size=(17,)).astype(np.int32))
  out = ops.embed(table, ids)
  np.testing.assert_array_equal(host(out), host(table)[host(ids)])


@pytest.mark.parametrize('dt', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('R,d', [(1, 64), (8, 512), (128, 768), (5, 4096),
                                 (1001, 768), (514, 1024), (128, 2048)])
def test_rmsnorm(ops, dt, R, d):
  rs = np.random.RandomState(R + d)
  x = dev(3 * rs.randn(R, d).astype(np.float32), dt)
  scale = dev(1 + 0.1 * rs.randn(d).astype(np.float32), dt)
  out = ops.rmsnorm(x, scale)
  want = ot5.layer_norm(host(x), host(scale), oracle_dtype(dt))
  # two roundings to bf16: allow one bf16 ulp (2^-8 relative) of slack
  np.testing.assert_allclose(host(out), want, atol=TOL[dt], rtol=2**-7 if
                             dt == torch.bfloat16 else 1e-5)


GEMM_SHAPES = [(1, 64, 32), (8, 96, 48), (16, 768, 768), (20, 768, 2304),
               (64, 1024, 1024), (128, 768, 768), (128, 2048, 768),
               (128, 768, 4096)]


@pytest.mark.parametrize('M,K,N', GEMM_SHAPES)
@pytest.mark.parametrize('epi', ['none', 'residual', 'geglu'])
def test_gemm_bf16(ops, M, K, N, epi):
  rs = np.random.RandomState(M * 7 + K + N)
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  a_np = host(a)
  if epi == 'geglu':
    w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    pw = ops.pack_weight(dev(w0), torch.bfloat16, gate_kernel=dev(w1))
    out = ops.gemm(a, pw)
    want = ot5.mlp_block(
        {'wi_0': {'kernel': w0}, 'wi_1': {'kernel': w1},
         'wo': {'kernel': np.eye(N, dtype=np.float32)}}, a_np,
        ('gelu', 'linear'), 'bfloat16')
  else:
    pw = ops.pack_weight(dev(w0), torch.bfloat16)
    res = None
    want = ot5.dense_general(a_np, w0, 'bfloat16')
    if epi == 'residual':
      res = dev(rs.randn(M, N).astype(np.float32), torch.bfloat16)
      want = ot5.bf16_round(want + host(res))
    out = ops.gemm(a, pw, residual=res)
  assert out.shape == want.shape
  np.testing.assert_allclose(host(out), want, atol=2e-2, rtol=2**-7)


BIG_TILES = [(2, 3), (2, 4), (2, 5), (4, 4), (4, 6), (4, 8), (8, 4), (8, 5),
             (8, 8)]


@pytest.mark.parametrize('mp,nt', BIG_TILES)
@pytest.mark.parametrize('wdt', [torch.bfloat16, torch.int8])
def test_gemm_large_tiles(ops, mp, nt, wdt):
  """Every large-tile kernel (t5d_gemm_tiled) against the oracle's dense layer
  and, bit for bit, against t5d_gemm on its small tiles (same split of K over
  the wavefronts, same summation order), for the three epilogues, with rows
  and columns that do not fill the last tile; then K split over 2 and 3
  workgroups (float32 parts added by a second kernel) against the oracle."""
  rs = np.random.RandomState(mp * 10 + nt + (wdt == torch.int8))
  M, K, N = 100, 1088, 16 * (2 * nt + 1)
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  res = dev(rs.randn(M, N).astype(np.float32), torch.bfloat16)
  if wdt == torch.int8:
    k0, k1 = ot5.quantize_int8(w0), ot5.quantize_int8(w1)
  else:
    k0, k1 = w0, w1
  pw = ops.pack_weight(dev(w0), torch.bfloat16, wdt)
  pg = ops.pack_weight(dev(w0), torch.bfloat16, wdt, gate_kernel=dev(w1))
  plain = ot5.dense_general(host(a), k0, 'bfloat16')
  want = {
      'none': plain,
      'residual': ot5.bf16_round(plain + host(res)),
      'geglu': ot5.mlp_block(
          {'wi_0': {'kernel': k0}, 'wi_1': {'kernel': k1},
           'wo': {'kernel': np.eye(N, dtype=np.float32)}}, host(a),
          ('gelu', 'linear'), 'bfloat16')}
  for epi in ('none', 'residual', 'geglu'):
    w = pg if epi == 'geglu' else pw
    r = res if epi == 'residual' else None
    got = ops.gemm_tiled(a, w, mp, nt, residual=r)
    np.testing.assert_allclose(host(got), want[epi], atol=2e-2, rtol=2**-7)
    assert torch.equal(got, ops.gemm(a, w, residual=r)), epi
  f32 = ops.gemm_tiled(a, pw, mp, nt, out_dtype=torch.float32)
  assert torch.equal(f32, ops.gemm(a, pw, out_dtype=torch.float32))
  for k_parts in (2, 3):
    got = ops.gemm_tiled(a, pw, mp, nt, k_parts, residual=res)
    np.testing.assert_allclose(host(got), want['residual'], atol=2e-2,
                               rtol=2**-7)


UNROLLED = ([(mp, nt, 4096, torch.bfloat16) for mp, nt in BIG_TILES] +
            [(mp, nt, 10240, torch.bfloat16) for mp, nt in ((2, 4), (4, 6))] +
            [(4, 4, 2048, torch.int8)])


@pytest.mark.parametrize('mp,nt,K,wdt', UNROLLED)
def test_gemm_large_tiles_with_the_k_loop_unrolled(ops, mp, nt, K, wdt):
  """The large-tile kernels whose K loop is straight-line code (K = 4096,
  10240; int8: 2048) with rows and columns that do not fill the last tile
  (their loads past the matrix edge are clamped, not skipped): bit for bit
  against t5d_gemm on its small tiles, which loops, and against the oracle."""
  rs = np.random.RandomState(mp * 10 + nt + K)
  M, N = 100, 16 * (2 * nt + 1)
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  res = dev(rs.randn(M, N).astype(np.float32), torch.bfloat16)
  k0 = ot5.quantize_int8(w0) if wdt == torch.int8 else w0
  pw = ops.pack_weight(dev(w0), torch.bfloat16, wdt)
  pg = ops.pack_weight(dev(w0), torch.bfloat16, wdt, gate_kernel=dev(w1))
  want = ot5.bf16_round(ot5.dense_general(host(a), k0, 'bfloat16') + host(res))
  got = ops.gemm_tiled(a, pw, mp, nt, residual=res)
  np.testing.assert_allclose(host(got), want, atol=2e-2, rtol=2**-7)
  assert torch.equal(got, ops.gemm(a, pw, residual=res))
  assert torch.equal(ops.gemm_tiled(a, pg, mp, nt), ops.gemm(a, pg))
  f32 = ops.gemm_tiled(a, pw, mp, nt, out_dtype=torch.float32)
  assert torch.equal(f32, ops.gemm(a, pw, out_dtype=torch.float32))


@pytest.mark.parametrize('M,K,N,wdt', [
    (20, 768, 784, torch.bfloat16), (100, 1024, 1040, torch.bfloat16),
    (50, 2048, 784, torch.bfloat16), (33, 2816, 1040, torch.bfloat16),
    (64, 1024, 12304, torch.bfloat16),  # 4 x 2 tiles, 4 pairs, ring of 3
    (50, 2048, 2064, torch.int8), (50, 2048, 6160, torch.int8),
    (64, 2048, 10256, torch.int8), (50, 5120, 2064, torch.int8)])
def test_gemm_small_tiles_with_the_k_loop_unrolled(ops, M, K, N, wdt):
  """The small-tile kernels whose K loop is straight-line code (K = 768,
  1024, 2048, 2816, 5120), with ragged rows and a last column group that is
  not full, against the oracle and, bit for bit, against the same layer with
  one more k-tile pair of zeros appended to K (which takes the looping
  kernel: same products in the same order, plus zeros).  Two of the shapes
  take tiles whose ring of weight tiles is deeper than their ring of
  activation rows and have more k-tile pairs than either (bfloat16 4 x 2 at
  K = 1024, int8 2 x 2 at K = 2048)."""
  rs = np.random.RandomState(M + K + N)
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  res = dev(rs.randn(M, N).astype(np.float32), torch.bfloat16)
  k0 = ot5.quantize_int8(w0) if wdt == torch.int8 else w0
  pw = ops.pack_weight(dev(w0), torch.bfloat16, wdt)
  want = ot5.bf16_round(ot5.dense_general(host(a), k0, 'bfloat16') + host(res))
  got = ops.gemm(a, pw, residual=res)
  np.testing.assert_allclose(host(got), want, atol=2e-2, rtol=2**-7)
  if wdt == torch.bfloat16:
    a_pad = torch.cat([a, torch.zeros((M, 64), dtype=a.dtype, device=a.device)], 1)
    w_pad = np.concatenate([w0, np.zeros((64, N), np.float32)], 0)
    pw_pad = ops.pack_weight(dev(w_pad), torch.bfloat16, wdt)
    assert torch.equal(got, ops.gemm(a_pad.contiguous(), pw_pad, residual=res))


def test_gemm_tiled_rejects_what_it_cannot_run(ops):
  a = dev(np.zeros((16, 64), np.float32), torch.bfloat16)
  pw = ops.pack_weight(dev(np.zeros((64, 64), np.float32)), torch.bfloat16)
  with pytest.raises(ValueError, match='no kernel for a tile'):
    ops.gemm_tiled(a, pw, 3, 3)
  with pytest.raises(ValueError, match='a split over K needs'):
    ops.gemm_tiled(a, pw, 2, 4, 2)  # no residual epilogue


@pytest.mark.parametrize('M,K,N', [(1, 768, 768), (5, 256, 512), (32, 768, 2304),
                                   (128, 768, 768), (128, 768, 4096),
                                   (100, 1024, 1024), (128, 64, 48),
                                   (128, 832, 2304), (20, 1536, 768),
                                   (64, 2048, 2048), (128, 2048, 6144)])
@pytest.mark.parametrize('mode', ['none', 'geglu', 'f32out'])
def test_norm_gemm_equals_rmsnorm_then_gemm(ops, M, K, N, mode):
  """The layer norm fused into the dense kernel against the two-kernel
  sequence: the normalised operand is rounded to bf16 exactly as the
  stand-alone kernel rounds it and the product is summed in the same order, so
  the results agree bit for bit unless the differently ordered sum of squares
  moves 1/rms by an ulp AND that flips a bf16 rounding; and against the
  oracle's layer_norm + dense to the dense-layer tolerance."""
  rs = np.random.RandomState(M + K + N)
  x = dev(rs.randn(M, K).astype(np.float32) * 3, torch.bfloat16)
  scale = dev(1 + 0.1 * rs.randn(K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  kw = {}
  if mode == 'geglu':
    w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    pw = ops.pack_weight(dev(w0), torch.bfloat16, gate_kernel=dev(w1))
  else:
    pw = ops.pack_weight(dev(w0), torch.bfloat16)
    if mode == 'f32out':
      kw['out_dtype'] = torch.float32
  two = ops.gemm(ops.rmsnorm(x, scale), pw, **kw)
  one = ops.gemm(x, pw, norm_scale=scale, **kw)
  diff = (one.float() - two.float()).abs()
  assert float((diff > 0).float().mean()) < 0.02, float((diff > 0).float().mean())
  assert float(diff.max()) <= 2e-2
  xn = ot5.layer_norm(host(x), host(scale), 'bfloat16')
  if mode == 'geglu':
    want = ot5.mlp_block(
        {'wi_0': {'kernel': w0}, 'wi_1': {'kernel': w1},
         'wo': {'kernel': np.eye(N, dtype=np.float32)}}, xn,
        ('gelu', 'linear'), 'bfloat16')
  elif mode == 'f32out':
    want = xn @ ot5.bf16_round(w0)
  else:
    want = ot5.dense_general(xn, w0, 'bfloat16')
  np.testing.assert_allclose(host(one), want, atol=2e-2, rtol=2**-7)


@pytest.mark.parametrize('M,K,N', [(16, 768, 768), (5, 256, 48),
                                   (64, 1024, 3072), (64, 2048, 2048),
                                   (64, 2048, 6144), (128, 1280, 512)])
@pytest.mark.parametrize('geglu', [False, True])
def test_norm_gemm_int8_weights(ops, M, K, N, geglu):
  """The fused layer norm with int8 weights (per-channel scales applied after
  the product, as in the plain kernel): against the two-kernel sequence and
  against the oracle's layer_norm + dense over the dequantised kernel."""
  rs = np.random.RandomState(M + K + N + 1)
  x = dev(rs.randn(M, K).astype(np.float32) * 3, torch.bfloat16)
  scale = dev(1 + 0.1 * rs.randn(K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  q0 = ot5.quantize_int8(w0)
  xn = ot5.layer_norm(host(x), host(scale), 'bfloat16')
  if geglu:
    w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    q1 = ot5.quantize_int8(w1)
    pw = ops.pack_weight(dev(w0), torch.bfloat16, torch.int8,
                         gate_kernel=dev(w1))
    want = ot5.mlp_block({'wi_0': {'kernel': q0}, 'wi_1': {'kernel': q1},
                          'wo': {'kernel': np.eye(N, dtype=np.float32)}},
                         xn, ('gelu', 'linear'), 'bfloat16')
  else:
    pw = ops.pack_weight(dev(w0), torch.bfloat16, torch.int8)
    want = ot5.dense_general(xn, q0, 'bfloat16')
  two = ops.gemm(ops.rmsnorm(x, scale), pw)
  one = ops.gemm(x, pw, norm_scale=scale)
  diff = (one.float() - two.float()).abs()
  assert float((diff > 0).float().mean()) < 0.02, float((diff > 0).float().mean())
  assert float(diff.max()) <= 2e-2
  np.testing.assert_allclose(host(one), want, atol=2e-2, rtol=2**-7)


@pytest.mark.parametrize('M,K,N', [(8, 512, 384), (3, 100, 70), (20, 64, 128),
                                   (8, 512, 1024), (33, 384, 512),
                                   (8, 512, 32128)])
@pytest.mark.parametrize('geglu', [False, True])
def test_norm_gemm_f32(ops, M, K, N, geglu):
  """float32: the layer norm inside the dense kernel (scale folded into the
  activations, 1/rms applied to the finished sums) against the two-kernel
  sequence and against the oracle's layer_norm + dense."""
  if geglu and N > 4096:
    pytest.skip('the logits layer has no gate')
  rs = np.random.RandomState(M + K + N + 5)
  x = rs.randn(M, K).astype(np.float32) * 3
  scale = (1 + 0.1 * rs.randn(K)).astype(np.float32)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  xn = ot5.layer_norm(x, scale, 'float32')
  if geglu:
    w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    pw = ops.pack_weight(dev(w0), torch.float32, gate_kernel=dev(w1))
    want = ot5.mlp_block({'wi_0': {'kernel': w0}, 'wi_1': {'kernel': w1},
                          'wo': {'kernel': np.eye(N, dtype=np.float32)}},
                         xn, ('gelu', 'linear'), 'float32')
  else:
    pw = ops.pack_weight(dev(w0), torch.float32)
    want = ot5.dense_general(xn, w0, 'float32')
  two = ops.gemm(ops.rmsnorm(dev(x), dev(scale)), pw)
  one = ops.gemm(dev(x), pw, norm_scale=dev(scale))
  np.testing.assert_allclose(host(one), host(two), atol=2e-5, rtol=2e-5)
  np.testing.assert_allclose(host(one), want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize('M,K,N', [(128, 768, 32128), (64, 1024, 32128),
                                   (20, 512, 8192), (100, 768, 8208),
                                   (1, 768, 32128), (65, 512, 16400)])
@pytest.mark.parametrize('f32out', [True, False])
def test_norm_gemm_wide_layer(ops, M, K, N, f32out):
  """The vocabulary-sized case of the fused layer norm + dense layer (rows
  resident in LDS, one wavefront sums all of K for its columns): against the
  two-kernel sequence, against the oracle's layer_norm + dense, and bit for
  bit against itself."""
  rs = np.random.RandomState(M + K + N + 9)
  x = dev(rs.randn(M, K).astype(np.float32) * 3, torch.bfloat16)
  scale = dev(1 + 0.1 * rs.randn(K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  pw = ops.pack_weight(dev(w0), torch.bfloat16)
  kw = {'out_dtype': torch.float32} if f32out else {}
  two = ops.gemm(ops.rmsnorm(x, scale), pw, **kw)
  one = ops.gemm(x, pw, norm_scale=scale, **kw)
  assert one.shape == (M, N) and one.dtype == two.dtype
  xn = ot5.layer_norm(host(x), host(scale), 'bfloat16')
  if f32out:
    # float32 sums in a different order agree to 1e-3; a row whose 1/rms
    # moved by an ulp can flip the bf16 rounding of a normalised element,
    # which shows as up to 2e-2 in that row's outputs
    want = xn @ ot5.bf16_round(w0)
    for ref in (host(two), want):
      err = np.abs(host(one) - ref)
      assert float((err > 1e-3 + 1e-4 * np.abs(ref)).mean()) < 2e-3
      np.testing.assert_allclose(host(one), ref, atol=2e-2, rtol=2**-7)
  else:
    want = ot5.dense_general(xn, w0, 'bfloat16')
    diff = (one.float() - two.float()).abs()
    assert float((diff > 0).float().mean()) < 0.02
    np.testing.assert_allclose(host(one), want, atol=2e-2, rtol=2**-7)
  assert torch.equal(one, ops.gemm(x, pw, norm_scale=scale, **kw))


def test_norm_gemm_rejects_what_it_does_not_cover(ops):
  x = dev(np.zeros((4, 64), np.float32))
  pwq = ops.pack_weight(dev(np.zeros((64, 32), np.float32)), torch.bfloat16)
  with pytest.raises(Exception, match='float32'):
    _lib_call_norm_gemm_mixed(ops, x, pwq)
  xb = dev(np.zeros((4, 2112), np.float32), torch.bfloat16)
  pwb = ops.pack_weight(dev(np.zeros((2112, 32), np.float32)), torch.bfloat16)
  with pytest.raises(Exception, match='2048'):
    ops.gemm(xb, pwb, norm_scale=dev(np.ones(2112, np.float32), torch.bfloat16))


@pytest.mark.parametrize('M', [8, 128])
def test_gemm_logits_f32_out(ops, M):
  K, N = 768, 32128
  rs = np.random.RandomState(M)
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  pw = ops.pack_weight(dev(w), torch.bfloat16)
  out = ops.gemm(a, pw, out_dtype=torch.float32)
  want = host(a) @ ot5.bf16_round(w)
  np.testing.assert_allclose(host(out), want, atol=1e-3, rtol=1e-4)
  # bitwise deterministic across launches
  out2 = ops.gemm(a, pw, out_dtype=torch.float32)
  assert torch.equal(out, out2)


@pytest.mark.parametrize('M,K,N', [(16, 768, 768), (64, 2048, 5120),
                                   (128, 768, 2304)])
@pytest.mark.parametrize('geglu', [False, True])
def test_gemm_int8_weights(ops, M, K, N, geglu):
  rs = np.random.RandomState(K + N + M)
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  q0 = ot5.quantize_int8(w0)
  if geglu:
    w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    q1 = ot5.quantize_int8(w1)
    pw = ops.pack_weight(dev(w0), torch.bfloat16, torch.int8,
                         gate_kernel=dev(w1))
    want = ot5.mlp_block({'wi_0': {'kernel': q0}, 'wi_1': {'kernel': q1},
                          'wo': {'kernel': np.eye(N, dtype=np.float32)}},
                         host(a), ('gelu', 'linear'), 'bfloat16')
  else:
    pw = ops.pack_weight(dev(w0), torch.bfloat16, torch.int8)
    want = ot5.dense_general(host(a), q0, 'bfloat16')
  out = ops.gemm(a, pw)
  np.testing.assert_allclose(host(out), want, atol=2e-2, rtol=2**-7)


@pytest.mark.parametrize('M,K,N', [(8, 512, 384), (8, 512, 32128),
                                   (3, 100, 70), (20, 64, 128)])
@pytest.mark.parametrize('epi', ['none', 'residual', 'geglu'])
def test_gemm_f32(ops, M, K, N, epi):
  rs = np.random.RandomState(M + K + N)
  a = rs.randn(M, K).astype(np.float32)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  if epi == 'geglu':
    w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    pw = ops.pack_weight(dev(w0), torch.float32, gate_kernel=dev(w1))
    out = ops.gemm(dev(a), pw)
    want = ot5.gelu(a @ w0) * (a @ w1)
  else:
    pw = ops.pack_weight(dev(w0), torch.float32)
    res = rs.randn(M, N).astype(np.float32) if epi == 'residual' else None
    out = ops.gemm(dev(a), pw, residual=None if res is None else dev(res))
    want = a @ w0 + (0 if res is None else res)
  np.testing.assert_allclose(host(out), want, atol=1e-4, rtol=1e-4)


def test_gemm_rejects_bad_shapes(ops):
  with pytest.raises(ValueError, match='tile'):
    ops.pack_weight(dev(np.zeros((40, 32), np.float32)), torch.bfloat16)


@pytest.mark.parametrize('M', [129, 200, 300])
@pytest.mark.parametrize('mode', ['residual', 'geglu', 'norm', 'norm_geglu'])
def test_dense_layers_beyond_128_rows_run_in_chunks(ops, M, mode):
  """More rows than one launch covers: the same results as the rows would get
  in separate calls of at most 128 (bit for bit), and the oracle's."""
  rs = np.random.RandomState(M)
  K, N = 256, 192
  a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
  w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  w1 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
  geglu = mode.endswith('geglu')
  pw = ops.pack_weight(dev(w0), torch.bfloat16,
                       gate_kernel=dev(w1) if geglu else None)
  kw = {}
  if mode.startswith('norm'):
    kw['norm_scale'] = dev(1 + 0.1 * rs.randn(K).astype(np.float32),
                           torch.bfloat16)
  res = (dev(rs.randn(M, N).astype(np.float32), torch.bfloat16)
         if mode == 'residual' else None)
  out = ops.gemm(a, pw, residual=res, **kw)
  parts = [ops.gemm(a[m:m + 128].contiguous(), pw,
                    residual=None if res is None else res[m:m + 128].contiguous(),
                    **kw) for m in range(0, M, 128)]
  assert torch.equal(out, torch.cat(parts))
  x = host(a)
  if 'norm_scale' in kw:
    x = ot5.layer_norm(x, host(kw['norm_scale']), 'bfloat16')
  if geglu:
    want = ot5.mlp_block({'wi_0': {'kernel': w0}, 'wi_1': {'kernel': w1},
                          'wo': {'kernel': np.eye(N, dtype=np.float32)}}, x,
                         ('gelu', 'linear'), 'bfloat16')
  else:
    want = ot5.dense_general(x, w0, 'bfloat16')
    if res is not None:
      want = ot5.bf16_round(want + host(res))
  np.testing.assert_allclose(host(out), want, atol=2e-2, rtol=2**-7)


def _self_attn_oracle(qkv, ck, cv, rel_emb, t, dtype):
  """Oracle decode-branch attention with selection 'projections'."""
  R, H, D, L = ck.shape
  HD = H * D
  sel = lambda o: np.eye(3 * HD, dtype=np.float32)[:, o * HD:(o + 1) * HD]
  params = {'query': {'kernel': sel(0)}, 'key': {'kernel': sel(1)},
            'value': {'kernel': sel(2)},
            'out': {'kernel': np.eye(HD, dtype=np.float32)}}
  bias = ot5.relpos_bias(rel_emb, L, L, False, dtype)
  x = qkv[:, None, :]
  cache = {'cached_key': ck, 'cached_value': cv, 'cache_index': np.array(t)}
  out, new = ot5.multi_head_attention(params, x, x, None, bias, num_heads=H,
                                      head_dim=D, dtype=dtype, decode=True,
                                      cache=cache)
  return out[:, 0], new


@pytest.mark.parametrize('dt', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('R,H,L,t', [(2, 3, 32, 0), (2, 3, 32, 5),
                                     (4, 6, 32, 31), (3, 2, 128, 77),
                                     (2, 2, 256, 130), (2, 2, 256, 255),
                                     (8, 12, 128, 127)])
def test_self_attention_step(ops, dt, R, H, L, t):
  from t5x_amd import network
  rs = np.random.RandomState(R * 1000 + L + t)
  D = 64
  od = oracle_dtype(dt)
  ck = np.zeros((R, H, D, L), np.float32)
  cv = np.zeros((R, H, D, L), np.float32)
  ck[..., :t] = rs.randn(R, H, D, t)
  cv[..., :t] = rs.randn(R, H, D, t)
  ck, cv = ot5.cast(ck, od), ot5.cast(cv, od)
  qkv = ot5.cast(rs.randn(R, 3 * H * D).astype(np.float32) *
                 np.concatenate([np.full(H * D, 0.125), np.ones(2 * H * D)]),
                 od)
  rel_emb = rs.randn(H, 32).astype(np.float32)
  want, new = _self_attn_oracle(qkv, ck, cv, rel_emb, t, od)

  bucket = network.relative_position_bucket(-np.arange(L), bidirectional=False)
  rel_bias = dev(ot5.cast(rel_emb, od)[:, bucket], dt)
  ck_d, cv_d = dev(ck, dt), dev(cv, dt)
  out = ops.self_attention_step(dev(qkv, dt), ck_d, cv_d, rel_bias,
                                dev(np.array(t, np.int32)))
  np.testing.assert_array_equal(host(ck_d), new['cached_key'])
  np.testing.assert_array_equal(host(cv_d), new['cached_value'])
  np.testing.assert_allclose(host(out), want, atol=TOL[dt], rtol=TOL[dt])


@pytest.mark.parametrize('dt', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('R,H,L,over', [(2, 3, 32, 0), (3, 2, 128, 5),
                                        (2, 2, 256, 1000)])
def test_self_attention_step_past_the_cache_end(ops, dt, R, H, L, over):
  """cache_index >= L (a decode loop longer than its cache): the kernels must
  not turn the index into an address.  Like the reference's one-hot insert and
  clamped bias slice (layers.py:258-303) they insert nothing, leave the caches
  as they are and attend to all L columns with the bias row of position L-1."""
  from t5x_amd import network
  rs = np.random.RandomState(R + L + over)
  D, t = 64, L + over
  od = oracle_dtype(dt)
  ck = ot5.cast(rs.randn(R, H, D, L).astype(np.float32), od)
  cv = ot5.cast(rs.randn(R, H, D, L).astype(np.float32), od)
  qkv = ot5.cast(rs.randn(R, 3 * H * D).astype(np.float32) *
                 np.concatenate([np.full(H * D, 0.125), np.ones(2 * H * D)]),
                 od)
  rel_emb = rs.randn(H, 32).astype(np.float32)
  want, new = _self_attn_oracle(qkv, ck, cv, rel_emb, t, od)
  np.testing.assert_array_equal(new['cached_key'], ck)  # nothing inserted

  bucket = network.relative_position_bucket(-np.arange(L), bidirectional=False)
  rel_bias = dev(ot5.cast(rel_emb, od)[:, bucket], dt)
  # guard bytes behind both caches: an insert at column t would land there
  guard = 2 * D * (over + 1) + 64
  flat_k = torch.zeros(ck.size + guard, dtype=dt, device='cuda')
  flat_v = torch.zeros(cv.size + guard, dtype=dt, device='cuda')
  ck_d = flat_k[:ck.size].view(R, H, D, L).copy_(dev(ck, dt))
  cv_d = flat_v[:cv.size].view(R, H, D, L).copy_(dev(cv, dt))
  out = ops.self_attention_step(dev(qkv, dt), ck_d, cv_d, rel_bias,
                                dev(np.array(t, np.int32)))
  np.testing.assert_array_equal(host(ck_d), ck)
  np.testing.assert_array_equal(host(cv_d), cv)
  assert not bool(flat_k[ck.size:].any()) and not bool(flat_v[cv.size:].any())
  np.testing.assert_allclose(host(out), want, atol=TOL[dt], rtol=TOL[dt])


@pytest.mark.parametrize('B,beams,H,L,t', [(3, 4, 2, 128, 0), (3, 4, 2, 128, 1),
                                           (3, 4, 3, 128, 77),
                                           (2, 4, 2, 128, 127),
                                           (2, 2, 2, 32, 9), (2, 8, 2, 256, 200),
                                           (2, 3, 2, 384, 300),
                                           (32, 4, 12, 128, 64)])
def test_self_attention_step_with_pending_gather(ops, B, beams, H, L, t):
  """The deferred reorder inside the kernel == cache_gather_beams followed by
  the plain step, bit for bit (outputs and both caches).  The first batch item
  keeps its beams in place, the second duplicates one beam (the common case
  after a beam-search step), the rest are random."""
  gen = torch.Generator(device='cuda')
  gen.manual_seed(B * 131 + beams * 17 + L + t)
  R, D, dt = B * beams, 64, torch.bfloat16
  ck = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  cv = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  qkv = torch.randn((R, 3 * H * D), generator=gen, device='cuda').to(dt)
  rel_bias = torch.randn((H, L), generator=gen, device='cuda').to(dt)
  src = torch.randint(0, beams, (B, beams), generator=gen, device='cuda',
                      dtype=torch.int32)
  src[0] = torch.arange(beams, dtype=torch.int32)
  src[1] = 0
  idx = torch.tensor(t, dtype=torch.int32, device='cuda')

  ck_a, cv_a = ck.clone(), cv.clone()
  valid = torch.tensor(t, dtype=torch.int32, device='cuda')
  for c in (ck_a, cv_a):
    ops.cache_gather_beams(c.view(B, beams, H, D, L), src, valid_len=valid)
  want = ops.self_attention_step(qkv, ck_a, cv_a, rel_bias, idx)

  ck_b, cv_b = ck.clone(), cv.clone()
  got = ops.self_attention_step(qkv, ck_b, cv_b, rel_bias, idx,
                                pending_src=src)
  assert torch.equal(got, want)
  # columns 0..t are defined by the algorithm; the rest is never read
  assert torch.equal(ck_b[..., :t + 1], ck_a[..., :t + 1])
  assert torch.equal(cv_b[..., :t + 1], cv_a[..., :t + 1])

  # The same step with the value cache in blocks of 32 positions
  # ([R, H, L/32, 64, 32]), with the deferred reorder and without: identical
  # outputs and, converted back, identical caches.
  ck_c = ck.clone()
  cv_c = ops.block_cached_value(cv).view(R, H, D, L)
  got_c = ops.self_attention_step(qkv, ck_c, cv_c, rel_bias, idx,
                                  pending_src=src, value_blocked=True)
  assert torch.equal(got_c, want)
  assert torch.equal(ck_c[..., :t + 1], ck_a[..., :t + 1])
  assert torch.equal(ops.unblock_cached_value(cv_c)[..., :t + 1],
                     cv_a[..., :t + 1])
  cv_plain = cv.clone()
  ops.cache_gather_beams(cv_plain.view(B, beams, H, D, L), src, valid_len=valid)
  cv_d = ops.block_cached_value(cv_plain).view(R, H, D, L)
  ck_e = ck.clone()
  ops.cache_gather_beams(ck_e.view(B, beams, H, D, L), src, valid_len=valid)
  got_d = ops.self_attention_step(qkv, ck_e, cv_d, rel_bias, idx,
                                  value_blocked=True)
  assert torch.equal(got_d, want)
  assert torch.equal(ops.unblock_cached_value(cv_d)[..., :t + 1],
                     cv_a[..., :t + 1])

  # ... and with the key cache in the same blocks
  ck_f = ops.block_cached_value(ck).view(R, H, D, L)
  cv_f = ops.block_cached_value(cv).view(R, H, D, L)
  got_f = ops.self_attention_step(qkv, ck_f, cv_f, rel_bias, idx,
                                  pending_src=src, value_blocked=True,
                                  key_blocked=True)
  assert torch.equal(got_f, want)
  assert torch.equal(ops.unblock_cached_value(ck_f)[..., :t + 1],
                     ck_a[..., :t + 1])
  assert torch.equal(ops.unblock_cached_value(cv_f)[..., :t + 1],
                     cv_a[..., :t + 1])
  ck_plain = ck.clone()
  ops.cache_gather_beams(ck_plain.view(B, beams, H, D, L), src, valid_len=valid)
  ck_g = ops.block_cached_value(ck_plain).view(R, H, D, L)
  cv_g = ops.block_cached_value(cv_plain).view(R, H, D, L)
  got_g = ops.self_attention_step(qkv, ck_g, cv_g, rel_bias, idx,
                                  value_blocked=True, key_blocked=True)
  assert torch.equal(got_g, want)
  assert torch.equal(ops.unblock_cached_value(ck_g)[..., :t + 1],
                     ck_a[..., :t + 1])
  with pytest.raises(ValueError):
    ops.self_attention_step(qkv, ck_g, cv_g, rel_bias, idx, key_blocked=True)


def _lib_call_norm_gemm_mixed(ops, x, pw):
  """float32 activations with packed bfloat16 weights, straight at the C entry
  (the Python wrapper has no such combination)."""
  from t5x_amd import _lib
  scale = dev(np.ones(x.shape[1], np.float32))
  out = torch.empty((x.shape[0], pw.N), dtype=torch.float32, device='cuda')
  _lib.call('t5d_norm_gemm', _lib.stream_handle(), _lib.F32, pw.w_dtype,
            _lib.F32, x.data_ptr(), scale.data_ptr(), 1e-6, pw.data.data_ptr(),
            None, out.data_ptr(), x.shape[0], x.shape[1], pw.N, 0)


def inherit_slots(slot_of, parents):
  """Host model of the slot rule: slot_of[e] = slot of old beam e, parents[e] =
  old beam that new beam e continues.  Returns (src, dst): the first child of
  a parent keeps the parent's slot, further children take, in order, the slots
  that no new beam reads."""
  K = len(parents)
  src = [int(slot_of[p]) for p in parents]
  dst, taken = [None] * K, set()
  for e in range(K):
    if src[e] not in taken:
      dst[e] = src[e]
      taken.add(src[e])
  free = [x for x in range(K) if x not in set(src)]
  for e in range(K):
    if dst[e] is None:
      dst[e] = free.pop(0)
  return src, dst


@pytest.mark.parametrize('B,beams,H,L,t', [(3, 4, 2, 128, 0), (3, 4, 3, 128, 77),
                                           (2, 2, 2, 32, 9), (2, 8, 2, 256, 200),
                                           (32, 4, 12, 128, 64)])
@pytest.mark.parametrize('blocked', [0, 1, 2])
def test_self_attention_step_with_destination_slots(ops, B, beams, H, L, t,
                                                     blocked):
  """Beams that inherit their parents' slots: with the caches of the old beams
  scattered over the slots (slot_of), the step over (src, dst) slot maps gives
  the outputs of gather-then-step and leaves new beam e's cache in slot
  dst[e]; rows whose slot is inherited are not rewritten (their columns beyond
  t keep the old content), only further children of a parent are copied."""
  gen = torch.Generator(device='cuda')
  gen.manual_seed(B * 71 + beams * 13 + L + t)
  rs = np.random.RandomState(B + beams + t)
  R, D, dt = B * beams, 64, torch.bfloat16
  ck = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  cv = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  qkv = torch.randn((R, 3 * H * D), generator=gen, device='cuda').to(dt)
  rel_bias = torch.randn((H, L), generator=gen, device='cuda').to(dt)
  idx = torch.tensor(t, dtype=torch.int32, device='cuda')
  slot_of = np.stack([rs.permutation(beams) for _ in range(B)])
  parents = rs.randint(0, beams, size=(B, beams))
  parents[0] = np.arange(beams)           # nothing moves
  parents[1] = rs.permutation(beams)      # a re-ranking: nothing is copied
  if B > 2:
    parents[2] = 0                        # one parent, beams - 1 copies
  maps = [inherit_slots(slot_of[b], parents[b]) for b in range(B)]
  src = torch.tensor([m[0] for m in maps], dtype=torch.int32, device='cuda')
  dst = torch.tensor([m[1] for m in maps], dtype=torch.int32, device='cuda')
  for b in range(B):
    s_, d_ = maps[b]
    assert sorted(d_) == list(range(beams))
    assert not ({d for s0, d in zip(s_, d_) if d != s0} & set(s_))
    if b == 1:
      assert s_ == d_

  # reference: caches in beam order, gathered by parent, then the plain step
  so = torch.as_tensor(slot_of, device='cuda').long()
  pa = torch.as_tensor(parents, device='cuda').long()
  rows = (torch.arange(B, device='cuda')[:, None] * beams)
  logical_k = ck[(rows + so).reshape(-1)]   # cache of old beam e
  logical_v = cv[(rows + so).reshape(-1)]
  ck_a = logical_k[(rows + pa).reshape(-1)].clone()
  cv_a = logical_v[(rows + pa).reshape(-1)].clone()
  want = ops.self_attention_step(qkv, ck_a, cv_a, rel_bias, idx)

  # blocked 1: the value cache in blocks of 32 positions, 2: the key cache too
  ck_b = (ops.block_cached_value(ck).view(R, H, D, L) if blocked == 2
          else ck.clone())
  cv_b = (ops.block_cached_value(cv).view(R, H, D, L) if blocked
          else cv.clone())
  got = ops.self_attention_step(qkv, ck_b, cv_b, rel_bias, idx,
                                pending_src=src, pending_dst=dst,
                                value_blocked=blocked > 0,
                                key_blocked=blocked == 2)
  assert torch.equal(got, want)
  ck_out = ops.unblock_cached_value(ck_b) if blocked == 2 else ck_b
  cv_out = ops.unblock_cached_value(cv_b) if blocked else cv_b
  at = (rows + dst.long()).reshape(-1)      # where new beam e's cache is now
  assert torch.equal(ck_out[at][..., :t + 1], ck_a[..., :t + 1])
  assert torch.equal(cv_out[at][..., :t + 1], cv_a[..., :t + 1])
  # inherited slots were not rewritten beyond the new column
  keep = (src == dst).reshape(-1)
  if t + 1 < L and bool(keep.any()):
    assert torch.equal(ck_out[at][keep][..., t + 1:],
                       ck[(rows + src.long()).reshape(-1)][keep][..., t + 1:])


_TAIL_CASES = [
    (3, 4, 2, 128, 0, 40),      # from an empty cache across the first block
    (2, 4, 3, 128, 58, 70),     # two block ends, up to the cache end
    (2, 8, 2, 64, 20, 44),      # 8 beams (the wider workgroup)
    (5, 1, 3, 256, 118, 20),    # rows never reordered: into the second chunk
    (3, 1, 2, 256, 250, 6),     # ... up to the cache end
    (9, 1, 2, 96, 0, 96),       # ... one chunk, every position
    (32, 4, 12, 128, 60, 6),    # the benchmark shape
    (2, 4, 2, 256, 120, 12),    # beams over two chunks
    (3, 4, 2, 128, 27, 8, True),   # gathered in place (no destination slots)
    (2, 8, 1, 96, 60, 6, True),
]


def _random_tail_cases(n, seed):
  """More of the same with random sizes: every workgroup size the launch can
  pick (4, 2 or 1 units), beam counts that are not powers of two, cache
  lengths on both sides of the chunk boundary."""
  rs = np.random.RandomState(seed)
  out = []
  for _ in range(n):
    beams = int(rs.choice([1, 1, 2, 3, 4, 5, 8]))
    B = int(rs.randint(1, 41 if beams <= 4 else 9))
    H = int(rs.randint(1, 13))
    L = int(rs.choice([32, 64, 96, 128, 160, 256]))
    steps = int(rs.randint(3, 11))
    t0 = int(rs.randint(0, L - steps + 1))
    in_place = bool(beams > 1 and L <= 128 and rs.randint(0, 3) == 0)
    out.append((B, beams, H, L, t0, steps, in_place))
  return out


_TAIL_CASES += _random_tail_cases(12, 7)


@pytest.mark.parametrize('B,beams,H,L,t0,steps,in_place', [
    c if len(c) == 7 else c + (False,) for c in _TAIL_CASES])
def test_self_attention_steps_in_the_decode_loop_layout(ops, B, beams, H, L, t0,
                                                         steps, in_place):
  """Consecutive steps on caches in the decode loops' own layout (keys by
  position, values in finished blocks plus a position-major tail, a block
  written when its last position arrives) with the beams re-ranked, dropped
  and duplicated at every step: outputs equal gather-then-step on
  reference-layout caches bit for bit at every step, and so do the caches
  converted back.  beams == 1: rows that are never reordered.  in_place: the
  gather without destination slots (beam e keeps slot e)."""
  gen = torch.Generator(device='cuda')
  gen.manual_seed(B * 7 + beams * 131 + L + t0)
  rs = np.random.RandomState(B + beams + L + t0)
  R, D, dt = B * beams, 64, torch.bfloat16
  # reference-layout caches holding t0 positions (zeros beyond, as a decode
  # leaves them)
  ck = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  cv = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  ck[..., t0:] = 0
  cv[..., t0:] = 0
  rel_bias = torch.randn((H, L), generator=gen, device='cuda').to(dt)
  rows = torch.arange(B, device='cuda')[:, None] * beams
  # tail-layout caches with the beams scattered over the slots
  slot_of = np.stack([np.arange(beams) if in_place else rs.permutation(beams)
                      for _ in range(B)])
  so = torch.as_tensor(slot_of, device='cuda').long()
  phys_k, phys_v = torch.empty_like(ck), torch.empty_like(cv)
  phys_k[(rows + so).reshape(-1)] = ck
  phys_v[(rows + so).reshape(-1)] = cv
  tk = ops.tail_cached_key(phys_k)
  tv = ops.tail_cached_value(phys_v, t0)
  assert torch.equal(ops.untail_cached_key(tk), phys_k)
  assert torch.equal(ops.untail_cached_value(tv, t0), phys_v)
  for t in range(t0, t0 + steps):
    qkv = torch.randn((R, 3 * H * D), generator=gen, device='cuda').to(dt)
    idx = torch.tensor(t, dtype=torch.int32, device='cuda')
    if beams > 1:
      parents = rs.randint(0, beams, size=(B, beams))
      parents[0] = np.arange(beams)         # nothing moves
      if B > 1:
        parents[1] = rs.permutation(beams)  # a re-ranking: nothing is copied
      if in_place:
        maps = [(list(parents[b]), list(range(beams))) for b in range(B)]
      else:
        maps = [inherit_slots(slot_of[b], parents[b]) for b in range(B)]
      src = torch.tensor([m[0] for m in maps], dtype=torch.int32, device='cuda')
      dst = (None if in_place else
             torch.tensor([m[1] for m in maps], dtype=torch.int32,
                          device='cuda'))
      pa = torch.as_tensor(parents, device='cuda').long()
      ck = ck[(rows + pa).reshape(-1)].clone()
      cv = cv[(rows + pa).reshape(-1)].clone()
      slot_of = np.array([m[1] for m in maps])
    else:
      src = dst = None
    want = ops.self_attention_step(qkv, ck, cv, rel_bias, idx)
    got = ops.self_attention_step(qkv, tk, tv, rel_bias, idx, pending_src=src,
                                  pending_dst=dst, tail=True)
    assert torch.equal(got, want), t
    n = min(t + 1, L)
    at = (rows + torch.as_tensor(slot_of, device='cuda').long()).reshape(-1)
    if t % 7 == 0 or t == t0 + steps - 1 or t % 32 in (30, 31, 0):
      assert torch.equal(ops.untail_cached_key(tk)[at][..., :n], ck[..., :n]), t
      assert torch.equal(ops.untail_cached_value(tv, n)[at][..., :n],
                         cv[..., :n]), t


def test_self_attention_step_past_the_cache_end_in_the_decode_loop_layout(ops):
  """A cache index at or beyond L: nothing is inserted and all L columns are
  attended, as the reference-layout kernel does."""
  gen = torch.Generator(device='cuda')
  gen.manual_seed(5)
  R, H, D, L, dt = 6, 2, 64, 64, torch.bfloat16
  ck = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  cv = torch.randn((R, H, D, L), generator=gen, device='cuda').to(dt)
  rel_bias = torch.randn((H, L), generator=gen, device='cuda').to(dt)
  qkv = torch.randn((R, 3 * H * D), generator=gen, device='cuda').to(dt)
  tk, tv = ops.tail_cached_key(ck), ops.tail_cached_value(cv, L)
  for t in (L, L + 3, -1):
    idx = torch.tensor(t, dtype=torch.int32, device='cuda')
    ck_a, cv_a = ck.clone(), cv.clone()
    want = ops.self_attention_step(qkv, ck_a, cv_a, rel_bias, idx)
    got = ops.self_attention_step(qkv, tk, tv, rel_bias, idx, tail=True)
    assert torch.equal(got, want), t
    assert torch.equal(ops.untail_cached_key(tk), ck_a)
    assert torch.equal(ops.untail_cached_value(tv, L), cv_a)
  with pytest.raises(Exception, match='tail layout covers'):
    big = torch.zeros((1, 1, 64, 512 + 32), dtype=dt, device='cuda')
    ops.self_attention_step(
        torch.zeros((1, 192), dtype=dt, device='cuda'), big, big.clone(),
        torch.zeros((1, 512), dtype=dt, device='cuda'),
        torch.tensor(0, dtype=torch.int32, device='cuda'), tail=True)


@pytest.mark.parametrize('dt', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('B,beams,H,E', [(2, 1, 3, 64), (3, 4, 2, 512),
                                         (2, 2, 2, 128), (1, 8, 2, 264),
                                         (2, 3, 2, 1024), (1, 1, 2, 2048)])
def test_cross_attention_step(ops, dt, B, beams, H, E):
  rs = np.random.RandomState(B * 100 + beams * 10 + E)
  D = 64
  od = oracle_dtype(dt)
  if dt == torch.float32 and E > 1024:
    pytest.skip('float32 rows cover at most 1024 positions per workgroup')
  lens = rs.randint(1, E + 1, size=(B,)).astype(np.int32)
  lens[0] = E
  k = ot5.cast(rs.randn(B, E, H, D).astype(np.float32), od)
  v = ot5.cast(rs.randn(B, E, H, D).astype(np.float32), od)
  R = B * beams
  q = ot5.cast(0.125 * rs.randn(R, H * D).astype(np.float32), od)
  eye = np.eye(H * D, dtype=np.float32)
  params = {'query': {'kernel': eye}, 'out': {'kernel': eye}}
  tokens = (np.arange(E)[None, :] < lens[:, None]).astype(np.int32)
  mask = ot5.make_attention_mask(np.ones((R, 1)),
                                 np.repeat(tokens, beams, axis=0) > 0)
  want, _ = ot5.multi_head_attention(
      params, q[:, None, :], None, mask, None, num_heads=H, head_dim=D,
      dtype=od, projected_kv=(np.repeat(k, beams, axis=0),
                              np.repeat(v, beams, axis=0)))
  kd = dev(np.ascontiguousarray(k.transpose(0, 2, 1, 3)), dt)  # [B,H,E,D]
  vd = dev(np.ascontiguousarray(v.transpose(0, 2, 3, 1)), dt)  # [B,H,D,E]
  if dt == torch.bfloat16:
    # blocks of 32 positions: zero-pad E (the padding is beyond every length)
    Ep = (E + 31) // 32 * 32
    kd = ops.tile_cross_key(torch.nn.functional.pad(kd, (0, 0, 0, Ep - E)))
    vd = ops.tile_cross_value(torch.nn.functional.pad(vd, (0, Ep - E)))
  out = ops.cross_attention_step(dev(q, dt), kd, vd, dev(lens), beams)
  np.testing.assert_allclose(host(out), want[:, 0], atol=TOL[dt],
                             rtol=TOL[dt])


@pytest.mark.parametrize('B,beams,H,E', [(3, 4, 2, 512), (32, 4, 12, 512),
                                         (40, 1, 12, 256), (64, 1, 16, 512),
                                         (20, 2, 12, 96)])
def test_cross_attention_work_order(ops, B, beams, H, E):
  """t5d_cross_attention_units: a permutation of the (item, head) pairs that
  carries every item's valid length; with it the two cross-attention kernels
  give bit for bit what they give in the natural order.  For a launch of one
  to two workgroups per CU the heaviest units sit alone, i.e. every position
  that shares its CU with another one (p and p + n_cu) holds a unit no longer
  than any unit that sits alone."""
  rs = np.random.RandomState(B * 7 + H)
  D, d = 64, 256
  lens = rs.randint(0, E + 1, size=(B,)).astype(np.int32)
  lens[0] = E
  lens_d = dev(lens)
  units = ops.cross_attention_units(lens_d, H, E)
  u = host(units).astype(np.int64) & 0xFFFFFFFF
  h, b, n = u & 0xFF, (u >> 8) & 0xFF, u >> 16
  assert sorted(zip(b.tolist(), h.tolist())) == [(i, j) for i in range(B)
                                                 for j in range(H)]
  np.testing.assert_array_equal(n, lens[b])
  n_cu = torch.cuda.get_device_properties(0).multi_processor_count
  total = B * H
  if n_cu < total <= 2 * n_cu:
    pairs = total - n_cu
    alone = n[pairs:n_cu]
    assert alone.size == 0 or max(n[:pairs].max(), n[n_cu:].max()) <= alone.min()
    # the paired: heaviest with lightest
    assert (np.diff(n[:pairs]) <= 0).all() and (np.diff(n[n_cu:]) >= 0).all()
  elif total > 2 * n_cu:
    assert (np.diff(n) <= 0).all()
  k = (0.5 * rs.randn(B, H, E, D)).astype(np.float32)
  v = rs.randn(B, H, D, E).astype(np.float32)
  kd = ops.tile_cross_key(dev(k, torch.bfloat16))
  vd = ops.tile_cross_value(dev(v, torch.bfloat16))
  q = dev(0.125 * rs.randn(B * beams, H * D).astype(np.float32), torch.bfloat16)
  want = ops.cross_attention_step(q, kd, vd, lens_d, beams)
  got = ops.cross_attention_step(q, kd, vd, lens_d, beams, units=units)
  assert torch.equal(got, want)
  x = dev(rs.randn(B * beams, d).astype(np.float32), torch.bfloat16)
  scale = dev(1 + 0.1 * rs.randn(d).astype(np.float32), torch.bfloat16)
  wq = ops.pack_weight(dev((rs.randn(d, H * D) / 16).astype(np.float32)),
                       torch.bfloat16)
  want = ops.cross_attention_step_norm_q(x, scale, wq, kd, vd, lens_d, beams)
  got = ops.cross_attention_step_norm_q(x, scale, wq, kd, vd, lens_d, beams,
                                        units=units)
  assert torch.equal(got, want)


@pytest.mark.parametrize('rows,n,k', [(1, 10, 3), (4, 1000, 8), (3, 128512, 8),
                                      (2, 24, 24), (5, 77, 64)])
def test_top_k_exact_with_ties(ops, rows, n, k):
  rs = np.random.RandomState(n + k)
  x = rs.randint(0, max(2, n // 3), size=(rows, n)).astype(np.float32)
  x[:, ::5] = -1e7
  vals, idx = ops.top_k(dev(x), k)
  wv, wi = odec.top_k(x, k)
  np.testing.assert_array_equal(host(idx), wi)
  np.testing.assert_array_equal(host(vals), wv)


@pytest.mark.parametrize('B,beams,V', [(2, 2, 4), (2, 2, 8), (3, 4, 1000),
                                       (32, 4, 32128), (2, 8, 5000),
                                       (1, 1, 32128)])
def test_beam_topk(ops, B, beams, V):
  rs = np.random.RandomState(B + beams + V)
  logits = (3 * rs.randn(B * beams, V)).astype(np.float32)
  logits[:, 1] = -1e10
  live = np.sort(-np.abs(rs.randn(B, beams)).astype(np.float32), axis=1)
  live[0, 0] = -1e7  # a dead beam: candidates collapse into exact ties
  if B > 1:
    logits[beams:2 * beams] = logits[beams]  # identical rows: cross-beam ties
    live[1, :] = live[1, 0]
  k = 2 * beams
  vals, idx, row_max, row_lse = ops.beam_topk(dev(logits), dev(live), k)
  # log-softmax statistics to tolerance ...
  lp = odec.log_softmax(logits)
  want_lse = -(lp - (logits - logits.max(-1, keepdims=True)))[:, 0]
  np.testing.assert_allclose(host(row_lse), want_lse, atol=1e-5, rtol=1e-6)
  np.testing.assert_array_equal(host(row_max), logits.max(-1))
  # ... and the selection bit-exact given the same log-probs.
  cand = ((logits - host(row_max)[:, None]) - host(row_lse)[:, None]).astype(
      np.float32)
  flat = (cand.reshape(B, beams, V) + live[:, :, None]).astype(
      np.float32).reshape(B, beams * V)
  wv, wi = odec.top_k(flat, k)
  np.testing.assert_array_equal(host(idx), wi)
  np.testing.assert_array_equal(host(vals), wv)


@pytest.mark.parametrize('B,beams,H,E,d', [(3, 4, 2, 512, 768),
                                           (2, 8, 3, 288, 256),
                                           (32, 4, 12, 512, 768),
                                           (2, 1, 2, 64, 1024),
                                           (2, 3, 2, 128, 64),
                                           (2, 4, 2, 384, 832)])
def test_cross_attention_with_fused_norm_and_query_projection(ops, B, beams, H,
                                                              E, d):
  """One kernel against rmsnorm -> dense -> cross_attention_step.  The
  projection uses the dense kernel's split and summation order, so the only
  source of difference is the order of the sum of squares (one ulp of 1/rms,
  which now and then flips a bf16 rounding of a normalised element)."""
  gen = torch.Generator(device='cuda')
  gen.manual_seed(B * 7 + beams + E + d)
  bf = torch.bfloat16
  R, HD = B * beams, H * 64
  rnd = lambda *shape: torch.randn(shape, generator=gen, device='cuda')
  x = (2 * rnd(R, d)).to(bf)
  scale = (1 + 0.1 * rnd(d)).to(bf)
  wq = ops.pack_weight(rnd(d, HD) / (8 * d ** 0.5), bf)
  ck = ops.tile_cross_key(rnd(B, H, E, 64).to(bf))
  cv = ops.tile_cross_value(rnd(B, H, 64, E).to(bf))
  lens = torch.randint(1, E + 1, (B,), generator=gen, device='cuda',
                       dtype=torch.int32)
  lens[0] = E
  q = ops.gemm(ops.rmsnorm(x, scale), wq)
  want = ops.cross_attention_step(q, ck, cv, lens, beams)
  got = ops.cross_attention_step_norm_q(x, scale, wq, ck, cv, lens, beams)
  diff = (got.float() - want.float()).abs()
  assert float((diff > 0).float().mean()) < 0.02, float((diff > 0).float().mean())
  assert float(diff.max()) <= 2e-2, float(diff.max())


@pytest.mark.parametrize('V', [32128, 4096 * 8, 4100, 512, 250])
@pytest.mark.parametrize('pattern', ['one_thread', 'one_wave', 'all_equal',
                                     'descending'])
def test_beam_topk_adversarial_placements(ops, V, pattern):
  """Placements that stress how the row kernel splits the vocabulary over
  lanes: all winners in the registers of one thread (consecutive elements and
  elements 4096 apart), all in one wavefront, a constant row (pure index
  ties), and a sorted row.  Selection must equal the oracle's top_k exactly."""
  B, beams = 2, 4
  k = 2 * beams
  rs = np.random.RandomState(V)
  logits = rs.randn(B * beams, V).astype(np.float32)
  if pattern == 'one_thread':
    hot = [4 * 77 + c for c in range(4)] + [4 * 77 + 4096 * u for u in range(1, 8)]
    hot = [j for j in hot if j < V]
    logits[:, hot] += 20 + rs.rand(B * beams, len(hot)).astype(np.float32)
  elif pattern == 'one_wave':
    hot = np.arange(4 * 64 * 3, min(V, 4 * 64 * 4))[:40]
    logits[:, hot] += 20
  elif pattern == 'all_equal':
    logits[:] = 0.5
  else:
    logits[:] = -np.arange(V, dtype=np.float32)[None, :] / 64
  live = np.sort(-np.abs(rs.randn(B, beams)).astype(np.float32), axis=1)
  if pattern == 'all_equal':
    live[:] = -1.0
  vals, idx, row_max, row_lse = ops.beam_topk(dev(logits), dev(live), k)
  cand = ((logits - host(row_max)[:, None]) - host(row_lse)[:, None]).astype(
      np.float32)
  flat = (cand.reshape(B, beams, V) + live[:, :, None]).astype(
      np.float32).reshape(B, beams * V)
  wv, wi = odec.top_k(flat, k)
  np.testing.assert_array_equal(host(idx), wi)
  np.testing.assert_array_equal(host(vals), wv)
  lp = odec.log_softmax(logits)
  want_lse = -(lp - (logits - logits.max(-1, keepdims=True)))[:, 0]
  np.testing.assert_allclose(host(row_lse), want_lse, atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize('dt', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('B,beams,H,L,valid', [(2, 2, 2, 32, None),
                                               (3, 4, 3, 128, 57),
                                               (2, 8, 1, 64, 64),
                                               (4, 3, 2, 40, 1)])
def test_cache_gather_beams(ops, dt, B, beams, H, L, valid):
  rs = np.random.RandomState(B + beams + L)
  layers = 3
  x = rs.randn(layers, 2, B, beams, H, 64, L).astype(np.float32)
  idx = rs.randint(0, beams, size=(B, beams)).astype(np.int32)
  idx[0] = np.arange(beams)  # identity item is skipped
  t = dev(x, dt)
  before = host(t).copy()
  want = before.copy()
  b = np.arange(B)[:, None]
  nv = L if valid is None else valid
  want[:, :, :, :, :, :, :nv] = before[:, :, b, idx][..., :nv]
  vl = None if valid is None else dev(np.array(valid - 1, np.int32))
  stride = t[0, 0].numel() * t.element_size()
  ops.cache_gather_beams(t[0, 0], dev(idx), valid_len=vl, valid_offset=1,
                         n_tensors=layers * 2, tensor_stride_bytes=stride)
  got = host(t)
  el = 16 // t.element_size()
  nv_pad = min(L, (nv + el - 1) // el * el)
  np.testing.assert_array_equal(got[..., :nv], want[..., :nv])
  # columns past the 16-byte chunk holding the last valid one are untouched
  np.testing.assert_array_equal(got[..., nv_pad:], before[..., nv_pad:])


def test_gather_beams_out_of_place(ops):
  rs = np.random.RandomState(0)
  x = rs.randint(0, 100, size=(3, 4, 129)).astype(np.int32)
  idx = rs.randint(0, 4, size=(3, 8)).astype(np.int32)
  out = ops.gather_beams(dev(x), dev(idx))
  np.testing.assert_array_equal(host(out), x[np.arange(3)[:, None], idx])
  y = rs.randn(3, 4).astype(np.float32)
  out = ops.gather_beams(dev(y), dev(idx))
  np.testing.assert_array_equal(host(out), y[np.arange(3)[:, None], idx])


@pytest.mark.parametrize('V,topk', [(7, 3), (1000, 40), (32128, 40),
                                    (32128, 1), (50, 0)])
@pytest.mark.parametrize('temp', [0.0, 0.7, 1.0])
@pytest.mark.parametrize('rescale', [True, False])
def test_sample_tokens_topk(ops, V, topk, temp, rescale):
  rs = np.random.RandomState(V + topk)
  R = 6
  logits = (2 * rs.randn(R, V)).astype(np.float32)
  logits[:, ::4] = logits[:, 1:2]  # ties, also at the cutoff for small k
  g = odec.GumbelNoise(seed=3).noise(0, (R, V))
  temps = np.full((R,), temp, np.float32)
  tok, lp = ops.sample_tokens(dev(logits), dev(g), dev(temps), topk, 0.0,
                              rescale)
  if temp > 1e-4:
    scaled = (logits / np.maximum(np.float32(temp), np.float32(1e-4))).astype(
        np.float32)
    if topk:
      scaled = obs.topk_mask(scaled, topk, np.float32(-1e7))
    want_tok = np.argmax(scaled + g, axis=-1)
    src = scaled if rescale else logits
    want_lp = odec.log_softmax(src)[np.arange(R), want_tok]
  else:
    want_tok = np.argmax(logits, axis=-1)
    want_lp = (np.zeros(R, np.float32) if rescale else
               odec.log_softmax(logits)[np.arange(R), want_tok])
  np.testing.assert_array_equal(host(tok), want_tok)
  np.testing.assert_allclose(host(lp), want_lp, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize('V', [1000, 32128, 32127])
@pytest.mark.parametrize('topp', [0.3, 0.9])
@pytest.mark.parametrize('rescale', [True, False])
def test_sample_tokens_topp_vocab(ops, V, topp, rescale):
  """Top-p at vocabulary width against the oracle's mask; probabilities near
  the threshold can fall either side of it by a rounding of the softmax, so
  rows whose oracle mask has an element within 1e-6 (relative) of the
  threshold probability are skipped (none with these seeds).  V = 32127 takes
  the generic kernel (rows not 16-byte aligned)."""
  rs = np.random.RandomState(V + int(10 * topp))
  R = 5
  logits = (3 * rs.randn(R, V)).astype(np.float32)
  g = odec.GumbelNoise(seed=5).noise(0, (R, V))
  temp = np.float32(0.8)
  temps = np.full((R,), temp, np.float32)
  tok, lp = ops.sample_tokens(dev(logits), dev(g), dev(temps), 0, topp, rescale)
  scaled = (logits / temp).astype(np.float32)
  masked = obs.topp_mask(scaled, np.float32(topp), np.float32(-1e7))
  want_tok = np.argmax(masked + g, axis=-1)
  src = masked if rescale else logits
  want_lp = odec.log_softmax(src)[np.arange(R), want_tok]
  np.testing.assert_array_equal(host(tok), want_tok)
  np.testing.assert_allclose(host(lp), want_lp, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize('k', [1, 16, 17, 40, 128, 129, 1000])
def test_sample_tokens_topk_cutoff_with_ties(ops, k):
  """The k-th largest as cutoff when it sits inside a run of equal values, for
  k on both sides of the per-wavefront bound's limits and of the candidate
  list's capacity: the kept set is everything >= the k-th largest."""
  V, R = 32128, 3
  rs = np.random.RandomState(k)
  logits = rs.randn(R, V).astype(np.float32)
  logits[0, rs.permutation(V)[:600]] = 5.0     # 600 equal maxima
  logits[1] = np.round(logits[1] * 4) / 4       # heavy ties everywhere
  g = odec.GumbelNoise(seed=k).noise(0, (R, V))
  temps = np.ones((R,), np.float32)
  tok, lp = ops.sample_tokens(dev(logits), dev(g), dev(temps), k, 0.0, True)
  masked = obs.topk_mask(logits, k, np.float32(-1e7))
  want_tok = np.argmax(masked + g, axis=-1)
  want_lp = odec.log_softmax(masked)[np.arange(R), want_tok]
  np.testing.assert_array_equal(host(tok), want_tok)
  np.testing.assert_allclose(host(lp), want_lp, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize('R,V,k', [(6, 32128, 40), (64, 32128, 40),
                                   (3, 32128, 1), (5, 32128, 64),
                                   (128, 4096, 7), (4, 8000, 33)])
def test_sample_tokens_topk_in_two_launches(ops, R, V, k):
  """The top-k choice with a workspace (rows cut into parts that list their own
  k largest, then one workgroup per row on the lists) against the oracle and
  against the one-launch path: same tokens; log-probs to float32 rounding.
  Rows are mixed: plain random rows, ties at the cutoff, a run of equal values
  longer than a part's list (that row falls back to the whole-row path), a
  greedy row (temperature 0), a row whose k largest sit in one part."""
  rs = np.random.RandomState(R + V + k)
  logits = (2 * rs.randn(R, V)).astype(np.float32)
  logits[0, ::4] = logits[0, 1]                       # ties everywhere
  logits[1 % R, rs.permutation(V)[:600]] = 60.0       # 600 equal maxima
  logits[2 % R, :k + 5] += 30.0                       # all winners in part 0
  temps = np.full((R,), 0.7, np.float32)
  if R > 3:
    temps[3] = 0.0                                    # a greedy row
  if R > 4:
    temps[4] = 1.3                                    # its own temperature
  g = odec.GumbelNoise(seed=k).noise(0, (R, V))
  ws = ops.sample_tokens_workspace(R, 'cuda')
  ws.fill_(-7)                                        # contents are irrelevant
  tok, lp = ops.sample_tokens(dev(logits), dev(g), dev(temps), k, 0.0, True,
                              workspace=ws)
  tok1, lp1 = ops.sample_tokens(dev(logits), dev(g), dev(temps), k, 0.0, True)
  scaled = (logits / np.maximum(temps, np.float32(1e-4))[:, None]).astype(
      np.float32)
  masked = obs.topk_mask(scaled, k, np.float32(-1e7))
  want_tok = np.argmax(masked + g, axis=-1)
  want_lp = odec.log_softmax(masked)[np.arange(R), want_tok]
  greedy = temps <= 1e-4
  want_tok[greedy] = np.argmax(logits, axis=-1)[greedy]
  want_lp[greedy] = 0.0
  np.testing.assert_array_equal(host(tok), want_tok)
  np.testing.assert_array_equal(host(tok1), want_tok)
  np.testing.assert_allclose(host(lp), want_lp, atol=1e-5, rtol=1e-5)
  np.testing.assert_allclose(host(lp), host(lp1), atol=2e-6, rtol=2e-6)
  # which rows took the lists: all but the greedy row and the 600-tie row
  counts = host(ws)[:R * 4].reshape(R, 4)
  assert (counts[1 % R] < 0).any() and (counts[0] >= 0).all()
  if R > 3:
    assert (counts[3] < 0).all()


def test_sample_tokens_topp_table(ops):
  # t5x/binary_search_test.py:143-209 through the kernel: with a huge Gumbel
  # bonus on one index the sampled token reveals whether it survived the mask.
  # The reference table uses p equal to exact cumulative masses (0.3, 0.4),
  # where "mass >= p" is decided by the last bit of a float32 softmax sum in
  # the reference as much as here; p is nudged 1e-3 below those boundaries.
  probs = np.asarray([[0.0, 0.7, 0.04, 0.06, 0.2, 0.0],
                      [0.0, 0.2, 0.2, 0.2, 0.3, 0.1]])
  with np.errstate(divide='ignore'):
    logits = np.maximum(np.log(probs), -1e10).astype(np.float32)
  keep_table = {0.1: [[1], [4]], 0.299: [[1], [4]],
                0.399: [[1], [1, 2, 3, 4]], 0.8: [[1, 4], [1, 2, 3, 4]],
                0.95: [[1, 3, 4], [1, 2, 3, 4, 5]]}
  temps = dev(np.ones(2, np.float32))
  for p, keep in keep_table.items():
    for j in range(6):
      g = np.zeros((2, 6), np.float32)
      g[:, j] = 1000.0
      tok, _ = ops.sample_tokens(dev(logits), dev(g), temps, 0, p, True)
      for r in range(2):
        survived = int(host(tok)[r]) == j
        assert survived == (j in keep[r]), (p, r, j)


def test_measurement_aids_fill_and_read(ops):
  """t5d_measure_fill writes the documented pattern over exactly the buffer;
  t5d_measure_read reads it (any shift) without touching it or the sink, and
  both refuse sizes that are not a multiple of 16."""
  from t5x_amd import _lib
  n = 16 * 1000 + 16
  buf = torch.full((n + 64,), 0x5a, dtype=torch.uint8, device='cuda')
  sink = torch.zeros(4, dtype=torch.int32, device='cuda')
  s = _lib.stream_handle()
  _lib.call('t5d_measure_fill', s, buf.data_ptr(), n, 7, 3)
  words = buf[:n].view(torch.int32).view(-1, 4).cpu().numpy()
  np.testing.assert_array_equal(words[:, 0], 7 + np.arange(n // 16))
  np.testing.assert_array_equal(words[:, 1:], np.tile([1, 2, 3], (n // 16, 1)))
  assert bool((buf[n:] == 0x5a).all())
  before = buf.clone()
  for shift, tag in ((0, 0), (2, 5)):
    _lib.call('t5d_measure_read', s, buf.data_ptr(), n, shift, 3,
              sink.data_ptr(), tag)
  torch.cuda.synchronize()
  assert torch.equal(buf, before) and int(sink.abs().sum()) == 0
  with pytest.raises(ValueError, match='t5d_measure_fill'):
    _lib.call('t5d_measure_fill', s, buf.data_ptr(), n + 8, 7, 3)
  with pytest.raises(ValueError, match='tag=6'):
    _lib.call('t5d_measure_read', s, buf.data_ptr(), n, 0, 3, sink.data_ptr(), 6)


def test_gemm_random_shapes_every_tile_choice(ops):
  """t5d_gemm over 80 random shapes (rows 1..128, K a multiple of 32 up to
  4096, N a multiple of 16 up to 12288, bfloat16 and int8 weights, with and
  without a residual): whatever tile the planner picks, the result is the
  dense layer's (float32 products of the same operands on the device as the
  yardstick, tolerance 2e-2 + 2^-7 relative)."""
  rs = np.random.RandomState(2024)
  for case in range(80):
    M = int(rs.choice([1, 5, 16, 20, 32, 48, 50, 64, 96, 100, 128]))
    K = 32 * int(rs.randint(1, 129))
    N = 16 * int(rs.randint(1, 769))
    if K * N > 20e6:
      N = max(16, int(20e6 // K) // 16 * 16)
    int8 = bool(rs.randint(0, 2))
    with_res = bool(rs.randint(0, 2))
    a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
    w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    res = dev(rs.randn(M, N).astype(np.float32), torch.bfloat16) if with_res else None
    if int8:
      q = ot5.quantize_int8(w0)
      w_ref = dev(q['q'].astype(np.float32)) * dev(q['scale'].astype(np.float32))
      pw = ops.pack_weight(dev(w0), torch.bfloat16, torch.int8)
    else:
      w_ref = dev(w0).to(torch.bfloat16).float()
      pw = ops.pack_weight(dev(w0), torch.bfloat16)
    want = (a.float() @ w_ref).to(torch.bfloat16).float()
    if with_res:
      want = (want + res.float()).to(torch.bfloat16).float()
    got = ops.gemm(a, pw, residual=res).float()
    err = (got - want).abs()
    ok = err <= 2e-2 + 2.0**-7 * want.abs()
    assert bool(ok.all()), (case, M, K, N, int8, with_res, float(err.max()),
                            float((~ok).float().mean()))


def test_norm_gemm_random_shapes(ops):
  """t5d_norm_gemm (layer norm + dense in one kernel) over 60 random shapes
  (K a multiple of 64 up to 2048, N a multiple of 16, bfloat16 and int8
  weights, plain and gated-GELU epilogues, bfloat16 and float32 results)
  against the two-kernel sequence t5d_rmsnorm -> t5d_gemm, whose pieces are
  tested against the oracle: same roundings, so within one bfloat16 flip of
  the sums."""
  rs = np.random.RandomState(77)
  for case in range(60):
    M = int(rs.choice([1, 7, 16, 33, 64, 100, 128]))
    K = 64 * int(rs.randint(1, 33))
    N = 16 * int(rs.randint(1, 400))
    int8 = bool(rs.randint(0, 2))
    geglu = bool(rs.randint(0, 2))
    f32_out = (not geglu) and bool(rs.randint(0, 2))
    wdt = torch.int8 if int8 else torch.bfloat16
    a = dev(rs.randn(M, K).astype(np.float32), torch.bfloat16)
    scale = dev((1.0 + 0.1 * rs.randn(K)).astype(np.float32), torch.bfloat16)
    w0 = (rs.randn(K, N) / np.sqrt(K)).astype(np.float32)
    gate = dev((rs.randn(K, N) / np.sqrt(K)).astype(np.float32)) if geglu else None
    pw = ops.pack_weight(dev(w0), torch.bfloat16, wdt, gate_kernel=gate)
    od = torch.float32 if f32_out else torch.bfloat16
    got = ops.gemm(a, pw, norm_scale=scale, out_dtype=od).float()
    want = ops.gemm(ops.rmsnorm(a, scale), pw, out_dtype=od).float()
    err = (got - want).abs()
    ok = err <= 2e-2 + 2.0**-6 * want.abs()
    assert bool(ok.all()), (case, M, K, N, int8, geglu, f32_out,
                            float(err.max()), float((~ok).float().mean()))
    # the row statistics are summed in another order than the norm kernel's:
    # a rare 1-ulp flip of a normalised value, nothing systematic
    assert float((err > 0).float().mean()) < 0.2, (case, M, K, N)


def test_cross_attention_random_shapes(ops):
  """t5d_cross_attention_step (bfloat16) over 40 random shapes — batch 1..48,
  1 / 2 / 4 / 8 beams, 1..16 heads, encoder length a multiple of 32 up to
  1024 with ragged valid lengths (1 included), small and large enough for
  the kernel's streaming-load variant — against float32 softmax attention of
  the same operands on the device."""
  rs = np.random.RandomState(99)
  bf = torch.bfloat16
  for case in range(40):
    B = int(rs.randint(1, 49))
    beams = int(rs.choice([1, 2, 4, 8]))
    H = int(rs.randint(1, 17))
    E = 32 * int(rs.randint(1, 33))
    if case % 8 == 0:   # 48 MB of keys and values and more per launch
      B, H, E = 48, 16, 32 * int(rs.randint(8, 33))
    lens = rs.randint(1, E + 1, size=(B,)).astype(np.int32)
    lens[rs.randint(0, B)] = E
    lens[rs.randint(0, B)] = 1
    gen = torch.Generator(device='cuda')
    gen.manual_seed(case)
    k = (0.5 * torch.randn((B, H, E, 64), generator=gen, device='cuda')).to(bf)
    v = torch.randn((B, H, 64, E), generator=gen, device='cuda').to(bf)
    R = B * beams
    q = (0.125 * torch.randn((R, H * 64), generator=gen, device='cuda')).to(bf)
    lens_d = dev(lens)
    out = ops.cross_attention_step(q, ops.tile_cross_key(k),
                                   ops.tile_cross_value(v), lens_d, beams)
    qf = q.float().view(B, beams, H, 64)
    s = torch.einsum('bkhd,bhed->bkhe', qf, k.float())
    s = s.to(bf).float()   # the reference rounds the scores to the activation type
    valid = torch.arange(E, device='cuda')[None, :] < lens_d[:, None]
    s = s.masked_fill(~valid[:, None, None, :], -1e10)
    p = torch.softmax(s, dim=-1).to(bf).float()
    want = torch.einsum('bkhe,bhde->bkhd', p, v.float()).reshape(R, H * 64)
    err = (out.float() - want).abs()
    assert float(err.max()) <= 2e-2 + 2.0**-6 * float(want.abs().max()), (
        case, B, beams, H, E, float(err.max()))
