"""Every benchmark configuration at its OWN shape against the CPU oracle, so
that the kernel variants the shapes select (workgroup tiles of the dense
kernels, wavefront counts of the attention kernels, fused or separate norms)
are the ones compared:

  cfg 1  T5.1.1-small, float32, greedy, B=8, E=64, L=32: whole predict_batch,
         tokens bit-exact, scores 1e-4.
  cfg 2  T5.1.1-base, bfloat16, 4 beams, B=32, ragged E=512, L=128, all 12
         decoder layers: the first beam-search steps in lock-step with the
         oracle (logits within the bfloat16 tolerance; top-2K indices, surviving
         beams and sequences bit-exact GIVEN the oracle's logits), then the HIP
         loop on its own with a near-tie report at every divergence.
  cfg 3  T5.1.1-large rows of the sampling workload (R=64, E=512, L=256): all
         24 layers over the first sampling steps in lock-step with the oracle
         and a two-layer step in mid-decode; the top-k-40 / temperature-0.7
         token choice on the oracle's logits with supplied Gumbel noise,
         bit-exact.
  cfg 4  T5.1.1-XL, int8 weights, R=16x4, E=512, L=128: all 24 layers through
         the cfg 2 recipe, and a two-layer step in mid-decode.
  cfg 5  T5.1.1-XXL, R=128, E=1024, L=256: every dense layer shape at 128
         rows, one decoder layer + logits at the full batch, four layers at
         128 rows (the 24-layer model as a whole: tests/test_gpu_model.py,
         graph-replay loop against kernel-per-call loop).

bfloat16 logits of stacks of one or two layers are held to 2e-2 for 99.9 % of
the logits (tests/test_gpu_model.py explains the remainder).  Deeper stacks
amplify single-ulp differences until any two bfloat16 evaluations that are
not bit-identical differ by more than that; there the yardstick is the oracle
run with float32 activations on the same (bfloat16-valued) parameters: the
HIP path must be no further from that truth than the bfloat16 oracle itself
(factor 1.25 on mean, 99.9th percentile and maximum).  Measured at the
T5.1.1-base shape, 12 layers: |oracle - truth| mean 1.43e-2, p99.9 5.98e-2,
max 9.8e-2; |hip - truth| 1.43e-2, 6.01e-2, 9.8e-2.
"""

import functools

import numpy as np
import pytest
import torch

from oracle import binary_search as obs
from oracle import decoding as odec
from oracle import models as omodels
from oracle import t5 as ot5
from tests.test_gpu_model import (check_logits, host, quantized_tree,
                                  step_at_width)

pytestmark = pytest.mark.gpu


def report(name, got, want):
  err = np.abs(got - want)
  print(f'{name}: max |dlogit| = {err.max():.3g}, mean {err.mean():.3g}, '
        f'p99.9 {np.quantile(err, 0.999):.3g}', flush=True)


# ---- cfg 1 ------------------------------------------------------------------------


def test_cfg1_small_float32_greedy_end_to_end():
  from t5x_amd import decoding, models, network
  print('cfg1: small float32 greedy B=8 E=64 L=32', flush=True)
  ocfg = ot5.T5Config(dtype='float32', **network.T5_1_1['small'])
  cfg = network.t5_1_1_config('small', dtype='float32')
  assert (cfg.num_heads * cfg.head_dim, cfg.emb_dim) == (384, 512)
  params = ot5.init_params(ocfg, seed=0)
  rs = np.random.Generator(np.random.PCG64(1))
  batch = {'encoder_input_tokens': rs.integers(2, 32128, size=(8, 64)).astype(
      np.int32), 'decoder_input_tokens': np.zeros((8, 32), np.int32)}
  om = omodels.EncoderDecoderModel(
      omodels.Transformer(ocfg),
      decode_fn=functools.partial(odec.temperature_sample, temperature=0.0))
  gm = models.EncoderDecoderModel(
      network.Transformer(cfg),
      decode_fn=functools.partial(decoding.temperature_sample,
                                  temperature=0.0))
  want, waux = om.predict_batch_with_aux(params, batch)
  got, gaux = gm.predict_batch_with_aux(params, batch)
  np.testing.assert_array_equal(host(got), want)
  np.testing.assert_allclose(host(gaux['scores']), waux['scores'], atol=1e-4)
  assert want.shape == (8, 32) and (want != 0).all(axis=1).sum() > 0


# ---- cfg 2 ------------------------------------------------------------------------

CFG2_STEPS = 8


def bf16_rounded(node):
  if isinstance(node, dict):
    return {k: bf16_rounded(v) for k, v in node.items()}
  return ot5.bf16_round(node)


def triangulate(where, got, want, truth, slack=1.25):
  """|hip - truth| against |oracle - truth| (truth: the oracle with float32
  activations on the same parameters): mean, 99.9th percentile and maximum of
  the HIP path's distance must not exceed the bfloat16 oracle's own by more
  than `slack`."""
  stats = lambda e: (e.mean(), np.quantile(e, 0.999), e.max())
  h, o = stats(np.abs(got - truth)), stats(np.abs(want - truth))
  d = np.abs(got - want)
  print(f'{where}: |hip - truth| mean {h[0]:.3g} p99.9 {h[1]:.3g} max '
        f'{h[2]:.3g}; |oracle - truth| mean {o[0]:.3g} p99.9 {o[1]:.3g} max '
        f'{o[2]:.3g}; |hip - oracle| mean {d.mean():.3g} max {d.max():.3g}',
        flush=True)
  for name, x, y in zip(('mean', 'p99.9', 'max'), h, o):
    assert x <= slack * y, (where, name, x, y)
  return h, o


def beam_search_at_full_depth(name, size, weight_dtype, B, K, E, Emin, L, N):
  """The first N beam-search steps of a benchmark configuration at its full
  depth and shape, three ways: (1) in lock-step with the oracle (all sides see
  the oracle's tokens and beam choices; logits held to the float32-activation
  yardstick at every step), (2) the selection kernels GIVEN the oracle's
  logits, bit-exact, (3) the graph-replay loop on its own logits, with a
  near-tie report wherever a beam parts from the oracle's."""
  from t5x_amd import decoding, models, network
  print(f'{name}: {size} bfloat16 ({weight_dtype or "bf16"} weights) beam {K}, '
        f'B={B} E={E} L={L}, full depth, first {N} steps', flush=True)
  kw = dict(network.T5_1_1[size], num_encoder_layers=0)
  ocfg = ot5.T5Config(dtype='bfloat16', **kw)
  tcfg = ot5.T5Config(dtype='float32', **kw)
  cfg = network.T5Config(dtype='bfloat16', weight_dtype=weight_dtype, **kw)
  # bfloat16-valued parameters: every side multiplies by the same numbers
  # (int8: every side quantises those the same way)
  hip_params = bf16_rounded(ot5.init_params(ocfg, seed=0, with_encoder=False))
  params = (quantized_tree(hip_params) if weight_dtype == 'int8'
            else hip_params)
  rs = np.random.Generator(np.random.PCG64(1))
  enc_tok = rs.integers(2, 32128, size=(B, E)).astype(np.int32)
  lens = rs.integers(Emin, E + 1, size=(B,))
  lens[0], lens[1] = E, Emin
  enc_tok[np.arange(E)[None, :] >= lens[:, None]] = 0
  encoded = ot5.bf16_round(rs.standard_normal((B, E, cfg.emb_dim),
                                              dtype=np.float32))
  expand = lambda kv: [(np.repeat(k, K, 0), np.repeat(v, K, 0)) for k, v in kv]
  cross_kv = expand(ot5.project_cross_kv(params, ocfg, encoded))
  truth_kv = expand(ot5.project_cross_kv(params, tcfg, encoded))
  enc_rows = np.repeat(enc_tok, K, axis=0)
  inputs = np.zeros((B, L), np.int32)

  # (1) lock-step: all three sides see the oracle's token history and the
  # oracle's beam choices; logits compared every step.
  module = network.Transformer(cfg)
  enc_dev = torch.as_tensor(encoded, device='cuda').to(torch.bfloat16)
  gcache = decoding.cache_map(
      lambda x: decoding.flat_batch_beam_expand(x, K), module.init_cache(B, L))
  tcache = ot5.init_cache(tcfg, B * K, L)
  trace, scatter = [], []   # scatter: mean |hip - oracle| logit per step

  def tokens_to_logits(state):
    nonlocal gcache, tcache
    if trace:
      alive = trace[-1]['top_alive_indices']
      idx = torch.as_tensor(alive.astype(np.int32), device='cuda')
      gcache = decoding.cache_map(
          lambda x: decoding.unflatten_beam_dim(x, B, K), gcache)
      gcache = decoding.cache_gather_beams(gcache, idx, B, K, K)
      gcache = decoding.cache_map(decoding.flatten_beam_dim, gcache)
      tcache = odec.cache_map(
          lambda x: odec.unflatten_beam_dim(x, B, K), tcache)
      tcache = odec.cache_gather_beams(tcache, alive, B, K, K)
      tcache = odec.cache_map(odec.flatten_beam_dim, tcache)
    tok = state.cur_token
    want, new_cache = ot5.decode(params, ocfg, None, enc_rows, tok, tok,
                                 decode=True, cache=state.cache,
                                 max_decode_length=L, cross_kv=cross_kv)
    truth, tcache = ot5.decode(params, tcfg, None, enc_rows, tok, tok,
                               decode=True, cache=tcache, max_decode_length=L,
                               cross_kv=truth_kv)
    got, new_vars = module.apply(
        {'params': hip_params, 'cache': gcache},
        network.BeamShared(enc_dev, K), network.BeamShared(enc_tok, K),
        torch.as_tensor(tok.astype(np.int32), device='cuda'), None,
        decode=True, max_decode_length=L, mutable=['cache'],
        method=module.decode)
    gcache = new_vars['cache']
    got = host(got)[:, 0]
    triangulate(f'{name} step {len(trace)}', got, want[:, 0], truth[:, 0])
    scatter.append(float(np.abs(got - want[:, 0]).mean()))
    assert scatter[-1] < 3e-2
    return want[:, 0], new_cache

  oseqs, oscores = odec.beam_search(
      inputs, ot5.init_cache(ocfg, B, L), tokens_to_logits, 1, num_decodes=K,
      alpha=0.6, max_decode_step=N, trace=trace)
  assert len(trace) == N
  del truth_kv, tcache

  # (2) the selection kernels GIVEN the oracle's logits: top-2K indices,
  # surviving beams, sequences and flags bit-exact at every step.
  step = [0]

  def oracle_logits(state):
    out = torch.as_tensor(trace[step[0]]['flat_logits'], device='cuda')
    step[0] += 1
    return out, state.cache

  loop = decoding.BeamLoop(inputs, {}, oracle_logits, 1, num_decodes=K,
                           alpha=0.6, max_decode_step=N)
  for s in range(N):
    assert loop.cond()
    loop.body()
    tr = trace[s]
    np.testing.assert_array_equal(host(loop.topk_bufs[1]), tr['topk_indices'])
    np.testing.assert_allclose(host(loop.topk_bufs[0]), tr['topk_log_probs'],
                               atol=2e-5, rtol=0)
    np.testing.assert_array_equal(host(loop.top_alive),
                                  tr['top_alive_indices'])
    np.testing.assert_array_equal(host(loop.cur.live_seqs), tr['live_seqs'])
    np.testing.assert_array_equal(host(loop.cur.finished_seqs),
                                  tr['finished_seqs'])
    np.testing.assert_array_equal(host(loop.cur.finished_flags).astype(bool),
                                  tr['finished_flags'])
    np.testing.assert_allclose(host(loop.cur.live_logprobs),
                               tr['live_logprobs'], atol=2e-5, rtol=0)
  assert not loop.cond()
  seqs, scores = loop.finish()
  np.testing.assert_array_equal(host(seqs), oseqs)
  np.testing.assert_allclose(host(scores), oscores, atol=2e-5, rtol=0)

  # (3) the HIP loop on its own logits (whole iterations replayed as a graph).
  # A beam may part from the oracle's where the oracle's own candidates are a
  # near-tie; at the first step an item differs, the smallest gap between
  # neighbours of the oracle's top 2K must be within what the logit tolerance
  # can move (2e-2 on either score, plus the prefix scores' own drift).
  model = models.EncoderDecoderModel(module, decode_fn=decoding.beam_search)
  fn = models.StepFunction(model, hip_params, network.BeamShared(enc_dev, K),
                           network.BeamShared(enc_tok, K), L)
  fused = decoding.BeamLoop(inputs, module.init_cache(B, L), fn, 1,
                            num_decodes=K, alpha=0.6, max_decode_step=N)
  assert fused.fused is not None
  same = np.ones((B,), bool)
  first = {}
  for s in range(N):
    assert fused.cond()
    fused.body()
    fused.fused.synchronize()
    live = host(fused.cur.live_seqs)
    for b in np.nonzero(same)[0]:
      if not np.array_equal(live[b], trace[s]['live_seqs'][b]):
        same[b] = False
        gaps = -np.diff(trace[s]['topk_log_probs'][b])
        first[int(b)] = (s, float(gaps.min()))
  print(f'{name} end to end: {int(same.sum())} of {B} items keep the oracle\'s '
        f'beams through {N} steps; first divergences (item: step, smallest '
        f'gap in the oracle\'s top {2 * K}): {first}', flush=True)
  for b, (s, gap) in first.items():
    assert gap < 4e-2 + 2e-2 * s, (b, s, gap)
  # Where nothing parted, the scores (sums of N log-probabilities) agree to
  # the tolerance accumulated over the steps: per step the logit tolerance, or
  # twice the mean distance between the two bfloat16 evaluations measured in
  # lock-step above where depth has taken that beyond it (24 layers: 1.7e-2).
  got_lp = host(fused.cur.live_logprobs)
  if same.any():
    np.testing.assert_allclose(got_lp[same], trace[-1]['live_logprobs'][same],
                               atol=N * max(2e-2, 2 * max(scatter)))
  # (With random-init weights the best candidates of a step lie 1e-3 .. 1e-2
  # apart, closer than two bfloat16 evaluations of a 12-layer stack agree, so
  # most items part from the oracle's beams within a few steps, each at such
  # a near-tie; the count is reported, not asserted.)


def test_cfg2_base_beam4_first_steps_at_full_depth():
  """At 12 layers two bfloat16 evaluations of the same weights that are not
  bit-identical differ by more than 2e-2 in a few percent of the logits: the
  oracle itself is that far from its own float32-activation run (measured at
  this shape: mean 1.4e-2, 99.9th percentile 6e-2).  The logits are therefore
  held to that yardstick at every step (no further from the float32 truth than
  the oracle is), and everything discrete is compared exactly given equal
  logits."""
  beam_search_at_full_depth('cfg2', 'base', None, B=32, K=4, E=512, Emin=128,
                            L=128, N=CFG2_STEPS)


def test_cfg4_xl_int8_beam4_first_steps_at_full_depth():
  """T5.1.1-XL, all 24 decoder layers, int8 weight-only kernels with
  per-output-channel scales (stand-alone layer norms, int8 tiles widened at
  the matrix instruction, the large-tile vocabulary projection), batch 16 x 4
  beams, encoder 512, 128 positions: the same three-way check."""
  beam_search_at_full_depth('cfg4', 'xl', 'int8', B=16, K=4, E=512, Emin=512,
                            L=128, N=4)


def test_cfg3_large_sampling_first_steps_at_full_depth():
  """T5.1.1-large, all 24 decoder layers, batch 64, encoder 512, 256
  positions, temperature 0.7 with top-k 40 and supplied Gumbel noise: four
  steps in lock-step with the oracle (every side is fed the oracle's sampled
  tokens); logits held to the float32-activation yardstick, and the token
  choice on the oracle's logits bit-exact at every step."""
  from t5x_amd import network, ops
  B, E, L, N = 64, 512, 256, 4
  print(f'cfg3: large bfloat16 sampling, B={B} E={E} L={L}, 24 layers, first '
        f'{N} steps', flush=True)
  kw = dict(network.T5_1_1['large'], num_encoder_layers=0)
  ocfg = ot5.T5Config(dtype='bfloat16', **kw)
  tcfg = ot5.T5Config(dtype='float32', **kw)
  cfg = network.T5Config(dtype='bfloat16', **kw)
  params = bf16_rounded(ot5.init_params(ocfg, seed=0, with_encoder=False))
  rs = np.random.Generator(np.random.PCG64(3))
  enc_tok = rs.integers(2, 32128, size=(B, E)).astype(np.int32)
  encoded = ot5.bf16_round(rs.standard_normal((B, E, cfg.emb_dim),
                                              dtype=np.float32))
  cross_kv = ot5.project_cross_kv(params, ocfg, encoded)
  truth_kv = ot5.project_cross_kv(params, tcfg, encoded)
  module = network.Transformer(cfg)
  enc_dev = torch.as_tensor(encoded, device='cuda').to(torch.bfloat16)
  ocache, tcache = ot5.init_cache(ocfg, B, L), ot5.init_cache(tcfg, B, L)
  gcache = module.init_cache(B, L)
  noise = odec.GumbelNoise(seed=7)
  temps = np.full((B,), 0.7, np.float32)
  dev = lambda a: torch.as_tensor(a, device='cuda')
  tok = np.zeros((B, 1), np.int32)
  for s in range(N):
    want, ocache = ot5.decode(params, ocfg, None, enc_tok, tok, tok,
                              decode=True, cache=ocache, max_decode_length=L,
                              cross_kv=cross_kv)
    truth, tcache = ot5.decode(params, tcfg, None, enc_tok, tok, tok,
                               decode=True, cache=tcache, max_decode_length=L,
                               cross_kv=truth_kv)
    got, new_vars = module.apply(
        {'params': params, 'cache': gcache}, network.BeamShared(enc_dev, 1),
        network.BeamShared(enc_tok, 1), dev(tok), None, decode=True,
        max_decode_length=L, mutable=['cache'], method=module.decode)
    gcache = new_vars['cache']
    got, want = host(got)[:, 0], want[:, 0]
    triangulate(f'cfg3 step {s}', got, want, truth[:, 0])
    g = noise.noise(s, want.shape)
    hip_tok, hip_lp = ops.sample_tokens(dev(want), dev(g), dev(temps), 40, 0.0,
                                        True)
    scaled = (want / np.float32(0.7)).astype(np.float32)
    masked = obs.topk_mask(scaled, 40, np.float32(-1e7))
    want_tok = np.argmax(masked + g, axis=-1)
    np.testing.assert_array_equal(host(hip_tok), want_tok)
    np.testing.assert_allclose(
        host(hip_lp), odec.log_softmax(masked)[np.arange(B), want_tok],
        atol=1e-5, rtol=1e-5)
    tok = want_tok.astype(np.int32)[:, None]


# ---- cfg 3 / cfg 4 / cfg 5: one step at the full shape -------------------------------


def test_cfg3_large_sampling_rows_at_full_shape():
  from t5x_amd import ops
  print('cfg3: large bfloat16 R=64 E=512 L=256, 2 layers, t=141', flush=True)
  got, want = step_at_width(1024, 16, 2816, B=64, K=1, E=512, Emin=512, L=256,
                            t=141)
  report('cfg3 step', got, want)
  check_logits(got, want, 'bfloat16', 'cfg3')
  # temperature 0.7, top-k 40, supplied Gumbel noise: the token choice on the
  # oracle's logits is bit-exact.
  R, V = want.shape
  g = odec.GumbelNoise(seed=7).noise(141, (R, V))
  temps = np.full((R,), 0.7, np.float32)
  dev = lambda a: torch.as_tensor(a, device='cuda')
  tok, lp = ops.sample_tokens(dev(want), dev(g), dev(temps), 40, 0.0, True)
  scaled = (want / np.float32(0.7)).astype(np.float32)
  masked = obs.topk_mask(scaled, 40, np.float32(-1e7))
  want_tok = np.argmax(masked + g, axis=-1)
  np.testing.assert_array_equal(host(tok), want_tok)
  np.testing.assert_allclose(
      host(lp), odec.log_softmax(masked)[np.arange(R), want_tok], atol=1e-5,
      rtol=1e-5)


def test_cfg4_xl_int8_beam_rows_at_full_shape():
  print('cfg4: XL int8 weights R=16x4 E=512 L=128, 2 layers, t=50', flush=True)
  got, want = step_at_width(2048, 32, 5120, B=16, K=4, E=512, Emin=512, L=128,
                            t=50, weight_dtype='int8')
  report('cfg4 step', got, want)
  check_logits(got, want, 'bfloat16', 'cfg4')


def test_cfg5_xxl_greedy_rows_at_full_shape():
  print('cfg5: XXL bfloat16 R=128 E=1024 L=256, 1 layer, t=200', flush=True)
  got, want = step_at_width(4096, 64, 10240, B=128, K=1, E=1024, Emin=1024,
                            L=256, t=200, layers=1)
  report('cfg5 step', got, want)
  check_logits(got, want, 'bfloat16', 'cfg5')
  # greedy: the argmax of the oracle's logits, through the sampling kernel
  from t5x_amd import ops
  R = want.shape[0]
  dev = lambda a: torch.as_tensor(a, device='cuda')
  tok, _ = ops.sample_tokens(dev(want), None, dev(np.zeros((R,), np.float32)),
                             0, 0.0, True)
  np.testing.assert_array_equal(host(tok), np.argmax(want, axis=-1))


def test_cfg5_xxl_four_layers_at_128_rows():
  """Four XXL decoder layers + logits at the benchmark's 128 rows (stand-alone
  layer norms, large-tile dense kernels on four layers' buffers in a row,
  two-chunk self-attention at position 200); the encoder side is cut to 128
  positions to bound the oracle's cross K/V projections (the full 1024 are
  covered by the one-layer case above).  Four layers of this width scatter two
  bfloat16 evaluations beyond 2e-2 in a few percent of the logits (measured:
  mean 7e-3, 99.9th percentile 3e-2), so the yardstick is the
  float32-activation oracle, as for the other configurations at depth."""
  print('cfg5: XXL bfloat16 R=128 E=128 L=256, 4 layers, t=200', flush=True)
  got, want, truth = step_at_width(4096, 64, 10240, B=128, K=1, E=128,
                                   Emin=100, L=256, t=200, layers=4,
                                   round_weights=True, truth=True)
  report('cfg5 four layers', got, want)
  triangulate('cfg5 four layers', got, want, truth)


@pytest.mark.parametrize('K,N,epi', [(4096, 12288, 'none'),
                                     (4096, 4096, 'residual'),
                                     (4096, 20480, 'geglu'),
                                     (10240, 4096, 'residual'),
                                     (4096, 32128, 'logits')])
@pytest.mark.parametrize('wdt', ['bfloat16', 'int8'])
def test_cfg5_dense_layers_at_128_rows(K, N, epi, wdt):
  """The XXL dense layers at the benchmark's 128 rows: qkv, attention output,
  gated MLP input (N = 2 x 10240 packed columns), MLP output, vocabulary."""
  from t5x_amd import ops
  print(f'cfg5 dense: M=128 K={K} N={N} {epi} {wdt}', flush=True)
  rs = np.random.RandomState(K + N)
  M = 128
  dev = lambda a, dt=None: torch.as_tensor(a, device='cuda').to(
      dt or torch.float32)
  a = ot5.bf16_round(rs.randn(M, K).astype(np.float32))
  cols = N // 2 if epi == 'geglu' else N
  w0 = (rs.randn(K, cols) / np.sqrt(K)).astype(np.float32)
  w1 = (rs.randn(K, cols) / np.sqrt(K)).astype(np.float32)
  wt = torch.bfloat16 if wdt == 'bfloat16' else torch.int8
  kern = (lambda w: w) if wdt == 'bfloat16' else ot5.quantize_int8
  if epi == 'geglu':
    pw = ops.pack_weight(dev(w0), torch.bfloat16, wt, gate_kernel=dev(w1))
    out = ops.gemm(dev(a, torch.bfloat16), pw)
    h0 = ot5.dense_general(a, kern(w0), 'bfloat16')
    h1 = ot5.dense_general(a, kern(w1), 'bfloat16')
    want = ot5.bf16_round(ot5.bf16_round(ot5.gelu(h0)) * h1)
  else:
    pw = ops.pack_weight(dev(w0), torch.bfloat16, wt)
    res = (ot5.bf16_round(rs.randn(M, N).astype(np.float32))
           if epi == 'residual' else None)
    out = ops.gemm(dev(a, torch.bfloat16), pw,
                   residual=None if res is None else dev(res, torch.bfloat16),
                   out_dtype=torch.float32 if epi == 'logits' else None)
    want = ot5.dense_general(a, kern(w0), 'bfloat16',
                             'float32' if epi == 'logits' else None)
    if res is not None:
      want = ot5.bf16_round(want + res)
  got = host(out)
  err = np.abs(got - want)
  # one bfloat16 ulp at |x| < 4 is 1.6e-2 (an output rounded the other way);
  # float32 logits are held to 1e-3
  tol = 1e-3 if epi == 'logits' else 2e-2
  assert err.max() <= tol * max(1.0, np.abs(want).max() / 4), err.max()
  assert (err > 0).mean() < 0.02 or epi == 'logits', (err > 0).mean()


# ---- bfloat16: no further from the truth than the oracle -----------------------------


@pytest.mark.parametrize('layers', [1, 2, 6, 12])
def test_bfloat16_error_is_bounded_by_the_oracles_own(layers):
  """Triangulation at the T5.1.1-base / beam-4 shape (R=128, ragged E=512,
  L=128, t=77).  `truth` is the oracle with float32 activations; the bfloat16
  oracle and the HIP path run on the same (bfloat16-rounded) parameters.  Both
  bfloat16 results scatter around the truth by rounding noise that the model
  amplifies with depth; the HIP path's distance from the truth must not exceed
  the oracle's own by more than a quarter in mean, 99.9th percentile and
  maximum.  Depths 1, 2, 6, 12 stand for the per-layer outputs (each through
  the final norm and the logits layer)."""
  print(f'triangulation: base shape, {layers} layers', flush=True)
  got, want, truth = step_at_width(768, 12, 2048, B=32, K=4, E=512, Emin=128,
                                   L=128, t=77, layers=layers,
                                   round_weights=True, truth=True)
  triangulate(f'{layers} layers', got, want, truth)
