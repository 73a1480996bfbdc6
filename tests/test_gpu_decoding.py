"""The HIP-backed decode loops (t5x_amd.decoding) against the reference's own
known answers (tests/golden/decoding_cases.py, literal vectors of
t5x/decoding_test.py) and, on randomised inputs, against the CPU oracle.
Token ids, beam indices and sequences are compared exactly.
"""

import functools

import numpy as np
import pytest
import torch

from oracle import decoding as odec
from tests.golden import decoding_cases as gc

pytestmark = pytest.mark.gpu
EOS_ID = 1


@pytest.fixture(scope='module')
def decoding():
  from t5x_amd import decoding as d
  return d


def host(t):
  if isinstance(t, torch.Tensor):
    t = t.detach()
    return (t.float() if t.dtype == torch.bfloat16 else t).cpu().numpy()
  return np.asarray(t)


def const_logits(logits, calls=None):
  def fn(state):
    if calls is not None:
      calls.append(state)
    return np.array(logits, dtype=np.float32), state.cache
  return fn


@pytest.mark.parametrize('name', sorted(gc.SAMPLE_CASES))
def test_single_trial_known_answers(decoding, name):
  case = gc.SAMPLE_CASES[name]
  seqs, log_prob = decoding._temperature_sample_single_trial(
      np.array(case['inputs'], np.int32), {}, const_logits(case['logits']),
      EOS_ID, 0, **case['kwargs'])
  np.testing.assert_array_equal(case['expected'], host(seqs))
  if 'scores' in case:
    np.testing.assert_array_almost_equal(case['scores'], host(log_prob))


@pytest.mark.parametrize('name', sorted(gc.OUTER_SAMPLE_CASES))
def test_temperature_sample_known_answers(decoding, name):
  case = gc.OUTER_SAMPLE_CASES[name]
  calls = []
  decodes, scores = decoding.temperature_sample(
      np.array(case['inputs'], np.int32), {},
      const_logits(case['logits'], calls), EOS_ID, 0, **case['kwargs'])
  np.testing.assert_array_equal(np.array(case['expected'])[:, None, :],
                                host(decodes))
  if case['scores'] is not None:
    np.testing.assert_array_equal(host(scores), case['scores'])
  if case['calls'] is not None:
    assert len(calls) == case['calls']


def test_per_item_temperature(decoding):
  case = gc.PER_ITEM_TEMPERATURE
  decodes, scores = decoding.temperature_sample(
      case['inputs'], {}, const_logits(case['logits']), EOS_ID, 0,
      **case['kwargs'])
  np.testing.assert_array_equal(host(decodes), case['expected'])
  np.testing.assert_array_equal(host(scores), case['scores'])


def test_state_callback(decoding):
  def state_callback_fn(state):
    sequences = host(state.sequences).copy()
    for i, cur in enumerate(host(state.cur_index)):
      if sequences[i, cur] == 3:
        sequences[i, cur + 1] = EOS_ID
    return state.replace(sequences=sequences)

  seqs, _ = decoding._temperature_sample_single_trial(
      np.array([[0, 5, 6, 7, 0], [0, 8, 9, 0, 0]], np.int32), {},
      const_logits(gc.PICK_3_3), EOS_ID, 0, topk=0, temperature=0.0,
      state_callback_fn=state_callback_fn)
  np.testing.assert_array_equal([[5, 6, 7, 3, EOS_ID], [8, 9, 3, EOS_ID, 0]],
                                host(seqs))


def test_logit_callback(decoding):
  def logit_callback_fn(logits, state):
    del state
    logits[0, 2] = 0
    logits[1, 3] = 0
    return logits

  seqs, _ = decoding._temperature_sample_single_trial(
      np.array([[0, 5, 6, 7, 0], [0, 8, 9, 0, 0]], np.int32), {},
      const_logits(np.full((2, 4), -1e7, np.float32)), EOS_ID, 0, topk=0,
      temperature=0.0, logit_callback_fn=logit_callback_fn)
  np.testing.assert_array_equal([[5, 6, 7, 2, 2], [8, 9, 3, 3, 3]], host(seqs))


class ForcedDraws:
  """Noise source that makes argmax(logits + noise) return a chosen token per
  step — the seam decoding_test.py:226-254 gets by patching
  jax.random.categorical."""

  def __init__(self, draws):
    self.draws = draws

  def noise(self, step, shape):
    g = np.zeros(shape, np.float32)
    for r, tok in enumerate(self.draws[step]):
      g[r, tok] = 1e6
    return g


def test_forced_draws_early_stop_and_log_prob(decoding):
  case = gc.FORCED_DRAWS
  logits = np.random.RandomState(0).randn(2, 4).astype(np.float32)
  seqs, log_prob = decoding._temperature_sample_single_trial(
      np.array(case['inputs'], np.int32), {}, const_logits(logits), EOS_ID,
      ForcedDraws(case['draws']), topk=0)
  np.testing.assert_array_equal(case['expected'], host(seqs))
  lp = odec.log_softmax(logits.astype(np.float64))
  want = [sum(lp[r, t] for r, t in terms) for terms in case['logprob_terms']]
  np.testing.assert_allclose(want, host(log_prob), atol=1e-5)


def test_num_decodes_expansion_and_sort(decoding, monkeypatch):
  case = gc.NUM_DECODES
  seen = {}

  def fake_trial(inputs, cache, fn, eos, rng, *args, **kwargs):
    seen['inputs'] = host(inputs)
    seen['initial_index'] = kwargs.get('initial_index')
    return (torch.as_tensor(np.array(case['trial_decodes'], np.int32),
                            device='cuda'),
            torch.as_tensor(np.array(case['trial_log_prob'], np.float32),
                            device='cuda'))

  monkeypatch.setattr(decoding, '_temperature_sample_single_trial', fake_trial)
  for with_index in (False, True):
    kw = {}
    if with_index:
      kw['initial_index'] = np.array(case['initial_index'], np.int32)
    decodes, scores = decoding.temperature_sample(
        np.array(case['inputs'], np.int32), {}, None, EOS_ID, 0,
        num_decodes=3, **kw)
    np.testing.assert_array_equal(seen['inputs'], case['expanded_inputs'])
    if with_index:
      np.testing.assert_array_equal(host(seen['initial_index']),
                                    case['expanded_initial_index'])
    np.testing.assert_array_equal(host(decodes), case['decodes'])
    np.testing.assert_allclose(host(scores), case['scores'])


def test_error_messages(decoding):
  with pytest.raises(ValueError, match='At most one of `topp` or `topk`'):
    decoding.temperature_sample(np.zeros((1, 2), np.int32), {},
                                const_logits(gc.PICK_2_3[:1]), EOS_ID, 0,
                                topk=2, topp=0.5)
  with pytest.raises(ValueError, match='Cannot decode more steps'):
    decoding.temperature_sample(np.zeros((1, 2), np.int32), {},
                                const_logits(gc.PICK_2_3[:1]), EOS_ID, 0,
                                topk=0, max_decode_steps=3)


# ---- helpers ---------------------------------------------------------------


def test_beam_dim_helpers(decoding):
  x = np.array([[0, 5, 1, 0], [0, 8, 6, 9]], dtype=np.int32)
  y = decoding.add_beam_dim(x, beam_size=3)
  assert tuple(y.shape) == (2, 3, 4)
  np.testing.assert_array_equal([[[0, 5, 1, 0]] * 3, [[0, 8, 6, 9]] * 3],
                                host(y))
  np.testing.assert_array_equal(
      [[0, 5, 1, 0], [0, 5, 1, 0], [0, 8, 6, 9], [0, 8, 6, 9]],
      host(decoding.flat_batch_beam_expand(x, beam_size=2)))


@pytest.mark.parametrize('dt,L', [(torch.bfloat16, 16), (torch.float32, 8),
                                  (torch.float32, 5)])
def test_beam_dim_helpers_with_a_leading_layer_axis(decoding, dt, L):
  """offset=1 (caches of scanned layers, [layers, batch, ...]) against the
  oracle's helpers; the gather runs in place on rows of 16-byte multiples and
  out of place otherwise (L=5)."""
  from oracle import decoding as odec
  rs = np.random.RandomState(L)
  layers, B, K, H = 3, 2, 4, 2
  x = rs.randn(layers, B, H, 64, L).astype(np.float32)
  xd = torch.as_tensor(x, device='cuda').to(dt)
  xr = host(xd)
  y = decoding.add_beam_dim(xd, K, offset=1)
  np.testing.assert_array_equal(host(y), odec.add_beam_dim(xr, K, offset=1))
  flat = decoding.flatten_beam_dim(y, offset=1)
  np.testing.assert_array_equal(
      host(flat), odec.flatten_beam_dim(odec.add_beam_dim(xr, K, 1), 1))
  np.testing.assert_array_equal(
      host(decoding.unflatten_beam_dim(flat, B, K, offset=1)), host(y))
  z = rs.randn(layers, B, K, H, 64, L).astype(np.float32)
  zd = torch.as_tensor(z, device='cuda').to(dt)
  zr = host(zd).copy()
  idx = rs.randint(0, K, size=(B, K)).astype(np.int32)
  tree = {'decoder': {'layers': {'cached_key': zd,
                                 'cache_index': torch.zeros((), dtype=torch.int32,
                                                            device='cuda')}}}
  got = decoding.cache_gather_beams(tree, idx, B, K, K, offset=1)
  want = odec.cache_gather_beams(
      {'decoder': {'layers': {'cached_key': zr,
                              'cache_index': np.int32(0)}}}, idx, B, K, K,
      offset=1)
  np.testing.assert_array_equal(
      host(got['decoder']['layers']['cached_key']),
      want['decoder']['layers']['cached_key'])


@pytest.mark.parametrize('batch,k', [(1, 16), (8, 16), (9, 11), (32, 11)])
def test_top_k_two_stage(decoding, batch, k):
  rs = np.random.RandomState(batch * 100 + k)
  seq_len = 2047 * k * batch
  seq = np.arange(seq_len)
  rs.shuffle(seq)
  x = seq.reshape(batch, seq_len // batch).astype(np.float32)
  vals, idx = decoding.top_k_two_stage(x, k)
  wv, wi = odec.top_k(x, k)
  np.testing.assert_array_equal(host(vals), wv)
  np.testing.assert_array_equal(host(idx), wi)


def test_cache_map_exclusions(decoding):
  cache = {
      'layers_0': {'cached_key': torch.ones(3, 6), 'cache_index': torch.ones(3)},
      'layers_1': {'relpos_bias': {'cached_bias': torch.ones(1, 5, 3)},
                   'self_attention': {'cached_key': torch.ones(2, 7),
                                      'cache_index': torch.tensor(1)}},
      'position_embedder': {'position_embedder_index': torch.tensor([-1])},
  }
  for apply_to_index in (False, True):
    out = decoding.cache_map(lambda x: x + 4, cache,
                             apply_to_index=apply_to_index)
    fi, fo = decoding._flatten_dict(cache), decoding._flatten_dict(out)
    assert fi.keys() == fo.keys()
    for path, v in fi.items():
      untouched = path[-1] in ('cached_bias', 'position_embedder_index') or (
          path[-1] == 'cache_index' and not apply_to_index)
      assert torch.equal(fo[path], v if untouched else v + 4)


def test_align_prompts(decoding):
  case = gc.ALIGN
  right = decoding._right_align_prompts(np.array(case['prompts'], np.int32))
  np.testing.assert_array_equal(case['right'], right)
  np.testing.assert_array_equal(case['left'],
                                decoding._left_align_prompts(right))


# ---- beam search -------------------------------------------------------------


def test_beam_search_markov_toy(decoding):
  batch_size, beam_size, decode_length = 2, 2, 7
  edge, logits0 = gc.markov_edge_potentials()

  def tokens_to_logits(state):
    cur_iter = host(state.cache['cur_iter'])
    t = np.maximum(0, cur_iter[:, 0].astype(np.int32) - 1)
    tok = host(state.cur_token)[:, 0]
    logits = np.where(cur_iter == 0, logits0[None, :], edge[t, tok, :])
    return logits, {'cur_iter': cur_iter + 1}

  top_scoring, _ = decoding.beam_search(
      np.zeros([batch_size, decode_length]),
      {'cur_iter': np.zeros((batch_size, 1), np.float32)}, tokens_to_logits,
      eos_id=4, num_decodes=beam_size, alpha=0.0, max_decode_len=decode_length)
  top_scoring = host(top_scoring)
  got = [''.join(gc.MARKOV_STATES[t] for t in top_scoring[0, i, :])
         for i in range(beam_size)]
  assert got == gc.MARKOV_EXPECTED


def _expected_scores(expected, batch_logits, prompts):
  out = []
  for beams, logits, prompt in zip(expected, batch_logits, prompts):
    lp = odec.log_softmax(np.asarray(logits, np.float64))
    out.append([
        sum(0 if (p != 0 or tok == 0) else lp[tok]
            for tok, p in zip(beam, prompt)) for beam in beams])
  return out


@pytest.mark.parametrize('name', sorted(gc.BEAM_CASES))
def test_beam_search_known_answers(decoding, name):
  case = gc.BEAM_CASES[name]
  beam_size = 2
  states = []

  def tokens_to_logits(state):
    states.append(state)
    logits = np.repeat(case['logits'][:, None, :], beam_size, axis=1)
    return logits.reshape(-1, logits.shape[-1]), state.cache

  inputs = np.array(case['inputs'], np.int32)
  cache, rest = {}, 1024
  if case.get('with_cache'):
    cache = {
        'cached_bias': np.ones((1, rest), np.float32),
        'decoder/layers_0/self_attention/cached_key':
            np.ones((inputs.shape[0], rest), np.float32),
        'decoder/layers_0/self_attention/cache_index':
            np.ones((inputs.shape[0],), np.float32),
    }
  seqs, scores = decoding.beam_search(inputs, cache, tokens_to_logits, EOS_ID,
                                      num_decodes=beam_size, **case['kwargs'])
  seqs, scores = host(seqs), host(scores)
  assert np.all(np.diff(scores) >= 0)
  np.testing.assert_array_equal(case['expected'], seqs)
  if 'score_prompt' in case:
    np.testing.assert_allclose(
        _expected_scores(case['expected'], case['logits'],
                         case['score_prompt']), scores, atol=1e-5)
  if 'first_tokens' in case:
    np.testing.assert_array_equal(case['first_tokens'],
                                  host(states[0].cur_token))
    first_cache = states[0].cache
    assert tuple(first_cache['cached_bias'].shape) == (1, rest)
    assert tuple(first_cache[
        'decoder/layers_0/self_attention/cached_key'].shape) == (
            inputs.shape[0] * beam_size, rest)
    assert tuple(first_cache[
        'decoder/layers_0/self_attention/cache_index'].shape) == (
            inputs.shape[0] * beam_size,)


def _table_model(table, eos_bias_step=None):
  """Deterministic toy LM: logits depend on (current token, position)."""
  def fn(state):
    tok = host(state.cur_token)[:, 0]
    pos = host(state.cur_index)
    pos = np.broadcast_to(pos, tok.shape) % table.shape[0]
    return table[pos, tok].astype(np.float32), state.cache
  return fn


@pytest.mark.parametrize('seed,B,K,V,L,alpha', [(0, 3, 2, 11, 9, 0.6),
                                                (1, 4, 4, 37, 12, 0.6),
                                                (2, 2, 3, 16, 8, 0.0),
                                                (3, 5, 4, 300, 10, 1.0)])
def test_beam_search_random_table_matches_oracle(decoding, seed, B, K, V, L,
                                                 alpha):
  """Random toy language model where EOS is likely, so the finished pool, the
  brevity penalty and early termination are all exercised; every per-step
  state of the HIP loop must equal the oracle's bit for bit given the same
  log-probabilities, so sequences are compared exactly and scores tightly."""
  rs = np.random.RandomState(seed)
  table = (2.0 * rs.randn(L + 2, V, V)).astype(np.float32)
  table[:, :, 0] = -1e9  # never emit PAD
  table[:, :, EOS_ID] += 1.0
  inputs = np.zeros((B, L), np.int32)
  if seed % 2:
    inputs[0, 1:3] = [5, 7]  # one forced prefix
  want_seqs, want_scores = odec.beam_search(
      inputs, {}, _table_model(table), EOS_ID, num_decodes=K, alpha=alpha)
  seqs, scores = decoding.beam_search(
      inputs, {}, _table_model(table), EOS_ID, num_decodes=K, alpha=alpha)
  np.testing.assert_array_equal(host(seqs), want_seqs)
  np.testing.assert_allclose(host(scores), want_scores, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize('temperature,topk', [(0.0, 0), (0.7, 5), (1.0, 0)])
def test_temperature_sample_random_table_matches_oracle(decoding, temperature,
                                                        topk):
  rs = np.random.RandomState(5)
  B, V, L, nd = 4, 23, 10, 2
  table = (2.0 * rs.randn(L + 2, V, V)).astype(np.float32)
  table[:, :, 0] = -1e9
  inputs = np.zeros((B, L), np.int32)
  inputs[1, 1:4] = [3, 4, 5]
  noise = odec.GumbelNoise(seed=11)
  kw = dict(num_decodes=nd, temperature=temperature, topk=topk)
  want_seqs, want_lp = odec.temperature_sample(
      inputs, {}, _table_model(table), EOS_ID, noise, **kw)
  seqs, lp = decoding.temperature_sample(
      inputs, {}, _table_model(table), EOS_ID, noise, **kw)
  np.testing.assert_array_equal(host(seqs), want_seqs)
  np.testing.assert_allclose(host(lp), want_lp, rtol=1e-5, atol=1e-5)
