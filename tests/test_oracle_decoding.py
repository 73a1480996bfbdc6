"""Pins oracle/decoding.py to the reference's own known answers.

Every expected array is a literal held by t5x/decoding_test.py (see
tests/golden/decoding_cases.py for the line ranges); the closed-form checks
(stable sort for top-k, log-softmax sums) cover what those leave open.
"""

import numpy as np
import pytest

from oracle import decoding
from tests.golden import decoding_cases as gc

EOS_ID = 1


def const_logits(logits, counter=None):
  def fn(state):
    if counter is not None:
      counter.append(state)
    return np.array(logits, dtype=np.float32), {}
  return fn


@pytest.mark.parametrize('name', sorted(gc.SAMPLE_CASES))
def test_single_trial_known_answers(name):
  case = gc.SAMPLE_CASES[name]
  seqs, log_prob = decoding._temperature_sample_single_trial(
      np.array(case['inputs'], np.int32), {}, const_logits(case['logits']),
      EOS_ID, 0, **case['kwargs'])
  np.testing.assert_array_equal(case['expected'], seqs)
  if 'scores' in case:
    np.testing.assert_array_almost_equal(case['scores'], log_prob)


@pytest.mark.parametrize('name', sorted(gc.OUTER_SAMPLE_CASES))
def test_temperature_sample_known_answers(name):
  case = gc.OUTER_SAMPLE_CASES[name]
  calls = []
  decodes, scores = decoding.temperature_sample(
      np.array(case['inputs'], np.int32), {},
      const_logits(case['logits'], calls), EOS_ID, 0, **case['kwargs'])
  np.testing.assert_array_equal(np.array(case['expected'])[:, None, :],
                                decodes)
  if case['scores'] is not None:
    np.testing.assert_array_equal(scores, case['scores'])
  if case['calls'] is not None:
    assert len(calls) == case['calls']


def test_per_item_temperature():
  case = gc.PER_ITEM_TEMPERATURE
  decodes, scores = decoding.temperature_sample(
      case['inputs'], {}, const_logits(case['logits']), EOS_ID, 0,
      **case['kwargs'])
  np.testing.assert_array_equal(decodes, case['expected'])
  np.testing.assert_array_equal(scores, case['scores'])


def test_state_callback():
  # decoding_test.py:140-179: callback plants EOS after the first sampled 3.
  def state_callback_fn(state):
    sequences = np.array(state.sequences)
    for i, cur in enumerate(state.cur_index):
      if sequences[i, cur] == 3:
        sequences[i, cur + 1] = EOS_ID
    return state.replace(sequences=sequences)

  seqs, _ = decoding._temperature_sample_single_trial(
      np.array([[0, 5, 6, 7, 0], [0, 8, 9, 0, 0]], np.int32), {},
      const_logits(gc.PICK_3_3), EOS_ID, 0, topk=0, temperature=0.0,
      state_callback_fn=state_callback_fn)
  np.testing.assert_array_equal([[5, 6, 7, 3, EOS_ID], [8, 9, 3, EOS_ID, 0]],
                                seqs)


def test_logit_callback():
  # decoding_test.py:181-212
  def logit_callback_fn(logits, state):
    del state
    logits[0, 2] = 0
    logits[1, 3] = 0
    return logits

  flat = np.full((2, 4), -1e7, np.float32)
  seqs, _ = decoding._temperature_sample_single_trial(
      np.array([[0, 5, 6, 7, 0], [0, 8, 9, 0, 0]], np.int32), {},
      const_logits(flat), EOS_ID, 0, topk=0, temperature=0.0,
      logit_callback_fn=logit_callback_fn)
  np.testing.assert_array_equal([[5, 6, 7, 2, 2], [8, 9, 3, 3, 3]], seqs)


def _forced_categorical(draws):
  def fn(key, logits):
    del logits
    return np.array(draws[key.step])
  return fn


def test_forced_draws_early_stop_and_log_prob():
  # decoding_test.py:214-254 and :301-344
  case = gc.FORCED_DRAWS
  rs = np.random.RandomState(0)
  logits = rs.randn(2, 4).astype(np.float32)
  seqs, log_prob = decoding._temperature_sample_single_trial(
      np.array(case['inputs'], np.int32), {}, const_logits(logits), EOS_ID, 0,
      topk=0, categorical_fn=_forced_categorical(case['draws']))
  np.testing.assert_array_equal(case['expected'], seqs)
  lp = decoding.log_softmax(logits.astype(np.float64))
  want = [sum(lp[r, t] for r, t in terms) for terms in case['logprob_terms']]
  np.testing.assert_allclose(want, log_prob, atol=1e-5)


@pytest.mark.parametrize('with_index', [False, True])
def test_num_decodes_expansion_and_sort(with_index):
  # decoding_test.py:346-449
  case = gc.NUM_DECODES
  seen = {}

  def fake_trial(inputs, cache, fn, eos, rng, *args, **kwargs):
    seen['inputs'] = inputs
    seen['initial_index'] = kwargs.get('initial_index')
    return np.array(case['trial_decodes']), np.array(case['trial_log_prob'])

  def spy_cache_map(fn, cache, apply_to_index=False):
    seen['apply_to_index'] = apply_to_index
    return cache

  kw = {}
  if with_index:
    kw['initial_index'] = np.array(case['initial_index'], np.int32)
  decodes, scores = decoding.temperature_sample(
      np.array(case['inputs'], np.int32), {}, None, EOS_ID, 0, num_decodes=3,
      single_trial_fn=fake_trial, cache_map_fn=spy_cache_map, **kw)
  np.testing.assert_array_equal(seen['inputs'], case['expanded_inputs'])
  if with_index:
    np.testing.assert_array_equal(seen['initial_index'],
                                  case['expanded_initial_index'])
    assert seen['apply_to_index']
  np.testing.assert_array_equal(decodes, case['decodes'])
  np.testing.assert_allclose(scores, case['scores'])


def test_topp_log_probs_seen_by_categorical():
  # decoding_test.py:771-804
  case = gc.TOPP_LOG_PROBS
  seen = []

  def cat(key, logits):
    seen.append(np.array(logits))
    return np.array([0], np.int32)

  calls = []
  decodes, _ = decoding.temperature_sample(
      np.zeros((1, 1), np.int32), {}, const_logits(case['logits'], calls),
      EOS_ID, 0, categorical_fn=cat, **case['kwargs'])
  assert len(calls) == 1
  np.testing.assert_array_equal(decodes, [[[0]]])
  np.testing.assert_array_almost_equal(seen[0], case['seen_logits'])


def test_topp_and_topk_both_set_raises():
  with pytest.raises(ValueError, match='At most one of `topp` or `topk`'):
    decoding.temperature_sample(np.zeros((1, 2), np.int32), {},
                                const_logits(gc.PICK_2_3[:1]), EOS_ID, 0,
                                topk=2, topp=0.5)


def test_max_decode_steps_too_long_raises():
  with pytest.raises(ValueError, match='Cannot decode more steps'):
    decoding.temperature_sample(np.zeros((1, 2), np.int32), {},
                                const_logits(gc.PICK_2_3[:1]), EOS_ID, 0,
                                topk=0, max_decode_steps=3)


# ---- helpers ---------------------------------------------------------------


def test_add_beam_dim_and_expand():
  # decoding_test.py:806-823
  x = np.array([[0, 5, 1, 0], [0, 8, 6, 9]], dtype=np.int32)
  y = decoding.add_beam_dim(x, beam_size=3)
  assert y.shape == (2, 3, 4)
  np.testing.assert_array_equal(
      [[[0, 5, 1, 0]] * 3, [[0, 8, 6, 9]] * 3], y)
  np.testing.assert_array_equal(
      [[0, 5, 1, 0], [0, 5, 1, 0], [0, 8, 6, 9], [0, 8, 6, 9]],
      decoding.flat_batch_beam_expand(x, beam_size=2))


def test_beam_dim_helpers_with_a_leading_layer_axis():
  """offset=1 (caches of scanned layers, [layers, batch, ...],
  t5x/decoding.py:773-870): the beam axis goes after the batch axis, which is
  then axis 1.  Closed form: plain NumPy indexing."""
  rs = np.random.RandomState(0)
  x = rs.randn(2, 3, 5).astype(np.float32)            # [layers, batch, d]
  y = decoding.add_beam_dim(x, 4, offset=1)
  assert y.shape == (2, 3, 4, 5)
  np.testing.assert_array_equal(y, np.broadcast_to(x[:, :, None], y.shape))
  flat = decoding.flatten_beam_dim(y, offset=1)
  assert flat.shape == (2, 12, 5)
  np.testing.assert_array_equal(flat, np.repeat(x, 4, axis=1))
  np.testing.assert_array_equal(
      decoding.unflatten_beam_dim(flat, 3, 4, offset=1), y)
  np.testing.assert_array_equal(
      decoding.flat_batch_beam_expand(x, 4, offset=1), flat)
  z = rs.randn(2, 3, 4, 5).astype(np.float32)
  idx = rs.randint(0, 4, size=(3, 4))
  got = decoding.cache_gather_beams({'k': z, 'cache_index': np.int32(7)}, idx,
                                    3, 4, 4, offset=1)
  np.testing.assert_array_equal(got['k'], z[:, np.arange(3)[:, None], idx])
  assert got['cache_index'] == 7


@pytest.mark.parametrize('batch,k', [(1, 16), (8, 16), (9, 11), (32, 11)])
def test_top_k_two_stage_equals_plain_top_k(batch, k):
  # decoding_test.py:825-843
  rs = np.random.RandomState(batch * 100 + k)
  seq_len = 2047 * k * batch
  seq = np.arange(seq_len)
  rs.shuffle(seq)
  x = seq.reshape(batch, seq_len // batch).astype(np.float32)
  v2, i2 = decoding.top_k_two_stage(x, k)
  v1, i1 = decoding.top_k(x, k)
  np.testing.assert_array_equal(v1, v2)
  np.testing.assert_array_equal(i1, i2)
  # closed form: the k largest values in descending order
  np.testing.assert_array_equal(v1, -np.sort(-x, axis=-1)[:, :k])


def test_top_k_ties_prefer_lower_index():
  x = np.array([[1.0, 3.0, 3.0, 0.0, 3.0, 1.0]], np.float32)
  v, i = decoding.top_k(x, 4)
  np.testing.assert_array_equal(i, [[1, 2, 4, 0]])
  np.testing.assert_array_equal(v, [[3, 3, 3, 1]])


def _cache_fixture(with_excluded):
  c = {
      'layers_0': {'cached_key': np.ones([3, 6]),
                   'cached_values': np.ones([3, 6]),
                   'cache_index': np.ones([3])},
      'layers_1': {
          'self_attention': {'cached_key': np.ones([2, 7]),
                             'cached_values': np.ones([5, 8]),
                             'cache_index': np.array(1)},
          'encoder_decoder_attention': {'cached_key': np.ones([10, 12, 2]),
                                        'cached_values': np.ones([4, 7, 2]),
                                        'cache_index': np.ones([4, 5, 6])}},
  }
  if with_excluded:
    c['layers_1']['relpos_bias'] = {'cached_bias': np.ones([1, 5, 3])}
    c['position_embedder'] = {'position_embedder_index': np.array([-1])}
  return c


@pytest.mark.parametrize('apply_to_index', [False, True])
def test_cache_map(apply_to_index):
  # decoding_test.py:845-961
  cache = _cache_fixture(with_excluded=apply_to_index)
  out = decoding.cache_map(lambda x: x + 4, cache,
                           apply_to_index=apply_to_index)
  flat_in = decoding._flatten_dict(cache)
  flat_out = decoding._flatten_dict(out)
  assert flat_in.keys() == flat_out.keys()
  for path, v in flat_in.items():
    untouched = path[-1] in ('cached_bias', 'position_embedder_index') or (
        path[-1] == 'cache_index' and not apply_to_index)
    np.testing.assert_array_equal(flat_out[path], v if untouched else v + 4)


def test_align_prompts():
  case = gc.ALIGN
  right = decoding._right_align_prompts(np.array(case['prompts'], np.int32))
  np.testing.assert_array_equal(case['right'], right)
  np.testing.assert_array_equal(case['left'],
                                decoding._left_align_prompts(right))


def test_brevity_penalty_closed_form():
  for alpha in (0.0, 0.6, 1.0):
    for length in (1, 7, 128):
      want = ((5.0 + length) / 6.0)**alpha
      np.testing.assert_allclose(decoding.brevity_penalty(alpha, length), want,
                                 rtol=1e-6)
      np.testing.assert_allclose(
          decoding.brevity_penalty(alpha, np.array([length], np.int32)),
          [want], rtol=1e-6)


# ---- beam search -------------------------------------------------------------


def test_beam_search_markov_toy():
  # decoding_test.py:963-1069
  batch_size, beam_size, decode_length = 2, 2, 7
  edge, logits0 = gc.markov_edge_potentials()

  def tokens_to_logits(state):
    cur_iter = state.cache['cur_iter']
    t = np.maximum(0, cur_iter[:, 0].astype(np.int32) - 1)
    tok = state.cur_token[:, 0]
    cur_logits = edge[t, tok, :]
    logits = np.where(cur_iter == 0, logits0[None, :], cur_logits)
    return logits, {'cur_iter': cur_iter + 1}

  top_scoring, _ = decoding.beam_search(
      np.zeros([batch_size, decode_length]),
      {'cur_iter': np.zeros((batch_size, 1))}, tokens_to_logits, eos_id=4,
      num_decodes=beam_size, alpha=0.0, max_decode_len=decode_length)
  got = [''.join(gc.MARKOV_STATES[t] for t in top_scoring[0, i, :])
         for i in range(beam_size)]
  assert got == gc.MARKOV_EXPECTED


def _expected_scores(expected, batch_logits, prompts):
  out = []
  for beams, logits, prompt in zip(expected, batch_logits, prompts):
    lp = decoding.log_softmax(np.asarray(logits, np.float64))
    out.append([
        sum(0 if (p != 0 or tok == 0) else lp[tok]
            for tok, p in zip(beam, prompt)) for beam in beams])
  return out


@pytest.mark.parametrize('name', sorted(gc.BEAM_CASES))
def test_beam_search_known_answers(name):
  case = gc.BEAM_CASES[name]
  beam_size = 2
  states = []

  def tokens_to_logits(state):
    states.append(state)
    logits = np.repeat(case['logits'][:, None, :], beam_size, axis=1)
    return decoding.flatten_beam_dim(logits), state.cache

  inputs = np.array(case['inputs'], np.int32)
  cache = {}
  rest = 1024
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
  assert np.all(np.diff(scores) >= 0)
  np.testing.assert_array_equal(case['expected'], seqs)
  if 'score_prompt' in case:
    np.testing.assert_allclose(
        _expected_scores(case['expected'], case['logits'],
                         case['score_prompt']), scores, atol=1e-5)
  if 'first_tokens' in case:
    np.testing.assert_array_equal(case['first_tokens'], states[0].cur_token)
    first_cache = states[0].cache
    assert first_cache['cached_bias'].shape == (1, rest)
    assert first_cache[
        'decoder/layers_0/self_attention/cached_key'].shape == (
            inputs.shape[0] * beam_size, rest)
    assert first_cache[
        'decoder/layers_0/self_attention/cache_index'].shape == (
            inputs.shape[0] * beam_size,)
