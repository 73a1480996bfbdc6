"""Host loop around predict_batch (t5x/utils.py:1543-1817) against the
reference's own expectation (t5x/utils_test.py:1024-1110: 8 examples, batch 2,
with and without flax_mutables -> indices 0..7 and element-wise results in
dataset order) and the properties the reference code fixes: padding with index
-1 is dropped, shard interleaving is undone, aux dicts are kept un-flattened,
the step signature decides whether rng / flax_mutables are passed."""

import types

import numpy as np
import pytest

from t5x_amd import infer


def _dataset(n):
  col = np.transpose(np.tile(np.arange(n), (2, 1)))  # [n, 2]
  return [(np.int64(i), {'a': col[i], 'b': col[i]}) for i in range(n)]


@pytest.mark.parametrize('use_flax_mutables', [True, False])
def test_get_infer_fn_predict_reference_vector(use_flax_mutables):
  batch_size, weight_const = 2, 7
  mutable_const = 5 if use_flax_mutables else 0

  def predict_batch(params, batch, flax_mutables):
    result = (flax_mutables['mutable_w'] * batch['b']
              if use_flax_mutables else 0)
    return result + params['weight'] * batch['a']

  train_state = types.SimpleNamespace(
      params={'weight': np.full((1,), weight_const)},
      flax_mutables=({'mutable_w': np.full((1,), mutable_const)}
                     if use_flax_mutables else None))
  layout = types.SimpleNamespace(batch_size=2, shard_id=0, num_shards=1,
                                 is_first_host_in_replica_set=True)
  partitioner = types.SimpleNamespace(get_data_layout=lambda bs: layout)
  infer_fn = infer.get_infer_fn(predict_batch, batch_size, None,
                                partitioner=partitioner)
  all_indices, all_inferences = zip(*infer_fn(_dataset(8), train_state))
  np.testing.assert_equal(all_indices, np.arange(8))
  np.testing.assert_equal(
      all_inferences,
      np.transpose(np.tile(np.arange(8) * (weight_const + mutable_const),
                           (2, 1))))


def test_padding_is_added_and_removed():
  seen = []

  def step(params, batch):
    seen.append(batch['a'].shape[0])
    return batch['a'][:, 0] * 10

  out = infer.get_infer_fn(step, 4)(_dataset(6), {'w': 1})
  assert seen == [4, 4]               # 6 examples padded to 8
  assert out == [(i, i * 10) for i in range(6)]


def test_more_than_one_data_shard_is_refused():
  layout = types.SimpleNamespace(shard_id=0, num_shards=2)
  part = types.SimpleNamespace(get_data_layout=lambda bs: layout)
  with pytest.raises(NotImplementedError, match='one GPU'):
    infer.get_infer_fn(lambda p, b: b, 4, None, part)


def test_rng_is_split_per_batch_and_passed_by_signature():
  class Key:
    def __init__(self, path=()):
      self.path = path
    def split(self):
      return Key(self.path + (0,)), Key(self.path + (1,))

  got = []

  def step(params, batch, rng):
    got.append(rng.path)
    return batch['a'][:, 0]

  infer.get_infer_fn(step, 2)(_dataset(6), None, rng=Key())
  # step_rng, rng = split(rng): first child goes to the step, second carries on
  assert got == [(0,), (1, 0), (1, 1, 0)]


def test_rng_none_is_passed_as_none():
  got = []

  def step(params, batch, rng):
    got.append(rng)
    return batch['a'][:, 0]

  infer.get_infer_fn(step, 2)(_dataset(4), None)
  assert got == [None, None]


@pytest.mark.parametrize('keep_numpy', [False, True])
def test_aux_values_stay_a_dict_of_sequences(keep_numpy):
  def step(params, batch):
    a = batch['a'][:, 0]
    return np.stack([a, a + 1], axis=1), {'scores': a * 0.5}

  out, aux = infer.get_infer_fn(step, 3, keep_aux_as_numpy=keep_numpy)(
      _dataset(5), None)
  assert out == [(i, [i, i + 1]) for i in range(5)]
  assert list(aux) == ['scores'] and len(aux['scores']) == 5
  np.testing.assert_allclose(np.asarray(aux['scores']), np.arange(5) * 0.5)
  if keep_numpy:
    assert isinstance(aux["scores"][0], (np.ndarray, np.generic))
  else:
    assert isinstance(aux['scores'][0], float)


def test_structured_inferences_keep_their_structure_per_example():
  def step(params, batch):
    a = batch['a'][:, 0]
    return {'x': a, 'y': (a * 2, a * 3)}

  out = infer.get_infer_fn(step, 2)(_dataset(4), None)
  assert out[3] == (3, {'x': 3, 'y': (6, 9)})


def test_unsized_dataset_raises_like_the_reference():
  with pytest.raises(TypeError, match='dataset length is unknown.'):
    infer.get_infer_fn(lambda p, b: b, 2)(iter(_dataset(4)), None)


def test_cache_room_check_on_host_tensors():
  """decoding._check_cache_room looks only at shapes and cache_index values,
  so it can be exercised without a GPU."""
  import pytest
  import torch
  from t5x_amd import decoding
  mk = lambda L, idx: {'decoder': {'layers_0': {'self_attention': {
      'cached_key': torch.zeros((2, 1, 64, L)),
      'cached_value': torch.zeros((2, 1, 64, L)),
      'cache_index': torch.tensor(idx, dtype=torch.int32)}}}}
  decoding._check_cache_room(mk(16, 0), 16, expect_empty=True)
  decoding._check_cache_room(mk(16, 5), 16, expect_empty=False)
  decoding._check_cache_room({}, 16, expect_empty=True)
  with pytest.raises(ValueError, match='holds 16 positions'):
    decoding._check_cache_room(mk(16, 0), 17, expect_empty=True)
  with pytest.raises(ValueError, match='already holds decode steps'):
    decoding._check_cache_room(mk(16, 5), 16, expect_empty=True)


# ---- several decodes in flight: host protocol (no GPU) ---------------------------


class _FakePrediction:
  """What begin_predict_batch returns, with a scripted number of polls."""
  log = []

  def __init__(self, name, polls_needed, value):
    self.name, self.left, self.value = name, polls_needed, value

  def poll(self, block=False):
    self.log.append((self.name, 'block' if block else 'poll'))
    if block:
      self.left = 0
    else:
      self.left = max(0, self.left - 1)
    return self.left == 0

  def result(self):
    assert self.left == 0
    self.log.append((self.name, 'result'))
    return self.value


class _FakeModel:
  def __init__(self, polls_needed=lambda k: 9 - 2 * k):
    self.begun, self.polls_needed = [], polls_needed

  def predict_batch(self, params, batch, rng=None):
    return batch['a'][:, 0] * params['w']

  def begin_predict_batch(self, params, batch, rng=None, in_flight=False):
    assert in_flight
    self.begun.append(int(batch['a'][0, 0]))
    k = len(self.begun)
    _FakePrediction.log.append((k, 'begin'))
    # by default later batches finish sooner: results must still come back in
    # order
    return _FakePrediction(k, self.polls_needed(k),
                           self.predict_batch(params, batch, rng))


def _max_running(log):
  running = most = 0
  for _, what in log:
    running += {'begin': 1, 'result': -1}.get(what, 0)
    most = max(most, running)
  return most


def test_decodes_in_flight_keep_order_and_bound_the_number_in_flight():
  import functools
  _FakePrediction.log = []
  model = _FakeModel()
  fn = infer.get_infer_fn(functools.partial(model.predict_batch), 2,
                          decodes_in_flight=3)
  out = fn(_dataset(8), {'w': 3})
  assert out == [(i, 3 * i) for i in range(8)]
  assert model.begun == [0, 2, 4, 6]
  log = _FakePrediction.log
  assert sorted(name for name, what in log if what == 'result') == [1, 2, 3, 4]
  # never more than 3 begun and not yet collected; the 4th batch begins only
  # after a result was taken
  assert _max_running(log) == 3
  first_result = min(i for i, (_, what) in enumerate(log) if what == 'result')
  assert all(name != 4 for name, _ in log[:first_result])
  # while one is waited for, the others are looked at (kept fed)
  assert {name for name, what in log[:first_result] if what == 'poll'} == {
      1, 2, 3}


def test_a_slow_batch_does_not_idle_the_places_of_the_others():
  _FakePrediction.log = []
  # the first batch needs far longer than the others
  model = _FakeModel(polls_needed=lambda k: 60 if k == 1 else 2)
  fn = infer.get_infer_fn(model.predict_batch, 1, decodes_in_flight=3)
  out = fn(_dataset(7), {'w': 2})
  assert out == [(i, 2 * i) for i in range(7)]      # still in order
  log = _FakePrediction.log
  assert _max_running(log) == 3
  done = [name for name, what in log if what == 'result']
  # every later batch was begun and collected while the first still ran
  assert done[-1] == 1 and sorted(done[:-1]) == [2, 3, 4, 5, 6, 7]


def test_decodes_in_flight_falls_back_to_the_plain_step():
  model = _FakeModel()
  # 1 in flight, or a step that is no bound method with a begin_ variant
  for fn in (infer.get_infer_fn(model.predict_batch, 2, decodes_in_flight=1),
             infer.get_infer_fn(lambda params, batch, rng=None:
                                model.predict_batch(params, batch), 2,
                                decodes_in_flight=3)):
    assert fn(_dataset(4), {'w': 2}) == [(i, 2 * i) for i in range(4)]
  assert model.begun == []


def test_an_overridden_step_is_called_not_the_inherited_begin_variant():
  """t5x/utils.py:1684-1700 calls `infer_step(params, batch, rng)`: a subclass
  that overrides the step keeps being called through its override, also when
  several decodes in flight are asked for; one that overrides the begin
  variant as well gets the overlap back."""

  class Doubling(_FakeModel):
    def predict_batch(self, params, batch, rng=None):
      return 2 * super().predict_batch(params, batch, rng)

  model = Doubling()
  fn = infer.get_infer_fn(model.predict_batch, 2, decodes_in_flight=3)
  assert fn(_dataset(4), {'w': 3}) == [(i, 6 * i) for i in range(4)]
  assert model.begun == []

  class DoublingBoth(Doubling):
    def begin_predict_batch(self, params, batch, rng=None, in_flight=False):
      return super().begin_predict_batch(params, batch, rng, in_flight)

  _FakePrediction.log = []
  model = DoublingBoth()
  fn = infer.get_infer_fn(model.predict_batch, 2, decodes_in_flight=3)
  assert fn(_dataset(4), {'w': 3}) == [(i, 6 * i) for i in range(4)]
  assert model.begun == [0, 2]


def test_model_subclass_overriding_predict_batch_with_aux_is_honoured():
  """The product's EncoderDecoderModel: `predict_batch` of a subclass that
  overrides only predict_batch_with_aux must reach the override, so the
  inherited begin_predict_batch (which would bypass it) is not used."""
  from t5x_amd import models

  class Post(models.EncoderDecoderModel):
    def predict_batch_with_aux(self, params, batch, rng=None, **kw):
      return batch['a'][:, 0] + params['w'], {'scores': batch['a'][:, 0]}

  model = Post(module=None)
  assert infer._begin_of(model.predict_batch) is None
  assert infer._begin_of(model.predict_batch_with_aux) is None
  base = models.EncoderDecoderModel(module=None)
  assert infer._begin_of(base.predict_batch) is not None
  assert infer._begin_of(base.predict_batch_with_aux) is not None
  fn = infer.get_infer_fn(model.predict_batch, 2)
  assert fn(_dataset(4), {'w': 5}) == [(i, i + 5) for i in range(4)]
  fn = infer.get_infer_fn(model.predict_batch_with_aux, 2)
  out, aux = fn(_dataset(4), {'w': 5})
  assert out == [(i, i + 5) for i in range(4)]
  assert aux == {'scores': [0, 1, 2, 3]}


class _FakeFused:
  """A fused step context: the loop condition turns false after `end`
  iterations; chunks complete one poll after they are asked about."""
  CHUNK_SLOTS = 4

  def __init__(self, end):
    self.end, self.enqueued, self.chunks, self.asked = end, 0, [], set()

  def keep_going(self):
    return self.end > 0

  def launch_chunk(self, n):
    self.enqueued += n
    self.chunks.append(self.enqueued)
    return len(self.chunks) - 1

  def chunk_running(self, ticket, block=False):
    if not block and ticket not in self.asked:
      self.asked.add(ticket)
      return None
    return self.chunks[ticket] < self.end

  def finish(self):
    pass


def test_loop_start_poll_protocol():
  import sys
  from t5x_amd import decoding

  class Loop(decoding._InFlight):
    def __init__(self, end):
      self.fused, self.step = _FakeFused(end), 0

    def cond(self):
      return self.fused.keep_going()

  loop = Loop(end=20)
  with pytest.raises(ValueError):
    loop.poll()
  loop.start(check_every=8)
  assert loop.fused.enqueued == 16          # two chunks ahead
  polls = 0
  while not loop.poll():
    polls += 1
    assert polls < 50
  # the condition turned false inside the third chunk: exactly one chunk was
  # enqueued past it, and none after the end was seen
  assert loop.fused.enqueued == 32 and loop.step == 32
  assert loop.poll()                         # stays ended
  done = Loop(end=0)
  done.start()
  assert done.poll() and done.fused.enqueued == 0
  # run_in_flight: blocks on one loop at a time, ends them all
  loops = [Loop(end=e) for e in (5, 40, 17)]
  decoding.run_in_flight(loops, check_every=8)
  assert all(l.poll() for l in loops)
  assert [l.fused.enqueued >= l.fused.end for l in loops] == [True] * 3
  assert all(l.fused.enqueued <= l.fused.end + 16 for l in loops)


def test_decode_context_bytes_and_in_flight_count_of_a_model():
  from t5x_amd import decoding, models, network
  base = network.Transformer.__new__(network.Transformer)
  base.config, base.dtype = network.t5_1_1_config('base', dtype='bfloat16'), 'bfloat16'
  # caches [12, 2, 128 rows, 12, 64, 128] + cross K/V [12, 2, 32, 12, 64, 512], bf16
  assert base.decode_context_bytes(32, 4, 512, 128) == 2 * 12 * 2 * 12 * 64 * (
      128 * 128 + 32 * 512)
  xxl = network.Transformer.__new__(network.Transformer)
  xxl.config, xxl.dtype = network.t5_1_1_config('xxl', dtype='bfloat16'), 'bfloat16'
  assert 60e9 < xxl.decode_context_bytes(128, 1, 1024, 256) < 70e9

  class Module:
    asked = None

    def batches_in_flight(self, *shape):
      Module.asked = shape
      return 2

  batch = {'encoder_input_tokens': np.zeros((5, 40), np.int32),
           'decoder_input_tokens': np.zeros((5, 16), np.int32)}
  model = models.EncoderDecoderModel(Module(), decode_fn=decoding.beam_search)
  assert model.batches_in_flight(batch, 4) == 2
  assert Module.asked == (5, 4, 40, 16)
  # a decode function that cannot be started without waiting: one at a time
  other = models.EncoderDecoderModel(Module(), decode_fn=lambda **kw: None)
  assert other.batches_in_flight(batch) == 1
  # a module that cannot say: one at a time
  assert models.EncoderDecoderModel(object()).batches_in_flight(batch) == 1
