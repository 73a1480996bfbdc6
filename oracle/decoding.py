"""NumPy restatement of t5x/decoding.py (test oracle, not product code).

The device-side `lax.while_loop`s become Python loops; every array is a NumPy
array with the dtype the reference would hold (float32 / int32 / bool).  Each
function cites the reference lines it follows.

Random sampling: the reference draws `random.categorical(rng1, logits)` from a
threefry key stream that is not reproducible without JAX.  Here `decode_rng`
is either an integer seed or a `GumbelNoise` object that hands out a
pre-generated Gumbel tensor per loop step, and categorical sampling is
`argmax(logits + gumbel)` (the definition of jax.random.categorical).  The
`categorical_fn` argument is the same seam the reference's tests use when they
patch `jax.random.categorical`.
"""

import dataclasses
import functools
from typing import Any, Callable, Mapping, Optional, Tuple, Union

import numpy as np

from oracle import binary_search

# t5x/decoding.py:33-39
NEG_INF = np.array(-1.0e7)
NEG_INF_VALUE = -1.0e7
MIN_TEMPERATURE = np.array(1e-4)

_F32 = np.float32
_I32 = np.int32


@dataclasses.dataclass
class DecodingState:
  """t5x/decoding.py:42-66."""
  cur_index: np.ndarray
  sequences: np.ndarray
  cur_token: np.ndarray
  cache: Mapping[str, Any]


@dataclasses.dataclass
class SamplingLoopState:
  """t5x/decoding.py:74-99."""
  step: np.ndarray
  cur_index: np.ndarray
  sequences: np.ndarray
  cache: Mapping[str, Any]
  cur_token: np.ndarray
  ended: np.ndarray
  rng: Any
  log_prob: np.ndarray

  def replace(self, **kw):
    return dataclasses.replace(self, **kw)


# ------------------------------------------------------------------------------
# jax primitives restated
# ------------------------------------------------------------------------------


def log_softmax(x):
  """jax.nn.log_softmax: shifted - log(sum(exp(shifted))), in x's dtype.

  float32 exp/log are evaluated in double and rounded once, i.e. as a
  correctly rounded float32 libm would; NumPy's own SIMD float32 log is a few
  ulp off, which is enough to break the exact score ties that the reference's
  beam-search known answers rely on (decoding_test.py:1071-1132).
  """
  x = np.asarray(x)
  shifted = x - np.max(x, axis=-1, keepdims=True)
  e = np.exp(shifted.astype(np.float64)).astype(x.dtype)
  s = np.sum(e, axis=-1, keepdims=True, dtype=x.dtype)
  lse = np.log(s.astype(np.float64)).astype(x.dtype)
  return (shifted - lse).astype(x.dtype)


def top_k(x, k):
  """lax.top_k: values descending, ties broken toward the lower index."""
  x = np.asarray(x)
  # Stable ascending sort of the negated keys == descending with ties kept in
  # index order.  Negation is exact and order reversing for non-NaN floats.
  idx = np.argsort(-x, axis=-1, kind='stable')[..., :k]
  return np.take_along_axis(x, idx, axis=-1), idx.astype(_I32)


class GumbelNoise:
  """Per-step Gumbel noise shared by the oracle and the HIP path.

  `noise(step, shape)` returns float32 noise for loop step `step`.  Either a
  pre-generated `[steps, rows, vocab]` tensor or a seed from which the step's
  tensor is regenerated (`PCG64(seed + step)`, `-log(-log(U))`).
  """

  def __init__(self, seed: int = 0, tensor: Optional[np.ndarray] = None):
    self.seed = int(seed)
    self.tensor = tensor

  def noise(self, step: int, shape) -> np.ndarray:
    if self.tensor is not None:
      g = np.asarray(self.tensor[step], dtype=_F32)
      assert g.shape == tuple(shape), (g.shape, shape)
      return g
    gen = np.random.Generator(np.random.PCG64(self.seed + int(step)))
    u = gen.uniform(np.finfo(_F32).tiny, 1.0, size=shape)
    return (-np.log(-np.log(u))).astype(_F32)


@dataclasses.dataclass(frozen=True)
class _Key:
  """Stand-in for a PRNG key: (noise source, step, which half of the split)."""
  source: GumbelNoise
  step: int
  leaf: int = 0

  def __eq__(self, other):
    return (isinstance(other, _Key) and self.source is other.source and
            self.step == other.step and self.leaf == other.leaf)


def make_key(decode_rng) -> _Key:
  if isinstance(decode_rng, _Key):
    return decode_rng
  if isinstance(decode_rng, GumbelNoise):
    return _Key(decode_rng, 0, 0)
  if decode_rng is None:
    decode_rng = 0  # t5x/decoding.py:345-346 (PRNGKey(0))
  return _Key(GumbelNoise(int(np.asarray(decode_rng).reshape(-1)[-1])), 0, 0)


def split(key: _Key) -> Tuple[_Key, _Key]:
  """random.split stand-in: (key used for this step's draw, key carried on)."""
  return _Key(key.source, key.step, 1), _Key(key.source, key.step + 1, 0)


def categorical(key: _Key, logits) -> np.ndarray:
  """jax.random.categorical == argmax(logits + gumbel)."""
  g = key.source.noise(key.step, np.shape(logits))
  return np.argmax(np.asarray(logits, dtype=_F32) + g, axis=-1)


# ------------------------------------------------------------------------------
# cache / beam helpers
# ------------------------------------------------------------------------------


def _flatten_dict(d, prefix=()):
  out = {}
  for k, v in d.items():
    if isinstance(v, Mapping) and v:
      out.update(_flatten_dict(v, prefix + (k,)))
    else:
      out[prefix + (k,)] = v
  return out


def _unflatten_dict(flat):
  out = {}
  for path, v in flat.items():
    cur = out
    for k in path[:-1]:
      cur = cur.setdefault(k, {})
    cur[path[-1]] = v
  return out


def cache_map(fn, cache, apply_to_index: bool = False):
  """t5x/decoding.py:739-770."""
  flat_cache = _flatten_dict(cache)
  if apply_to_index:
    keyvals = dict(flat_cache)
  else:
    keyvals = {k: v for k, v in flat_cache.items() if k[-1] != 'cache_index'}
  exclusion_list = ['cached_bias', 'position_embedder_index']
  keyvals = {k: v for k, v in keyvals.items() if k[-1] not in exclusion_list}
  keyvals = {k: fn(v) for k, v in keyvals.items()}
  flat_cache.update(keyvals)
  return _unflatten_dict(flat_cache)


def add_beam_dim(x, beam_size: int, offset: int = 0):
  """t5x/decoding.py:773-780."""
  x = np.expand_dims(np.asarray(x), axis=offset + 1)
  tile_dims = [1] * x.ndim
  tile_dims[offset + 1] = beam_size
  return np.tile(x, tile_dims)


def flatten_beam_dim(x, offset: int = 0):
  """t5x/decoding.py:783-788."""
  x = np.asarray(x)
  xshape = list(x.shape)
  b_sz = xshape.pop(offset)
  xshape[offset] *= b_sz
  return x.reshape(xshape)


def unflatten_beam_dim(x, batch_size: int, beam_size: int, offset: int = 0):
  """t5x/decoding.py:791-798."""
  x = np.asarray(x)
  assert batch_size * beam_size == x.shape[offset]
  xshape = list(x.shape)
  newshape = xshape[:offset] + [batch_size, beam_size] + xshape[offset + 1:]
  return x.reshape(newshape)


def flat_batch_beam_expand(x, beam_size: int, offset: int = 0):
  """t5x/decoding.py:801-805."""
  return flatten_beam_dim(add_beam_dim(x, beam_size, offset), offset)


def _gather_rows(x, beam_indices, axis0: int):
  """x[..., b, beam_indices[b, e], ...]: the one-hot einsum of :835-852,:897-904
  is an exact row pick (one term is 1*x, the rest 0*x; every x is finite)."""
  x = np.asarray(x)
  b = np.arange(beam_indices.shape[0])[:, None]
  if axis0 == 0:
    return x[b, beam_indices]
  return x[:, b, beam_indices]


def cache_gather_beams(nested, beam_indices, batch_size, old_beam_size,
                       new_beam_size, one_hot: bool = True, offset: int = 0):
  """t5x/decoding.py:808-870."""
  del batch_size, old_beam_size, new_beam_size, one_hot
  assert offset in (0, 1), 'general offsets not supported'
  return cache_map(lambda x: _gather_rows(x, beam_indices, offset), nested)


def _tree_map(fn, nested):
  if isinstance(nested, (list, tuple)):
    return type(nested)(_tree_map(fn, x) for x in nested)
  if isinstance(nested, Mapping):
    return {k: _tree_map(fn, v) for k, v in nested.items()}
  return fn(nested)


def gather_beams(nested, beam_indices, batch_size, old_beam_size,
                 new_beam_size, one_hot: bool = True):
  """t5x/decoding.py:873-915."""
  del batch_size, old_beam_size, new_beam_size, one_hot
  return _tree_map(lambda x: _gather_rows(x, beam_indices, 0), nested)


def top_k_two_stage(x, k):
  """t5x/decoding.py:918-966 (kept literally, including the lane reshape)."""
  x = np.asarray(x)
  batch, num_samples = x.shape
  num_lanes = 128
  if batch <= 8 and num_samples > 8 * num_lanes * k:
    if num_samples % num_lanes != 0:
      rounded = num_samples + (num_lanes - num_samples % num_lanes)
      x = np.pad(x, ((0, 0), (0, rounded - num_samples)), mode='constant',
                 constant_values=-np.inf)
      num_samples = rounded
    sublanes = int(num_samples / num_lanes)
    x_reshaped = np.reshape(x, (batch * num_lanes, sublanes))
    vals, indices = top_k(x_reshaped, k)
    indices = np.reshape(indices, (batch, num_lanes, k))
    index_offsets = np.reshape(sublanes * np.arange(num_lanes),
                               (1, num_lanes, 1))
    indices = np.reshape(index_offsets + indices, (batch, num_lanes * k))
    vals = np.reshape(vals, (batch, num_lanes * k))
    vals_s2, indices_s2 = top_k(vals, k)
    indices_s2 = np.take_along_axis(indices, indices_s2, axis=1)
    return vals_s2, indices_s2.astype(_I32)
  return top_k(x, k)


def gather_topk_beams(nested, score_or_log_prob, batch_size, new_beam_size):
  """t5x/decoding.py:969-996."""
  _, topk_indices = top_k(score_or_log_prob, new_beam_size)
  topk_indices = np.flip(topk_indices, axis=1)
  return gather_beams(nested, topk_indices, batch_size,
                      score_or_log_prob.shape[1], new_beam_size)


def brevity_penalty(alpha: float, length):
  """t5x/decoding.py:723-733: ((5 + length) / 6) ** alpha in float32.

  A Python-int `length` keeps the base in double until the power (weak typed
  scalar); an int32 array promotes to float32 before the division.
  """
  if isinstance(length, (int, np.integer)):
    base = _F32((5.0 + float(length)) / 6.0)
  else:
    base = (_F32(5.0) + np.asarray(length).astype(_F32)) / _F32(6.0)
  return np.power(base, _F32(alpha), dtype=_F32)


# ------------------------------------------------------------------------------
# Temperature sampling
# ------------------------------------------------------------------------------


def temperature_sample(
    inputs, cache, tokens_to_logits, eos_id: int, decode_rng=None,
    num_decodes: int = 1, temperature: Union[float, np.ndarray] = 1.0,
    topk: int = 1, topp: float = 0.0, cache_offset: int = 0,
    initial_index: Optional[np.ndarray] = None,
    max_decode_steps: Optional[Union[int, np.ndarray]] = None,
    max_decode_steps_hard_limit: Optional[int] = None,
    rescale_log_probs: bool = True,
    state_callback_fn: Optional[Callable] = None,
    logit_callback_fn: Optional[Callable] = None,
    categorical_fn: Optional[Callable] = None,
    single_trial_fn: Optional[Callable] = None,
    cache_map_fn: Optional[Callable] = None,
):
  """t5x/decoding.py:115-409."""
  decode_rng = make_key(decode_rng)  # :345-346
  inputs = np.asarray(inputs)

  if (max_decode_steps_hard_limit is not None and
      max_decode_steps_hard_limit > 0 and max_decode_steps is not None):
    max_decode_steps = np.minimum(max_decode_steps,
                                  max_decode_steps_hard_limit)  # :348-355

  if num_decodes > 1:  # :357-374
    expanded_inputs = flat_batch_beam_expand(inputs, num_decodes)
    expanded_cache = (cache_map_fn or cache_map)(
        functools.partial(flat_batch_beam_expand, beam_size=num_decodes,
                          offset=cache_offset),
        cache, apply_to_index=initial_index is not None)
    if initial_index is not None:
      initial_index = flat_batch_beam_expand(initial_index, num_decodes)
  else:
    expanded_inputs = inputs
    expanded_cache = cache

  trial = single_trial_fn or _temperature_sample_single_trial
  kw = dict(initial_index=initial_index, max_decode_steps=max_decode_steps,
            rescale_log_probs=rescale_log_probs,
            state_callback_fn=state_callback_fn,
            logit_callback_fn=logit_callback_fn)
  if single_trial_fn is None:
    kw['categorical_fn'] = categorical_fn
  expanded_decodes, expanded_log_prob = trial(
      expanded_inputs, expanded_cache, tokens_to_logits, eos_id, decode_rng,
      num_decodes, temperature, topk, topp, **kw)  # :378-393

  batch_size = inputs.shape[0]
  decodes = unflatten_beam_dim(expanded_decodes, batch_size, num_decodes)
  log_prob = unflatten_beam_dim(expanded_log_prob, batch_size, num_decodes)
  # :401-409 ascending by log prob (jnp.argsort is a stable sort).
  idxs = np.argsort(log_prob, axis=-1, kind='stable')[..., None]
  return (np.take_along_axis(decodes, idxs, axis=1),
          np.take_along_axis(log_prob, idxs[..., 0], axis=-1))


def _temperature_sample_single_trial(
    inputs, cache, tokens_to_logits, eos_id: int, prng_key,
    num_decodes: int = 1, temperature: Union[float, np.ndarray] = 1.0,
    topk: int = 20, topp: Union[float, np.ndarray] = 0.0,
    initial_index: Optional[np.ndarray] = None,
    max_decode_steps: Optional[Union[int, np.ndarray]] = None,
    rescale_log_probs: bool = True,
    state_callback_fn: Optional[Callable] = None,
    logit_callback_fn: Optional[Callable] = None,
    categorical_fn: Optional[Callable] = None,
):
  """t5x/decoding.py:412-715."""
  if topp and topk:  # :433-434
    raise ValueError('At most one of `topp` or `topk` may be non-zero.')
  if categorical_fn is None:
    categorical_fn = categorical
  prng_key = make_key(prng_key)

  inputs = np.asarray(inputs)
  batch_size, max_decode_len = inputs.shape

  if max_decode_steps is not None:  # :438-455
    if np.ndim(max_decode_steps) == 0 and max_decode_steps > inputs.shape[1]:
      raise ValueError('Cannot decode more steps than the sequence length.')
    max_decode_len = np.sum(inputs != 0, axis=1) + max_decode_steps
    max_decode_len = np.minimum(inputs.shape[1], max_decode_len)

  extra_input_tokens = 2  # :465-470
  expanded_prompt_inputs = np.append(
      inputs, np.zeros((batch_size, extra_input_tokens), dtype=inputs.dtype),
      axis=1)
  end_marker = np.array(eos_id)
  temperature = np.asarray(temperature, dtype=_F32)  # :473

  step = np.zeros((), dtype=_I32)
  rng0 = prng_key
  if initial_index is None:  # :480-492
    i0 = np.zeros((batch_size,), dtype=_I32)
    token0 = np.zeros((batch_size, 1), dtype=_I32)
  else:
    i0 = np.asarray(initial_index)
    token0 = np.take_along_axis(expanded_prompt_inputs, i0[:, None], axis=1)
  ended0 = np.zeros((batch_size, 1), dtype=bool)
  sequences0 = expanded_prompt_inputs
  log_prob0 = np.zeros((batch_size,), dtype=_F32)
  state = SamplingLoopState(step, i0, sequences0, cache, token0, ended0, rng0,
                            log_prob0)
  initial_eos_count = np.sum(sequences0 == end_marker, axis=-1,
                             keepdims=True)  # :507

  def sample_nonzero(logits, temp, rng1, row=None):  # :541-573
    scaled_logits = (logits / np.maximum(temp, _F32(MIN_TEMPERATURE))).astype(
        _F32)
    if topk:
      scaled_logits = binary_search.topk_mask(scaled_logits, topk,
                                              _F32(NEG_INF))
    if topp:
      scaled_logits = binary_search.topp_mask(scaled_logits, topp,
                                              _F32(NEG_INF))
    if row is not None and categorical_fn is categorical:
      # vmapped draw (:608-610): row `row` of this step's noise tensor.
      g = rng1.source.noise(rng1.step, (batch_size, logits.shape[-1]))
      next_token = np.argmax(scaled_logits + g[row:row + 1], axis=-1)
    else:
      next_token = categorical_fn(rng1, scaled_logits)
    next_token = np.asarray(next_token).astype(_I32)
    if rescale_log_probs:
      log_probs = log_softmax(scaled_logits)
    else:
      log_probs = log_softmax(logits)
    next_log_prob = np.take_along_axis(log_probs, next_token[:, None],
                                       axis=-1)[:, 0]
    return next_token, next_log_prob

  def sample_zero(logits, temp, rng1, row=None):  # :575-592
    del temp, rng1, row
    next_token = np.argmax(logits, -1).astype(_I32)
    if rescale_log_probs:
      next_log_prob = np.zeros(next_token.shape, dtype=_F32)
    else:
      log_probs = log_softmax(logits)
      next_log_prob = np.take_along_axis(log_probs, next_token[:, None],
                                         axis=-1)[:, 0]
    return next_token, next_log_prob

  while not np.all(state.ended):  # cond :509-515
    if state_callback_fn is not None:  # :520-521
      state = state_callback_fn(state)
    rng1, rng2 = split(state.rng)  # :524
    decoding_state = DecodingState(
        cur_index=state.cur_index,
        sequences=state.sequences[:, :-extra_input_tokens],
        cur_token=state.cur_token, cache=state.cache)
    logits, new_cache = tokens_to_logits(decoding_state)  # :533
    logits = np.array(logits, dtype=_F32)
    if logit_callback_fn is not None:  # :538-539
      logits = logit_callback_fn(logits, state)

    if temperature.ndim == 1:  # :595-612 per-item temperature
      temps = np.repeat(temperature, num_decodes)
      next_token = np.zeros((batch_size,), _I32)
      next_log_prob = np.zeros((batch_size,), _F32)
      for r in range(batch_size):
        fn = sample_nonzero if temps[r] > MIN_TEMPERATURE else sample_zero
        tok, lp = fn(logits[r:r + 1], temps[r], rng1, row=r)
        next_token[r], next_log_prob[r] = tok[0], lp[0]
    else:  # :613-621
      fn = sample_nonzero if temperature > MIN_TEMPERATURE else sample_zero
      next_token, next_log_prob = fn(logits, temperature, rng1)

    i = np.minimum(state.cur_index, max_decode_len)  # :631
    next_input_token = np.take_along_axis(state.sequences, (i + 1)[:, None],
                                          axis=1)[:, 0]  # :636-641
    out_of_prompt = next_input_token == 0  # :644
    next_token = (next_token * out_of_prompt +
                  next_input_token * ~out_of_prompt)  # :648
    next_log_prob = (state.log_prob + (next_log_prob * out_of_prompt) *
                     (~state.ended)[:, 0].astype(_I32)).astype(_F32)  # :652-654
    next_token = next_token[:, None]
    next_token_or_endpad = (next_token * ~state.ended).astype(
        state.sequences.dtype)  # :661
    one_hot = (np.arange(state.sequences.shape[1])[None, :] ==
               (i + 1)[:, None]).astype(state.sequences.dtype)  # :663-665
    new_sequences = (state.sequences * (1 - one_hot) +
                     next_token_or_endpad * one_hot)  # :666-668
    cur_eos_count = np.sum(new_sequences == end_marker, axis=-1,
                           keepdims=True)  # :675
    has_additional_eos = cur_eos_count > initial_eos_count  # :684
    ended = (state.ended | has_additional_eos |
             (i >= max_decode_len - 1)[:, None])  # :685-689
    state = SamplingLoopState(state.step + 1, (i + 1).astype(_I32),
                              new_sequences, new_cache,
                              next_token_or_endpad.astype(_I32), ended, rng2,
                              next_log_prob)

  if state_callback_fn is not None:  # :707-708
    state = state_callback_fn(state)
  return state.sequences[:, 1:-1], state.log_prob  # :715


# ------------------------------------------------------------------------------
# Beam search
# ------------------------------------------------------------------------------


@dataclasses.dataclass
class BeamState:
  """t5x/decoding.py:1002-1021."""
  cur_index: np.ndarray
  live_logprobs: np.ndarray
  finished_scores: np.ndarray
  live_seqs: np.ndarray
  finished_seqs: np.ndarray
  finished_flags: np.ndarray
  cache: Any
  initial_index: Optional[np.ndarray]


def beam_init(batch_size, beam_size, max_decode_len, cache, offset=0,
              live_seqs=None, initial_index=None) -> BeamState:
  """t5x/decoding.py:1024-1066."""
  cur_index0 = np.array(0)
  live_logprobs0 = np.tile(
      np.array([0.0] + [NEG_INF_VALUE] * (beam_size - 1), dtype=_F32),
      [batch_size, 1])
  finished_scores0 = (np.ones((batch_size, beam_size), dtype=_F32) *
                      _F32(NEG_INF_VALUE))
  live_seqs0 = (np.asarray(live_seqs) if live_seqs is not None else np.zeros(
      (batch_size, beam_size, max_decode_len), _I32))
  finished_seqs0 = np.zeros((batch_size, beam_size, max_decode_len), _I32)
  finished_flags0 = np.zeros((batch_size, beam_size), bool)
  beam_cache0 = cache_map(lambda x: add_beam_dim(x, beam_size, offset), cache,
                          apply_to_index=live_seqs is not None)
  return BeamState(cur_index0, live_logprobs0, finished_scores0, live_seqs0,
                   finished_seqs0, finished_flags0, beam_cache0, initial_index)


def _right_align_prompts(prompts):
  """t5x/decoding.py:1069-1095."""
  prompts = np.asarray(prompts)
  max_len = prompts.shape[1]
  nbits = np.ceil(np.log2(max_len)).astype(np.int32)
  indices = np.arange(max_len)
  prompt_max_index = np.argmax((prompts != 0) * indices[None, :], axis=1)
  shifts = max_len - prompt_max_index - 1
  for i in range(0, nbits + 1):
    bitmask = 2**i
    prompts = np.where((shifts & bitmask)[:, None] != 0,
                       np.pad(prompts, ((0, 0), (bitmask, 0)))[:, :-bitmask],
                       prompts)
  return prompts


def _left_align_prompts(prompts):
  """t5x/decoding.py:1098-1120."""
  prompts = np.asarray(prompts)
  max_len = prompts.shape[1]
  indices = np.arange(max_len)
  non_padding_positions = (prompts != 0) * (indices[None, :] + 1)
  m = np.where(non_padding_positions != 0, non_padding_positions, max_len + 1)
  shifts = np.argmin(m, axis=1)
  temp = prompts
  nbits = np.ceil(np.log2(max_len)).astype(np.int32)
  for i in range(0, nbits + 1):
    bitmask = 2**i
    temp = np.where((shifts & bitmask)[:, None] != 0,
                    np.pad(temp, ((0, 0), (0, bitmask)))[:, bitmask:], temp)
  return temp


def _pick_last_prompt_token(prompts):
  """t5x/decoding.py:1123-1127."""
  prompts = np.asarray(prompts)
  prompt_lengths = np.sum(prompts != 0, axis=1)
  return prompts[np.arange(prompts.shape[0]), prompt_lengths]


def beam_search(
    inputs, cache, tokens_to_logits, eos_id: int, num_decodes: int = 4,
    alpha: float = 0.6, max_decode_len: Optional[int] = None,
    max_decode_step: int = -1, min_log_prob: float = NEG_INF_VALUE,
    decode_rng=None, cache_offset: int = 0,
    initial_index: Optional[np.ndarray] = None, trace: Optional[list] = None,
):
  """t5x/decoding.py:1131-1569.  `trace`, when given, receives one dict of
  intermediate selections per loop step (test instrumentation only)."""
  del decode_rng
  inputs = np.asarray(inputs)
  beam_size = num_decodes
  batch_size = inputs.shape[0]
  end_marker = np.array(eos_id)
  if max_decode_len is None:
    max_decode_len = inputs.shape[1]
  max_decode_len += 1  # :1208

  right_aligned_input = None
  live_seqs = None
  if initial_index is not None:  # :1212-1235
    initial_index = np.asarray(initial_index)
    right_aligned_input = _right_align_prompts(inputs)
    length = inputs.shape[1]
    inputs = np.pad(right_aligned_input[:, -1][:, None],
                    ((0, 0), (0, length - 1)), constant_values=0)
    live_seqs = np.pad(right_aligned_input[:, -1][:, None],
                       ((0, 0), (0, max_decode_len - 1)), constant_values=0)
    live_seqs = np.broadcast_to(
        live_seqs[:, None, :],
        (live_seqs.shape[0], num_decodes, live_seqs.shape[-1])).astype(_I32)
  else:
    initial_index = np.zeros((batch_size,), dtype=_I32)

  state = beam_init(batch_size, beam_size, max_decode_len, cache, cache_offset,
                    live_seqs=live_seqs, initial_index=initial_index)

  min_brevity_penalty = brevity_penalty(alpha, max_decode_len)  # :1268

  def cond(state: BeamState) -> bool:  # :1250-1300
    cur_index = state.cur_index + np.min(state.initial_index)
    not_at_end = cur_index < max_decode_len - 1
    exceed_max_decode_step = (max_decode_step > 0) & np.all(
        state.cur_index >= max_decode_step)
    best_live_scores = (state.live_logprobs[:, -1:] /
                        min_brevity_penalty).astype(_F32)
    worst_finished_scores = np.min(state.finished_scores, axis=1,
                                   keepdims=True)
    worst_finished_scores = np.where(state.finished_flags,
                                     worst_finished_scores,
                                     _F32(NEG_INF_VALUE))
    search_terminated = np.all(worst_finished_scores > best_live_scores)
    raw_min_log_prob = _F32(min_log_prob) / min_brevity_penalty
    none_pass_min_prob_check = np.all(
        best_live_scores < raw_min_log_prob) & (state.cur_index > 0)
    return bool(not_at_end & (~search_terminated) &
                (~none_pass_min_prob_check) & (~exceed_max_decode_step))

  def body(state: BeamState) -> BeamState:  # :1302-1506
    cur = int(state.cur_index)
    flat_ids = flatten_beam_dim(state.live_seqs[:, :, cur:cur + 1])
    flat_cache = cache_map(
        functools.partial(flatten_beam_dim, offset=cache_offset), state.cache)
    decoding_state = DecodingState(
        cur_index=state.cur_index,
        sequences=flatten_beam_dim(state.live_seqs), cur_token=flat_ids,
        cache=flat_cache)
    flat_logits, new_flat_cache = tokens_to_logits(decoding_state)
    flat_logits = np.asarray(flat_logits, dtype=_F32)
    logits = unflatten_beam_dim(flat_logits, batch_size, beam_size)
    new_cache = cache_map(
        lambda x: unflatten_beam_dim(x, batch_size, beam_size, cache_offset),
        new_flat_cache)

    candidate_log_probs = log_softmax(logits)  # :1340
    log_probs = (candidate_log_probs +
                 state.live_logprobs[:, :, None]).astype(_F32)  # :1343-1345
    vocab_size = log_probs.shape[-1]
    beams_to_keep = 2 * beam_size
    flat_log_probs = log_probs.reshape((batch_size, beam_size * vocab_size))
    topk_log_probs, topk_indices = top_k_two_stage(flat_log_probs,
                                                   k=beams_to_keep)
    raw_topk_log_probs = topk_log_probs

    topk_ids = topk_indices % vocab_size  # :1366
    # :1374-1376.  At the last step cur + 1 == inputs.shape[1]; a traced scalar
    # index lowers to a dynamic slice, whose start XLA clamps into range.
    col = min(cur + 1, inputs.shape[1] - 1)
    next_input_token = inputs[:, None].astype(_I32)[:, :, col]
    out_of_prompt = next_input_token == 0
    inside_prompt_log_probs = np.concatenate([
        np.zeros((batch_size, 1), dtype=topk_log_probs.dtype),
        np.full_like(topk_log_probs[:, :beams_to_keep - 1], NEG_INF_VALUE)
    ], axis=1)
    topk_log_probs = (topk_log_probs * out_of_prompt +
                      inside_prompt_log_probs * ~out_of_prompt).astype(_F32)
    topk_ids = topk_ids * out_of_prompt + next_input_token * ~out_of_prompt
    topk_ids = topk_ids[:, :, None]

    topk_beam_indices = topk_indices // vocab_size  # :1404
    topk_seq = gather_beams(state.live_seqs, topk_beam_indices, batch_size,
                            beam_size, beams_to_keep).copy()
    topk_seq[:, :, cur + 1:cur + 2] = topk_ids  # :1412-1414

    newly_finished = topk_seq[:, :, cur + 1] == end_marker  # :1419
    new_log_probs = (topk_log_probs +
                     newly_finished * _F32(NEG_INF_VALUE)).astype(_F32)
    _, new_topk_indices = top_k(new_log_probs, beam_size)  # :1426
    new_topk_indices = np.flip(new_topk_indices, axis=1)
    top_alive_seq, top_alive_log_probs = gather_beams(
        [topk_seq, new_log_probs], new_topk_indices, batch_size, 2 * beam_size,
        beam_size)
    top_alive_indices = gather_beams(topk_beam_indices, new_topk_indices,
                                     batch_size, 2 * beam_size, beam_size)
    top_alive_cache = cache_gather_beams(new_cache, top_alive_indices,
                                         batch_size, beam_size, beam_size,
                                         True, cache_offset)

    lengths = state.cur_index + 1  # :1461-1468
    topk_lengths = np.repeat(initial_index[:, None], beams_to_keep, axis=1)
    lengths = (topk_lengths + lengths).astype(_I32)
    new_scores = (topk_log_probs / brevity_penalty(alpha, lengths)).astype(
        _F32)  # :1470
    new_scores = (new_scores +
                  (~newly_finished) * _F32(NEG_INF_VALUE)).astype(_F32)

    finished_seqs = np.concatenate([state.finished_seqs, topk_seq], axis=1)
    finished_scores = np.concatenate([state.finished_scores, new_scores],
                                     axis=1)
    finished_flags = np.concatenate([state.finished_flags, newly_finished],
                                    axis=1)
    top_finished_seq, top_finished_scores, top_finished_flags = (
        gather_topk_beams([finished_seqs, finished_scores, finished_flags],
                          finished_scores, batch_size, beam_size))

    if trace is not None:
      trace.append(dict(
          cur_index=cur, flat_logits=flat_logits,
          flat_log_probs=flat_log_probs, topk_log_probs=raw_topk_log_probs,
          topk_indices=topk_indices, new_topk_indices=new_topk_indices,
          top_alive_indices=top_alive_indices,
          live_logprobs=top_alive_log_probs, live_seqs=top_alive_seq,
          finished_scores=top_finished_scores, finished_seqs=top_finished_seq,
          finished_flags=top_finished_flags))

    return BeamState(
        cur_index=state.cur_index + 1, live_logprobs=top_alive_log_probs,
        finished_scores=top_finished_scores, live_seqs=top_alive_seq,
        finished_seqs=top_finished_seq, finished_flags=top_finished_flags,
        cache=top_alive_cache, initial_index=initial_index)

  while cond(state):  # :1509-1511
    state = body(state)

  any_finished = np.any(state.finished_flags, axis=1)  # :1516-1528
  finished_seqs = np.where(any_finished[:, None, None], state.finished_seqs,
                           state.live_seqs)
  finished_scores = np.where(any_finished[:, None], state.finished_scores,
                             state.live_logprobs)

  if right_aligned_input is not None:  # :1532-1564
    finished_seqs = finished_seqs[:, :, 1:]
    right_aligned_input = np.broadcast_to(
        right_aligned_input[:, None, :],
        (batch_size, finished_seqs.shape[1], right_aligned_input.shape[-1]))
    finished_seqs = np.concatenate([right_aligned_input, finished_seqs],
                                   axis=-1)
    flat_finished_seqs = np.reshape(finished_seqs,
                                    (-1, finished_seqs.shape[-1]))
    flat_finished_seqs = _left_align_prompts(flat_finished_seqs)
    left_aligned_seqs = np.reshape(flat_finished_seqs, finished_seqs.shape)
    finished_seqs = left_aligned_seqs[:, :, :max_decode_len - 1]
  else:
    finished_seqs = finished_seqs[:, :, 1:]  # :1567

  return finished_seqs, finished_scores
