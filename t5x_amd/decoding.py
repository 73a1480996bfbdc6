"""Decode loops with the reference's call signatures, driven from Python over
the HIP kernels (t5x/decoding.py is the interface being mirrored; line numbers
below refer to it).

Arrays are torch tensors on the GPU.  `tokens_to_logits` is any callable
`DecodingState -> (logits [rows, vocab], new_cache)`; NumPy results are
uploaded.  The per-step selection work — log_softmax, prefix add, top-2K over
beam x vocab, beam bookkeeping, cache reorder, sampling — runs in the kernels
declared in include/t5d.h; torch is used for allocation, views and the handful
of tiny prologue/epilogue array edits outside the step loop.

Contract differences from the functional reference, both invisible to a
caller that follows the protocol:
  * caches are updated IN PLACE: `tokens_to_logits` may mutate and return the
    cache it was given, and `cache_gather_beams` permutes beam slices in place;
  * `decode_rng` is an integer seed, a torch.Generator, or an object with a
    `noise(step, shape)` method returning that step's Gumbel tensor
    (jax.random.categorical(key, x) == argmax(x + gumbel)).
"""

import collections
import dataclasses
import functools
from typing import Any, Callable, Mapping, Optional, Tuple, Union

import numpy as np
import torch

from t5x_amd import ops

NEG_INF = np.array(-1.0e7)  # :33
NEG_INF_VALUE = -1.0e7
MIN_TEMPERATURE = np.array(1e-4)  # :39


def _device():
  if not torch.cuda.is_available():
    raise RuntimeError('t5x_amd.decoding needs a GPU: the decode loops run on '
                       'HIP kernels and have no CPU fallback')
  return torch.device('cuda')


def _dev(x, dtype=None):
  """Uploads array-likes; passes GPU tensors through."""
  if isinstance(x, torch.Tensor):
    t = x if x.is_cuda else x.to(_device())
  else:
    t = torch.as_tensor(np.asarray(x), device=_device())
  if dtype is not None and t.dtype != dtype:
    t = t.to(dtype)
  return t


@dataclasses.dataclass
class DecodingState:
  """:42-66."""
  cur_index: torch.Tensor
  sequences: torch.Tensor
  cur_token: torch.Tensor
  cache: Mapping[str, Any]


@dataclasses.dataclass
class SamplingLoopState:
  """:74-99."""
  step: torch.Tensor
  cur_index: torch.Tensor
  sequences: torch.Tensor
  cache: Mapping[str, Any]
  cur_token: torch.Tensor
  ended: torch.Tensor
  rng: Any
  log_prob: torch.Tensor

  def replace(self, **kw):
    return dataclasses.replace(self, **kw)


# ------------------------------------------------------------------------------
# cache / beam helpers (:739-915)
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


_NEVER_MAPPED = ('cached_bias', 'position_embedder_index')


def cache_map(fn, cache, apply_to_index: bool = False):
  """:739-770 — `cache_index` leaves are skipped unless apply_to_index; leaves
  named cached_bias / position_embedder_index always are."""
  flat_cache = _flatten_dict(cache)
  keyvals = {
      k: v for k, v in flat_cache.items()
      if (apply_to_index or k[-1] != 'cache_index') and
      k[-1] not in _NEVER_MAPPED
  }
  flat_cache.update({k: fn(v) for k, v in keyvals.items()})
  return _unflatten_dict(flat_cache)


def _check_cache_room(cache, positions: int, expect_empty: bool):
  """A decode loop writes one cache column per iteration: a cache shorter than
  the loop, or one that already holds steps when the loop starts from zero,
  would push cache_index past the end (the reference silently stops inserting
  there, layers.py:258-275).  Raises instead.  Only trees with this package's
  `cached_key` / `cache_index` leaves are looked at; reading the indices back
  is one host synchronisation per decode."""
  if not isinstance(cache, Mapping):
    return
  flat = _flatten_dict(cache)
  for path, leaf in flat.items():
    if path[-1] == 'cached_key' and hasattr(leaf, 'shape'):
      if leaf.shape[-1] < positions:
        raise ValueError(
            f'the decode loop runs up to {positions} steps but the cache '
            f'{"/".join(map(str, path))} holds {leaf.shape[-1]} positions')
  if not expect_empty:
    return
  idx = [leaf.reshape(-1) for path, leaf in flat.items()
         if path[-1] == 'cache_index' and isinstance(leaf, torch.Tensor)]
  if idx and bool((torch.cat(idx) != 0).any()):
    raise ValueError(
        'the cache already holds decode steps (cache_index != 0) but no '
        '`initial_index` was given: start from a cache as the cache '
        'initialisation returns it')


def add_beam_dim(x, beam_size: int, offset: int = 0):
  """:773-780."""
  x = _dev(x).unsqueeze(offset + 1)
  reps = [1] * x.dim()
  reps[offset + 1] = beam_size
  return x.repeat(*reps)


def flatten_beam_dim(x, offset: int = 0):
  """:783-788."""
  x = _dev(x)
  shape = list(x.shape)
  b = shape.pop(offset)
  shape[offset] *= b
  return x.reshape(shape)


def unflatten_beam_dim(x, batch_size: int, beam_size: int, offset: int = 0):
  """:791-798."""
  x = _dev(x)
  assert batch_size * beam_size == x.shape[offset]
  shape = list(x.shape)
  return x.reshape(shape[:offset] + [batch_size, beam_size] +
                   shape[offset + 1:])


def flat_batch_beam_expand(x, beam_size: int, offset: int = 0):
  """:801-805."""
  return flatten_beam_dim(add_beam_dim(x, beam_size, offset), offset)


def _gather_leaf(x, beam_indices):
  x = _dev(x)
  if x.dtype == torch.bool:
    return ops.gather_beams(x.to(torch.uint8).contiguous(),
                            beam_indices).to(torch.bool)
  return ops.gather_beams(x.contiguous(), beam_indices)


def gather_beams(nested, beam_indices, batch_size, old_beam_size,
                 new_beam_size, one_hot: bool = True):
  """:873-915 (the one-hot contraction is an exact row pick)."""
  del batch_size, old_beam_size, new_beam_size, one_hot
  beam_indices = _dev(beam_indices, torch.int32).contiguous()

  def walk(node):
    if isinstance(node, (list, tuple)):
      return type(node)(walk(n) for n in node)
    if isinstance(node, Mapping):
      return {k: walk(v) for k, v in node.items()}
    return _gather_leaf(node, beam_indices)

  return walk(nested)


def cache_gather_beams(nested, beam_indices, batch_size, old_beam_size,
                       new_beam_size, one_hot: bool = True, offset: int = 0,
                       valid_len: Optional[torch.Tensor] = None):
  """:808-870.  Same-size gathers of [B, beams, ..., L] leaves whose rows are
  16-byte multiples are done in place (valid prefix only when `valid_len`, a
  device int32 scalar, is given); anything else goes out of place."""
  del batch_size, one_hot
  assert offset in (0, 1), 'general offsets not supported'
  beam_indices = _dev(beam_indices, torch.int32).contiguous()

  def gather_fn(x):
    x = _dev(x)
    in_place = (old_beam_size == new_beam_size and x.dim() >= 3 + offset and
                x.is_contiguous() and x.element_size() in (2, 4) and
                (x.shape[-1] * x.element_size()) % 16 == 0 and
                new_beam_size <= 8 and x.data_ptr() % 16 == 0)
    if offset == 0:
      if in_place:
        return ops.cache_gather_beams(x, beam_indices, valid_len=valid_len)
      return _gather_leaf(x, beam_indices)
    if in_place:
      per_layer = x[0].numel() * x.element_size()
      ops.cache_gather_beams(x[0], beam_indices, valid_len=valid_len,
                             n_tensors=x.shape[0],
                             tensor_stride_bytes=per_layer)
      return x
    return torch.stack([_gather_leaf(x[l], beam_indices)
                        for l in range(x.shape[0])])

  return cache_map(gather_fn, nested)


def top_k_two_stage(x, k):
  """:918-966.  The reference's two-stage form is a TPU layout optimisation
  whose result equals lax.top_k; one exact kernel serves both."""
  return ops.top_k(_dev(x, torch.float32).contiguous(), k)


def gather_topk_beams(nested, score_or_log_prob, batch_size, new_beam_size):
  """:969-996."""
  _, topk_indices = ops.top_k(
      _dev(score_or_log_prob, torch.float32).contiguous(), new_beam_size)
  topk_indices = torch.flip(topk_indices, dims=[1]).contiguous()
  return gather_beams(nested, topk_indices, batch_size,
                      score_or_log_prob.shape[1], new_beam_size)


def brevity_penalty(alpha: float, length):
  """:723-733, float32.  A Python int keeps the base in double until the
  power; an int32 array promotes to float32 first."""
  if isinstance(length, (int, np.integer)):
    base = np.float32((5.0 + float(length)) / 6.0)
  else:
    if isinstance(length, torch.Tensor):
      length = length.cpu().numpy()
    base = ((np.float32(5.0) + np.asarray(length).astype(np.float32)) /
            np.float32(6.0))
  return np.power(base, np.float32(alpha), dtype=np.float32)


# ------------------------------------------------------------------------------
# Sampling noise
# ------------------------------------------------------------------------------


class _Key:
  """Stand-in for a PRNG key: which loop step's noise to draw."""

  def __init__(self, source, step):
    self.source, self.step = source, step


class _SeededNoise:
  """Gumbel noise from a torch generator (seeded per step)."""

  def __init__(self, seed):
    self.seed = int(seed)

  def noise(self, step, shape):
    gen = torch.Generator(device=_device())
    gen.manual_seed(self.seed * 1000003 + int(step))
    u = torch.rand(shape, generator=gen, device=_device(),
                   dtype=torch.float32)
    tiny = float(np.finfo(np.float32).tiny)
    return -torch.log(-torch.log(u.clamp_min(tiny)))


def _noise_source(decode_rng):
  if decode_rng is None:
    return _SeededNoise(0)  # :345-346
  if hasattr(decode_rng, 'noise'):
    return decode_rng
  if isinstance(decode_rng, torch.Generator):
    return _SeededNoise(decode_rng.initial_seed())
  return _SeededNoise(int(np.asarray(decode_rng).reshape(-1)[-1]))


# ------------------------------------------------------------------------------
# Temperature sampling (:115-715)
# ------------------------------------------------------------------------------


def _sample_setup(inputs, cache, tokens_to_logits, num_decodes, cache_offset,
                  initial_index, max_decode_steps,
                  max_decode_steps_hard_limit, state_callback_fn,
                  logit_callback_fn):
  """:340-385, what temperature_sample does before its trial: the arguments of
  the single trial (inputs, cache, initial_index, max_decode_steps, use_fused)."""
  if (max_decode_steps_hard_limit is not None and
      max_decode_steps_hard_limit > 0 and max_decode_steps is not None):
    max_decode_steps = np.minimum(max_decode_steps,
                                  max_decode_steps_hard_limit)
  inputs = _dev(inputs, torch.int32)
  # A step function that can run whole iterations on the device exposes
  # `fused_sample_step(...)`; it then owns the caches of all rows (the incoming
  # cache must be the untouched zero cache, which is then not even expanded).
  use_fused = (getattr(tokens_to_logits, 'fused_sample_step', None) is not None
               and getattr(cache, 'fresh', False) and initial_index is None and
               cache_offset == getattr(tokens_to_logits, 'cache_offset', 0) and
               state_callback_fn is None and logit_callback_fn is None)
  if not use_fused:
    _check_cache_room(cache, inputs.shape[1],
                      expect_empty=initial_index is None)
  if use_fused:
    expanded_inputs = (flat_batch_beam_expand(inputs, num_decodes)
                       if num_decodes > 1 else inputs)
    expanded_cache = cache
  elif num_decodes > 1:
    expanded_inputs = flat_batch_beam_expand(inputs, num_decodes)
    expanded_cache = cache_map(
        functools.partial(flat_batch_beam_expand, beam_size=num_decodes,
                          offset=cache_offset),
        cache, apply_to_index=initial_index is not None)
    if initial_index is not None:
      initial_index = flat_batch_beam_expand(
          _dev(initial_index, torch.int32), num_decodes)
  else:
    expanded_inputs, expanded_cache = inputs, cache
  return (expanded_inputs, expanded_cache, initial_index, max_decode_steps,
          use_fused)


def _sort_trials(expanded_decodes, expanded_log_prob, batch_size, num_decodes):
  """:387-409, the trials of each batch item sorted ascending by log-prob."""
  decodes = unflatten_beam_dim(expanded_decodes, batch_size, num_decodes)
  log_prob = unflatten_beam_dim(expanded_log_prob, batch_size, num_decodes)
  # Ascending, stable.  top_k of the negated scores is a stable descending
  # order of -log_prob, i.e. a stable ascending order of log_prob.
  if num_decodes > 1:
    _, idxs = ops.top_k((-log_prob).contiguous(), num_decodes)
    decodes = ops.gather_beams(decodes.contiguous(), idxs)
    log_prob = ops.gather_beams(log_prob.contiguous(), idxs)
  return decodes, log_prob


def temperature_sample(
    inputs, cache, tokens_to_logits, eos_id: int, decode_rng=None,
    num_decodes: int = 1, temperature: Union[float, np.ndarray] = 1.0,
    topk: int = 1, topp: float = 0.0, cache_offset: int = 0,
    initial_index=None, max_decode_steps=None,
    max_decode_steps_hard_limit: Optional[int] = None,
    rescale_log_probs: bool = True,
    state_callback_fn: Optional[Callable] = None,
    logit_callback_fn: Optional[Callable] = None,
):
  """:115-409 -> (decodes [B, num_decodes, L] i32, log_prob [B, num_decodes])
  sorted ascending by log-prob."""
  (expanded_inputs, expanded_cache, initial_index, max_decode_steps,
   use_fused) = _sample_setup(
       inputs, cache, tokens_to_logits, num_decodes, cache_offset,
       initial_index, max_decode_steps, max_decode_steps_hard_limit,
       state_callback_fn, logit_callback_fn)
  expanded_decodes, expanded_log_prob = _temperature_sample_single_trial(
      expanded_inputs, expanded_cache, tokens_to_logits, eos_id, decode_rng,
      num_decodes, temperature, topk, topp, initial_index=initial_index,
      max_decode_steps=max_decode_steps, rescale_log_probs=rescale_log_probs,
      state_callback_fn=state_callback_fn, logit_callback_fn=logit_callback_fn,
      use_fused=use_fused)
  return _sort_trials(expanded_decodes, expanded_log_prob,
                      np.shape(inputs)[0], num_decodes)


def begin_temperature_sample(
    inputs, cache, tokens_to_logits, eos_id: int, decode_rng=None,
    num_decodes: int = 1, temperature: Union[float, np.ndarray] = 1.0,
    topk: int = 1, topp: float = 0.0, cache_offset: int = 0,
    initial_index=None, max_decode_steps=None,
    max_decode_steps_hard_limit: Optional[int] = None,
    rescale_log_probs: bool = True,
    state_callback_fn: Optional[Callable] = None,
    logit_callback_fn: Optional[Callable] = None,
):
  """temperature_sample set up but not run -> Decode."""
  (expanded_inputs, expanded_cache, initial_index, max_decode_steps,
   use_fused) = _sample_setup(
       inputs, cache, tokens_to_logits, num_decodes, cache_offset,
       initial_index, max_decode_steps, max_decode_steps_hard_limit,
       state_callback_fn, logit_callback_fn)
  loop = SampleLoop(expanded_inputs, expanded_cache, tokens_to_logits, eos_id,
                    decode_rng, num_decodes, temperature, topk, topp,
                    initial_index, max_decode_steps, rescale_log_probs,
                    state_callback_fn, logit_callback_fn, use_fused)
  return Decode(loop, functools.partial(_sort_trials,
                                        batch_size=np.shape(inputs)[0],
                                        num_decodes=num_decodes))


temperature_sample.begin = begin_temperature_sample


class Decode:
  """A decode that has been set up but not necessarily run: the loop object
  plus what turns the loop's final state into the function's return value.
  `run()` runs it to its end; `start()` / `poll()` run it without waiting, so
  that several can be in flight; `result()` is the decode function's return
  value (it runs whatever is left of the loop)."""

  def __init__(self, loop, epilogue=None):
    self.loop, self._epilogue = loop, epilogue
    self._result = None
    self._ran = False

  def run(self):
    self.loop.run()
    self._ran = True

  def start(self, check_every: int = 8):
    self.loop.start(check_every)

  def poll(self, block: bool = False) -> bool:
    if self._ran:
      return True
    self._ran = self.loop.poll(block)
    return self._ran

  def result(self):
    if self._result is None:
      if not self._ran:
        if self.loop._tickets is None:
          self.loop.run()
        else:
          while not self.loop.poll(block=True):
            pass
        self._ran = True
      out = self.loop.finish()
      self._result = out if self._epilogue is None else self._epilogue(*out)
    return self._result


class _InFlight:
  """start() / poll() for a loop object: the loop runs on the device in chunks
  of iterations, a few of them enqueued ahead, and the host only asks whether
  the oldest chunk has ended and what the loop condition was then.  Nothing
  here waits unless asked to, so one host thread can keep several decodes (each
  on its own streams) in flight.  Iterations enqueued after the condition
  turned false change nothing on the device, so the final state is the one the
  plain loop reaches."""

  finished = False   # set by finish(): the decode context may serve another loop
  _ended = False
  _tickets = None

  def start(self, check_every: int = 8, ahead: int = 2):
    """Begins running the loop; returns at once (without a fused step: after
    running it to its end)."""
    self._tickets = collections.deque()
    if self.fused is None:
      self.run()
      self._ended = True
      return
    if ahead > self.fused.CHUNK_SLOTS:
      raise ValueError(f'at most {self.fused.CHUNK_SLOTS} chunks ahead')
    self._check_every = int(check_every)
    if not self.cond():
      self._ended = True
      return
    for _ in range(ahead):
      self._push_chunk()

  def _push_chunk(self):
    ticket = self.fused.launch_chunk(self._check_every)
    if ticket is not None:
      self._tickets.append(ticket)
      self.step += self._check_every

  def poll(self, block: bool = False) -> bool:
    """True once the loop has ended (finish() then returns its results).
    Enqueues further chunks as earlier ones end; with `block`, first waits
    for the oldest chunk in flight."""
    if self._tickets is None:
      raise ValueError('poll() before start()')
    while not self._ended:
      if not self._tickets:  # nothing left to enqueue
        self._ended = True
        break
      running = self.fused.chunk_running(self._tickets[0], block)
      block = False
      if running is None:
        break
      self._tickets.popleft()
      if running:
        self._push_chunk()
      else:
        self._ended = True
        self._tickets.clear()
    return self._ended


def run_in_flight(loops, check_every: int = 8):
  """Runs loop objects (BeamLoop, SampleLoop, or anything with start / poll)
  to their ends together: all are started, then the host waits on one of them
  at a time while keeping the others fed."""
  loops = list(loops)
  for loop in loops:
    loop.start(check_every)
  pending = [l for l in loops if not l.poll()]
  while pending:
    pending[0].poll(block=True)
    pending = [l for l in pending if not l.poll()]


class SampleLoop(_InFlight):
  """The loop of _temperature_sample_single_trial (:412-715) as an object:
  `cond()` / `body()` are the while-loop's condition and body, `finish()` the
  epilogue; `advance(n)` runs n iterations without reading the condition back
  (with the fused loop, iterations after every row ended change nothing).
  Exposing the pieces lets a caller time or single-step the loop."""

  def __init__(self, inputs, cache, tokens_to_logits, eos_id: int, prng_key,
               num_decodes: int = 1,
               temperature: Union[float, np.ndarray] = 1.0, topk: int = 20,
               topp: float = 0.0, initial_index=None, max_decode_steps=None,
               rescale_log_probs: bool = True,
               state_callback_fn: Optional[Callable] = None,
               logit_callback_fn: Optional[Callable] = None,
               use_fused: bool = False):
    if topp and topk:
      raise ValueError('At most one of `topp` or `topk` may be non-zero.')
    dev = _device()
    inputs = _dev(inputs, torch.int32)
    batch_size, length = inputs.shape
    inputs_np = inputs.cpu().numpy()

    max_decode_len = np.full((batch_size,), length, np.int32)
    if max_decode_steps is not None:  # :438-455
      if np.ndim(max_decode_steps) == 0 and max_decode_steps > length:
        raise ValueError('Cannot decode more steps than the sequence length.')
      max_decode_len = np.minimum(
          length, np.sum(inputs_np != 0, axis=1) + max_decode_steps).astype(
              np.int32)

    sequences_np = np.concatenate(
        [inputs_np, np.zeros((batch_size, 2), np.int32)], axis=1)  # :465-470
    if initial_index is None:
      i0 = np.zeros((batch_size,), np.int32)
      token0 = np.zeros((batch_size,), np.int32)
    else:
      i0 = _dev(initial_index).cpu().numpy().astype(np.int32)
      token0 = np.take_along_axis(sequences_np, i0[:, None], axis=1)[:, 0]
    initial_eos = np.sum(sequences_np == eos_id, axis=-1).astype(np.int32)

    temps = np.asarray(temperature, dtype=np.float32)
    if temps.ndim == 1:  # per-item temperatures (:595-612)
      temps = np.repeat(temps, num_decodes)
    else:
      temps = np.full((batch_size,), float(temps), np.float32)
    self.any_sampling = bool(np.any(temps > np.float32(MIN_TEMPERATURE)))

    self.tokens_to_logits, self.cache = tokens_to_logits, cache
    self.eos_id, self.topk, self.topp = eos_id, topk, topp
    self.rescale_log_probs = rescale_log_probs
    self.state_callback_fn = state_callback_fn
    self.logit_callback_fn = logit_callback_fn
    self.sequences = torch.as_tensor(sequences_np, device=dev).contiguous()
    self.cur_index = torch.as_tensor(i0, device=dev)
    self.cur_token = torch.as_tensor(token0.astype(np.int32), device=dev)
    self.ended = torch.zeros((batch_size,), dtype=torch.uint8, device=dev)
    self.log_prob = torch.zeros((batch_size,), dtype=torch.float32, device=dev)
    self.mdl = torch.as_tensor(max_decode_len, device=dev)
    self.eos0 = torch.as_tensor(initial_eos, device=dev)
    self.temps_dev = torch.as_tensor(temps, device=dev)
    self.all_ended = torch.zeros((), dtype=torch.int32, device=dev)
    self.tokens = torch.empty((batch_size,), dtype=torch.int32, device=dev)
    self.tok_lp = torch.empty((batch_size,), dtype=torch.float32, device=dev)
    # scratch memory for the token choice (both loops hand one over, so both
    # take the same kernels)
    self.sample_ws = ops.sample_tokens_workspace(batch_size, dev)
    self.source = _noise_source(prng_key)
    self.step = 0
    self.fused = None
    if use_fused:
      self.fused = tokens_to_logits.fused_sample_step(
          sequences=self.sequences, cur_index=self.cur_index,
          cur_token=self.cur_token, ended=self.ended, log_prob=self.log_prob,
          max_decode_len=self.mdl, initial_eos_count=self.eos0,
          temperature=self.temps_dev, all_ended=self.all_ended, eos_id=eos_id,
          topk=topk, topp=topp, rescale=rescale_log_probs,
          noise_source=self.source if self.any_sampling else None,
          owner=self)

  def _loop_state(self):
    return SamplingLoopState(
        torch.tensor(self.step, dtype=torch.int32), self.cur_index,
        self.sequences, self.cache, self.cur_token[:, None],
        self.ended.bool()[:, None], _Key(self.source, self.step),
        self.log_prob)

  def cond(self) -> bool:
    """:509-515, not every row ended (reads one flag back)."""
    if self.fused is not None:
      return self.fused.running()
    return not bool(self.all_ended.item())

  def body(self):
    """:517-700."""
    if self.fused is not None:
      self.fused.advance(1)
      self.step += 1
      return
    if self.state_callback_fn is not None:
      st = self.state_callback_fn(self._loop_state())
      self.sequences = _dev(st.sequences, torch.int32).contiguous()
      self.cur_index = _dev(st.cur_index, torch.int32).contiguous()
      self.cache = st.cache
    decoding_state = DecodingState(cur_index=self.cur_index,
                                   sequences=self.sequences[:, :-2],
                                   cur_token=self.cur_token[:, None],
                                   cache=self.cache)
    logits, self.cache = self.tokens_to_logits(decoding_state)
    if self.logit_callback_fn is not None:
      if not isinstance(logits, torch.Tensor):
        logits = np.array(logits, dtype=np.float32)
      logits = self.logit_callback_fn(logits, self._loop_state())
    logits = _dev(logits, torch.float32).contiguous()
    gumbel = None
    if self.any_sampling:
      gumbel = _dev(self.source.noise(self.step, tuple(logits.shape)),
                    torch.float32).contiguous()
    ops.sample_tokens(logits, gumbel, self.temps_dev, self.topk, self.topp,
                      self.rescale_log_probs, self.tokens, self.tok_lp,
                      workspace=self.sample_ws)
    ops.sample_update(self.tokens, self.tok_lp, self.sequences, self.cur_index,
                      self.cur_token, self.ended, self.log_prob, self.mdl,
                      self.eos0, self.all_ended, self.eos_id)
    self.step += 1

  def advance(self, n: int):
    if self.fused is not None:
      self.fused.advance(n)
      self.step += n
      return
    for _ in range(n):
      self.body()

  def run(self):
    if self.fused is not None:
      self.step = self.fused.run()
      return
    while True:  # nothing has ended at step 0
      self.body()
      if not self.cond():
        break

  def finish(self):
    if self.fused is not None:
      self.fused.finish()
      if self._tickets is not None:  # ran in chunks: iterations executed
        self.step = int(self.fused.step_count.item())
      # the context's buffers serve the next call too: hand out copies
      out = (self.fused.sequences[:, 1:-1].clone(),
             self.fused.log_prob.clone())
      self.finished = True
      return out
    if self.state_callback_fn is not None:
      st = self.state_callback_fn(self._loop_state())
      self.sequences = _dev(st.sequences, torch.int32)
    return self.sequences[:, 1:-1], self.log_prob


def _temperature_sample_single_trial(
    inputs, cache, tokens_to_logits, eos_id: int, prng_key,
    num_decodes: int = 1, temperature: Union[float, np.ndarray] = 1.0,
    topk: int = 20, topp: float = 0.0, initial_index=None,
    max_decode_steps=None, rescale_log_probs: bool = True,
    state_callback_fn: Optional[Callable] = None,
    logit_callback_fn: Optional[Callable] = None,
    use_fused: bool = False,
):
  """:412-715."""
  loop = SampleLoop(inputs, cache, tokens_to_logits, eos_id, prng_key,
                    num_decodes, temperature, topk, topp, initial_index,
                    max_decode_steps, rescale_log_probs, state_callback_fn,
                    logit_callback_fn, use_fused)
  loop.run()
  return loop.finish()


# ------------------------------------------------------------------------------
# Beam search (:999-1569)
# ------------------------------------------------------------------------------


def _right_align_prompts(prompts):
  """:1069-1095 (host side; prompts are small int arrays)."""
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
  """:1098-1120."""
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
  """:1123-1127."""
  prompts = np.asarray(prompts)
  return prompts[np.arange(prompts.shape[0]), np.sum(prompts != 0, axis=1)]


def beam_init(batch_size, beam_size, max_decode_len, cache, offset=0,
              live_seqs=None, initial_index=None):
  """:1024-1066 -> (BeamBuffers, beam-expanded cache)."""
  dev = _device()
  st = ops.BeamBuffers(batch_size, beam_size, max_decode_len, dev)
  st.live_logprobs.copy_(torch.tensor(
      [0.0] + [NEG_INF_VALUE] * (beam_size - 1), dtype=torch.float32,
      device=dev).expand(batch_size, beam_size))
  st.finished_scores.fill_(NEG_INF_VALUE)
  if live_seqs is not None:
    st.live_seqs.copy_(_dev(live_seqs, torch.int32))
  beam_cache = cache_map(lambda x: add_beam_dim(x, beam_size, offset), cache,
                         apply_to_index=live_seqs is not None)
  return st, beam_cache


class BeamLoop(_InFlight):
  """The beam_search loop (:1131-1569) as an object: `cond()` / `body()` are
  the while-loop's condition and body, `finish()` the epilogue.  beam_search()
  below is `while loop.cond(): loop.body()`; exposing the pieces lets a caller
  time or single-step the loop without re-implementing it."""

  def __init__(self, inputs, cache, tokens_to_logits, eos_id: int,
               num_decodes: int = 4, alpha: float = 0.6,
               max_decode_len: Optional[int] = None, max_decode_step: int = -1,
               min_log_prob: float = NEG_INF_VALUE, cache_offset: int = 0,
               initial_index=None):
    dev = _device()
    self.tokens_to_logits = tokens_to_logits
    self.eos_id = eos_id
    self.cache_offset = cache_offset
    self.max_decode_step = max_decode_step
    self.min_log_prob = min_log_prob
    inputs_np = _dev(inputs).cpu().numpy().astype(np.int32)
    self.beam_size = beam_size = num_decodes
    self.batch_size = batch_size = inputs_np.shape[0]
    if max_decode_len is None:
      max_decode_len = inputs_np.shape[1]
    max_decode_len += 1  # :1208
    self.max_decode_len = max_decode_len

    self.right_aligned_input = None
    live_seqs = None
    if initial_index is not None:  # :1212-1235
      initial_index_np = _dev(initial_index).cpu().numpy().astype(np.int32)
      self.right_aligned_input = _right_align_prompts(inputs_np)
      length = inputs_np.shape[1]
      last = self.right_aligned_input[:, -1][:, None]
      inputs_np = np.pad(last, ((0, 0), (0, length - 1)), constant_values=0)
      live_seqs = np.pad(last, ((0, 0), (0, max_decode_len - 1)),
                         constant_values=0)
      live_seqs = np.ascontiguousarray(np.broadcast_to(
          live_seqs[:, None, :], (batch_size, beam_size, max_decode_len)))
    else:
      initial_index_np = np.zeros((batch_size,), np.int32)

    # A step function that can run whole iterations on the device exposes
    # `fused_beam_step(loop)`; it then owns the beam-expanded caches (the
    # incoming cache must be the untouched zero cache) and the state is
    # updated in place.
    factory = getattr(tokens_to_logits, 'fused_beam_step', None)
    use_fused = (factory is not None and initial_index is None and
                 getattr(cache, 'fresh', False))
    self.fused = None
    if not use_fused:
      _check_cache_room(cache, max_decode_len - 1,
                        expect_empty=initial_index is None)
    self.cur, self._beam_cache = beam_init(
        batch_size, beam_size, max_decode_len, {} if use_fused else cache,
        cache_offset, live_seqs=live_seqs, initial_index=initial_index_np)
    self.nxt = (self.cur if use_fused else
                ops.BeamBuffers(batch_size, beam_size, max_decode_len, dev))
    self.inputs_dev = torch.as_tensor(np.ascontiguousarray(inputs_np),
                                      device=dev)
    self.init_idx_dev = torch.as_tensor(initial_index_np, device=dev)
    max_len_for_bp = max_decode_len + int(initial_index_np.max()) + 2
    self.brevity = torch.as_tensor(
        brevity_penalty(alpha, np.arange(max_len_for_bp, dtype=np.int32)),
        device=dev).contiguous()
    self.min_brevity = float(brevity_penalty(alpha, max_decode_len))  # :1268
    self.min_initial = int(initial_index_np.min())
    self.keep_going = torch.zeros((), dtype=torch.int32, device=dev)
    self.top_alive = torch.empty((batch_size, beam_size), dtype=torch.int32,
                                 device=dev)
    self.topk_bufs = None
    self.vocab_size = None
    self.step = 0
    if use_fused:
      self.fused = factory(self)
      if self.fused is None:  # configuration not covered: generic path
        _check_cache_room(cache, max_decode_len - 1, expect_empty=True)
        self.cur, self._beam_cache = beam_init(
            batch_size, beam_size, max_decode_len, cache, cache_offset)
        self.nxt = ops.BeamBuffers(batch_size, beam_size, max_decode_len, dev)

  @property
  def beam_cache(self):
    """The beam-expanded caches in the reference's tree layout (with the fused
    loop: copies made on request)."""
    if self.fused is not None:
      return self.fused.cache_tree()
    return self._beam_cache

  def cond(self) -> bool:
    """:1250-1300 (reads one flag back from the device)."""
    if self.fused is not None:
      return self.fused.keep_going()
    ops.beam_cond(self.cur, self.min_brevity, self.min_log_prob,
                  self.max_decode_step, self.min_initial, self.keep_going)
    return bool(self.keep_going.item())

  def run(self, check_every: int = 8):
    """Runs the loop to termination.  With a fused step the condition is read
    back only every `check_every` iterations: iterations enqueued after it
    turned false are no-ops on the device, so the final state is the same."""
    if self.fused is None:
      while self.cond():
        self.body()
      return
    while self.fused.keep_going():
      self.fused.launch(check_every)
      self.step += check_every

  def advance(self, n: int):
    """n loop iterations without looking at the condition in between (with the
    fused loop: iterations past its end change nothing)."""
    if self.fused is not None:
      self.fused.launch(n)
      self.step += n
      return
    for _ in range(n):
      self.body()

  def body(self):
    """:1302-1506."""
    if self.fused is not None:
      self.fused.launch(1)
      self.step += 1
      return
    cur, nxt = self.cur, self.nxt
    B, K, dev = self.batch_size, self.beam_size, cur.live_seqs.device
    step, off = self.step, self.cache_offset
    flat_ids = flatten_beam_dim(cur.live_seqs[:, :, step:step + 1])
    flat_cache = cache_map(functools.partial(flatten_beam_dim, offset=off),
                           self.beam_cache)
    decoding_state = DecodingState(
        cur_index=cur.cur_index, sequences=flatten_beam_dim(cur.live_seqs),
        cur_token=flat_ids, cache=flat_cache)
    flat_logits, new_flat_cache = self.tokens_to_logits(decoding_state)
    flat_logits = _dev(flat_logits, torch.float32).contiguous()
    if self.vocab_size is None:
      self.vocab_size = flat_logits.shape[-1]
      R, k2 = B * K, 2 * K
      self.topk_bufs = (
          torch.empty((B, k2), dtype=torch.float32, device=dev),
          torch.empty((B, k2), dtype=torch.int32, device=dev),
          torch.empty((R,), dtype=torch.float32, device=dev),
          torch.empty((R,), dtype=torch.float32, device=dev),
          torch.empty((2 * R * k2,), dtype=torch.int32, device=dev))
    new_cache = cache_map(lambda x: unflatten_beam_dim(x, B, K, off),
                          new_flat_cache)
    # :1340-1366 log_softmax + prefix add + top-2K over beam x vocab
    topk_vals, topk_idx, _, _ = ops.beam_topk(flat_logits, cur.live_logprobs,
                                              2 * K, self.topk_bufs)
    # :1366-1506 everything after the top-k
    ops.beam_update(cur, nxt, topk_vals, topk_idx, self.inputs_dev,
                    self.init_idx_dev, self.brevity, self.top_alive,
                    self.vocab_size, self.eos_id)
    # :1449-1457.  After this step the caches hold step + 1 valid columns.
    self._beam_cache = cache_gather_beams(new_cache, self.top_alive, B, K, K,
                                         True, off)
    self.cur, self.nxt = nxt, cur
    self.step += 1

  def finish(self):
    """:1513-1569."""
    if self.fused is not None:
      self.fused.finish()
    cur, dev = self.cur, self.cur.live_seqs.device
    # batch items with no finished sequence fall back to the live ones
    any_finished = cur.finished_flags.bool().any(dim=1)
    finished_seqs = torch.where(any_finished[:, None, None], cur.finished_seqs,
                                cur.live_seqs)
    finished_scores = torch.where(any_finished[:, None], cur.finished_scores,
                                  cur.live_logprobs)
    if self.right_aligned_input is not None:  # :1532-1564
      seqs = finished_seqs.cpu().numpy()[:, :, 1:]
      prompt = np.broadcast_to(
          self.right_aligned_input[:, None, :],
          (self.batch_size, seqs.shape[1], self.right_aligned_input.shape[-1]))
      seqs = np.concatenate([prompt, seqs], axis=-1)
      flat = _left_align_prompts(seqs.reshape(-1, seqs.shape[-1]))
      seqs = flat.reshape(seqs.shape)[:, :, :self.max_decode_len - 1]
      finished_seqs = torch.as_tensor(np.ascontiguousarray(seqs), device=dev)
    else:
      finished_seqs = finished_seqs[:, :, 1:]  # :1567
    self.finished = True
    return finished_seqs, finished_scores


def begin_beam_search(
    inputs, cache, tokens_to_logits, eos_id: int, num_decodes: int = 4,
    alpha: float = 0.6, max_decode_len: Optional[int] = None,
    max_decode_step: int = -1, min_log_prob: float = NEG_INF_VALUE,
    decode_rng=None, cache_offset: int = 0, initial_index=None,
):
  """beam_search (:1131-1569) set up but not run -> Decode."""
  del decode_rng
  return Decode(BeamLoop(inputs, cache, tokens_to_logits, eos_id, num_decodes,
                         alpha, max_decode_len, max_decode_step, min_log_prob,
                         cache_offset, initial_index))


def beam_search(
    inputs, cache, tokens_to_logits, eos_id: int, num_decodes: int = 4,
    alpha: float = 0.6, max_decode_len: Optional[int] = None,
    max_decode_step: int = -1, min_log_prob: float = NEG_INF_VALUE,
    decode_rng=None, cache_offset: int = 0, initial_index=None,
):
  """:1131-1569 -> (sequences [B, K, L] i32, scores [B, K] f32), the beam axis
  sorted ascending by score."""
  decode = begin_beam_search(inputs, cache, tokens_to_logits, eos_id,
                             num_decodes, alpha, max_decode_len,
                             max_decode_step, min_log_prob, decode_rng,
                             cache_offset, initial_index)
  decode.run()  # :1509
  return decode.result()


beam_search.begin = begin_beam_search
