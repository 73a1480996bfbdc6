"""NumPy restatement of the inference slice of t5x/models.py
(EncoderDecoderModel.predict_batch and helpers) — test oracle, not product
code.  `Transformer` stands in for the flax module with the same
`apply(variables, *args, method=..., mutable=..., **kwargs)` call shape.
"""

import dataclasses
import functools
import inspect
from typing import Any, Callable, Mapping, MutableMapping, Optional, Tuple

import numpy as np

from oracle import decoding
from oracle import t5


class Transformer:
  """network.Transformer (t5x/examples/t5/network.py:295-461) behind a
  flax-like `apply`."""

  def __init__(self, config: t5.T5Config, hoist_cross_kv: bool = True,
               scan_layers: bool = False):
    self.config = config
    self.dtype = config.dtype
    # t5x/examples/scalable_t5/network.py:324-352: with the decoder stack under
    # a scan (variable_axes={'cache': 0}) every cache leaf carries a leading
    # layer axis, [layers, batch, ...], under one 'decoder' scope, and
    # t5x/models.py:739-748 then decodes with cache_offset=1.  The layer
    # arithmetic is unchanged; only the cache tree's layout differs.
    self.scan_layers = scan_layers
    # Cross-attention K/V depend only on `encoded`; projecting them once per
    # batch is value-identical to the reference's per-step projection.
    self.hoist_cross_kv = hoist_cross_kv
    self._cross_kv_cache = None

  def apply(self, variables, *args, method=None, mutable=False, **kwargs):
    name = '__call__' if method is None else method.__name__
    return getattr(self, '_' + name.strip('_'))(variables, *args,
                                                mutable=mutable, **kwargs)

  # Bound-method handles so callers can write `method=module.encode`.
  def encode(self, *a, **k):
    raise TypeError('call through apply(..., method=module.encode)')

  def decode(self, *a, **k):
    raise TypeError('call through apply(..., method=module.decode)')

  def _encode(self, variables, encoder_input_tokens, encoder_segment_ids=None,
              enable_dropout=True, mutable=False):
    del encoder_segment_ids, enable_dropout, mutable
    return t5.encode(variables['params'], self.config, encoder_input_tokens)

  def _cross_kv(self, params, encoded):
    if not self.hoist_cross_kv:
      return None
    key = id(encoded)
    if self._cross_kv_cache is None or self._cross_kv_cache[0] != key:
      self._cross_kv_cache = (key, encoded,
                              t5.project_cross_kv(params, self.config, encoded))
    return self._cross_kv_cache[2]

  def _decode(self, variables, encoded, encoder_input_tokens,
              decoder_input_tokens, decoder_target_tokens,
              enable_dropout=True, decode=False, max_decode_length=None,
              mutable=False):
    del enable_dropout
    params = variables['params']
    if decode:
      cache = variables['cache']
      if self.scan_layers:
        cache = _unstack_cache(cache, self.config.num_decoder_layers)
      logits, cache = t5.decode(
          params, self.config, encoded, encoder_input_tokens,
          decoder_input_tokens, decoder_target_tokens, decode=True,
          cache=cache, max_decode_length=max_decode_length,
          cross_kv=self._cross_kv(params, encoded))
      if self.scan_layers:
        cache = _stack_cache(cache, self.config.num_decoder_layers)
      return (logits, {'cache': cache}) if mutable else logits
    return t5.decode(params, self.config, encoded, encoder_input_tokens,
                     decoder_input_tokens, decoder_target_tokens)

  def _call(self, variables, encoder_input_tokens, decoder_input_tokens,
            decoder_target_tokens, enable_dropout=True, decode=False,
            mutable=False):
    if decode and 'cache' not in variables:
      # Cache-initialisation pass (t5x/models.py:542-552): only shapes matter.
      b, l = np.shape(decoder_input_tokens)
      cache = t5.init_cache(self.config, b, l)
      if self.scan_layers:
        cache = _stack_cache(cache, self.config.num_decoder_layers)
      return None, {'cache': cache}
    encoded = self._encode(variables, encoder_input_tokens)
    return self._decode(variables, encoded, encoder_input_tokens,
                        decoder_input_tokens, decoder_target_tokens,
                        enable_dropout=enable_dropout, decode=decode,
                        mutable=mutable)


_CACHE_LEAVES = ('cached_key', 'cached_value', 'cache_index')


def _stack_cache(cache, num_layers):
  """Per-layer cache tree -> the scanned layout: one 'decoder' scope whose
  leaves have a leading layer axis."""
  per = [cache['decoder'][f'layers_{i}']['self_attention']
         for i in range(num_layers)]
  return {'decoder': {'decoder': {'self_attention': {
      n: np.stack([np.asarray(p[n]) for p in per]) for n in _CACHE_LEAVES}}}}


def _unstack_cache(cache, num_layers):
  sa = cache['decoder']['decoder']['self_attention']
  return {'decoder': {f'layers_{i}': {'self_attention': {
      n: np.asarray(sa[n])[i] for n in _CACHE_LEAVES}}
                      for i in range(num_layers)}}


@dataclasses.dataclass
class DecoderParams:
  """t5x/models.py:358-361."""
  return_all_decodes: bool = False
  num_decodes: int = 1


@dataclasses.dataclass
class _Vocab:
  eos_id: int = 1


class EncoderDecoderModel:
  """Inference slice of t5x/models.py:364-758."""

  def __init__(self, module, decode_fn: Callable = decoding.beam_search,
               output_vocabulary: Any = None,
               default_decoder_params: Optional[DecoderParams] = None):
    self.module = module
    self._decode_fn = decode_fn
    self._output_vocabulary = output_vocabulary or _Vocab()
    self._default_decoder_params = default_decoder_params or DecoderParams()

  @property
  def decode_fn(self):
    return self._decode_fn

  @property
  def output_vocabulary(self):
    return self._output_vocabulary

  def _compute_logits_from_slice(self, decoding_state, params, encoded_inputs,
                                 raw_inputs, max_decode_length):
    """t5x/models.py:484-515."""
    flat_ids = decoding_state.cur_token
    flat_cache = decoding_state.cache
    flat_logits, new_vars = self.module.apply(
        {'params': params, 'cache': flat_cache}, encoded_inputs, raw_inputs,
        flat_ids, flat_ids, enable_dropout=False, decode=True,
        max_decode_length=max_decode_length, mutable=['cache'],
        method=self.module.decode)
    flat_logits = np.squeeze(flat_logits, axis=1)
    return flat_logits, new_vars['cache']

  def _compute_kv_cache(self, params, encoded_inputs, encoder_input_tokens,
                        decoder_input_tokens, prefill_decoder_prompt=False):
    """t5x/models.py:517-582, no-prefill branch."""
    del encoded_inputs
    _, initial_variables = self.module.apply(
        {'params': params},
        encoder_input_tokens=np.ones_like(encoder_input_tokens),
        decoder_input_tokens=np.ones_like(decoder_input_tokens),
        decoder_target_tokens=np.ones_like(decoder_input_tokens),
        mutable=['cache'], decode=True, enable_dropout=False)
    cache = initial_variables['cache']
    if prefill_decoder_prompt:
      raise NotImplementedError('examples/t5 decode() has no `prefill` kwarg')
    return cache, None

  def predict_batch(self, params, batch, rng=None):
    """t5x/models.py:177-193."""
    return self.predict_batch_with_aux(params=params, batch=batch, rng=rng)[0]

  def predict_batch_with_aux(
      self, params, batch, rng=None,
      decoder_params: Optional[MutableMapping[str, Any]] = None,
      return_all_decodes: bool = None, num_decodes: int = None,
      prompt_with_targets: bool = False):
    """t5x/models.py:584-758."""
    if return_all_decodes is None:
      return_all_decodes = self._default_decoder_params.return_all_decodes
    if num_decodes is None:
      num_decodes = self._default_decoder_params.num_decodes

    encoder_input_tokens = batch['encoder_input_tokens']
    decoder_input_tokens = batch['decoder_input_tokens']
    if prompt_with_targets:  # :658-662
      decoder_prompt_inputs = decoder_input_tokens * (
          decoder_input_tokens != self.output_vocabulary.eos_id)
    else:
      decoder_prompt_inputs = np.zeros_like(decoder_input_tokens)

    encoded_inputs = self.module.apply(
        {'params': params}, encoder_input_tokens, enable_dropout=False,
        method=self.module.encode)

    # :674-687 prefill needs `initial_index` on the decode fn AND `prefill` on
    # module.decode; the examples/t5 module has no `prefill`.
    prefill_decoder_prompt = (
        'initial_index' in inspect.signature(self.decode_fn).parameters and
        'prefill' in inspect.signature(self.module.decode).parameters)
    cache, initial_index = self._compute_kv_cache(
        params, encoded_inputs=encoded_inputs,
        encoder_input_tokens=encoder_input_tokens,
        decoder_input_tokens=decoder_prompt_inputs,
        prefill_decoder_prompt=prefill_decoder_prompt)

    tokens_ids_to_logits = functools.partial(
        self._compute_logits_from_slice, params=params,
        encoded_inputs=decoding.flat_batch_beam_expand(encoded_inputs,
                                                       num_decodes),
        raw_inputs=decoding.flat_batch_beam_expand(encoder_input_tokens,
                                                   num_decodes),
        max_decode_length=decoder_input_tokens.shape[1])

    if decoder_params is None:
      decoder_params = {}
    if initial_index is not None:
      decoder_params['initial_index'] = initial_index
    if rng is not None:  # :724-732
      if decoder_params.get('decode_rng') is not None:
        raise ValueError(
            f'Got RNG both from the `rng` argument ({rng}) and'
            " `decoder_params['decode_rng']`"
            f' ({decoder_params["decode_rng"]}). Please specify one or the'
            ' other.')
      decoder_params['decode_rng'] = rng

    scanned = hasattr(self.module, 'scan_layers') and self.module.scan_layers
    if 'eos_id' not in decoder_params:
      decoder_params['eos_id'] = self.output_vocabulary.eos_id or 1
    decodes, scores = self._decode_fn(
        inputs=decoder_prompt_inputs, cache=cache,
        tokens_to_logits=tokens_ids_to_logits, num_decodes=num_decodes,
        cache_offset=1 if scanned else 0, **decoder_params)

    if return_all_decodes:
      return decodes, {'scores': scores}
    return decodes[:, -1, :], {'scores': scores[:, -1]}
