"""NumPy restatement of the T5.1.1 network the decode path runs
(t5x/examples/t5/layers.py and network.py) — test oracle, not product code.

Activation dtype `A` is 'float32' or 'bfloat16'.  bfloat16 is emulated on
float32 arrays by rounding to nearest-even at exactly the points where the
reference casts (`jnp.asarray(x, dtype)` / op results in `dtype`); matmuls
accumulate in float32 (the accumulator is backend defined in the reference).

Weight-only int8: a kernel may be given as `{'q': int8 [K, N], 'scale': f32
[N]}`; the dense layer then computes `A(x) @ q` exactly and multiplies each
output channel by its scale before the single rounding to `A`.
"""

import dataclasses
from typing import Any, Mapping, Optional, Sequence, Tuple

import numpy as np

_F32 = np.float32


@dataclasses.dataclass(frozen=True)
class T5Config:
  """t5x/examples/t5/network.py:25-44."""
  vocab_size: int = 32128
  dtype: str = 'float32'
  emb_dim: int = 512
  num_heads: int = 8
  num_encoder_layers: int = 6
  num_decoder_layers: int = 6
  head_dim: int = 64
  mlp_dim: int = 2048
  mlp_activations: Sequence[str] = ('gelu', 'linear')
  logits_via_embedding: bool = False
  float32_attention_logits: bool = False


def bf16_round(x):
  """float32 -> nearest-even bfloat16, returned as float32."""
  x = np.ascontiguousarray(x, dtype=_F32)
  u = x.view(np.uint32)
  bias = np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
  r = (u + bias) & np.uint32(0xFFFF0000)
  return r.view(_F32).reshape(x.shape)


def cast(x, dtype: str):
  """`jnp.asarray(x, dtype)` on the emulated representation."""
  if dtype == 'bfloat16':
    return bf16_round(x)
  return np.asarray(x, dtype=_F32)


def gelu(x):
  """flax.linen.gelu default (approximate=True): tanh form.  PARITY UNPINNED:
  no reference test evaluates it (layers_test.py:538-610 uses relu)."""
  x = np.asarray(x, dtype=_F32)
  c = _F32(np.sqrt(2.0 / np.pi))
  return (x * (_F32(0.5) * (_F32(1.0) + np.tanh(
      c * (x + _F32(0.044715) * (x * x * x)))))).astype(_F32)


def activation(name: str):
  """t5x/examples/t5/layers.py:417-431."""
  if name == 'linear':
    return lambda x: x
  if name == 'gelu':
    return gelu
  if name == 'relu':
    return lambda x: np.maximum(x, _F32(0))
  raise ValueError("don't know how to convert %s to an activation function" %
                   (name,))


def dense_general(x, kernel, dtype: str, out_dtype: Optional[str] = None):
  """t5x/examples/t5/layers.py:364-414: bias-free linear over the last axis;
  input and kernel are cast to `dtype`, the product is produced in `dtype`."""
  x = cast(x, dtype)
  if isinstance(kernel, Mapping):  # weight-only int8
    y = (x @ kernel['q'].astype(_F32)) * np.asarray(kernel['scale'], _F32)
  else:
    y = x @ cast(kernel, dtype)
  return cast(y, out_dtype or dtype)


def layer_norm(x, scale, dtype: str, epsilon: float = 1e-6):
  """T5 RMS norm, t5x/examples/t5/layers.py:683-702."""
  x = np.asarray(x, dtype=_F32)
  mean2 = np.mean(np.square(x), axis=-1, keepdims=True, dtype=_F32)
  inv = (_F32(1.0) / np.sqrt(mean2 + _F32(epsilon))).astype(_F32)
  y = cast(x * inv, dtype)
  return cast(y * cast(scale, dtype), dtype)


def relative_position_bucket(relative_position, bidirectional=True,
                             num_buckets=32, max_distance=128):
  """t5x/examples/t5/layers.py:580-625."""
  ret = 0
  n = -np.asarray(relative_position)
  if bidirectional:
    num_buckets //= 2
    ret = ret + (n < 0).astype(np.int32) * num_buckets
    n = np.abs(n)
  else:
    n = np.maximum(n, 0)
  max_exact = num_buckets // 2
  is_small = n < max_exact
  with np.errstate(divide='ignore'):
    val_if_large = max_exact + (
        np.log(n.astype(np.float32) / max_exact + np.finfo(np.float32).eps) /
        np.log(max_distance / max_exact) *
        (num_buckets - max_exact)).astype(np.int32)
  val_if_large = np.minimum(val_if_large, num_buckets - 1)
  return ret + np.where(is_small, n, val_if_large)


def relpos_bias(rel_embedding, qlen, klen, bidirectional, dtype: str):
  """t5x/examples/t5/layers.py:627-677 -> [1, H, qlen, klen] in `dtype`."""
  context_position = np.arange(qlen, dtype=np.int32)[:, None]
  memory_position = np.arange(klen, dtype=np.int32)[None, :]
  rp_bucket = relative_position_bucket(memory_position - context_position,
                                       bidirectional=bidirectional)
  table = cast(rel_embedding, dtype)  # [H, buckets]
  return table[:, rp_bucket][None]  # one-hot contraction == exact pick


def make_attention_mask(query_input, key_input, pairwise_fn=np.multiply):
  """t5x/examples/t5/layers.py:708-743 -> [batch, 1, len_q, len_kv]."""
  mask = pairwise_fn(np.expand_dims(query_input, -1),
                     np.expand_dims(key_input, -2))
  return np.expand_dims(mask, -3).astype(_F32)


def make_causal_mask(x):
  """t5x/examples/t5/layers.py:746-775."""
  idxs = np.broadcast_to(np.arange(x.shape[-1], dtype=np.int32), x.shape)
  return make_attention_mask(idxs, idxs, np.greater_equal)


def combine_masks(*masks):
  """t5x/examples/t5/layers.py:778-797."""
  masks = [m for m in masks if m is not None]
  if not masks:
    return None
  mask = masks[0]
  for other in masks[1:]:
    mask = np.logical_and(mask, other)
  return mask.astype(_F32)


def combine_biases(*masks):
  """t5x/examples/t5/layers.py:800-818."""
  masks = [m for m in masks if m is not None]
  if not masks:
    return None
  out = masks[0]
  for other in masks[1:]:
    out = out + other
  return out


def make_decoder_mask(decoder_target_tokens):
  """t5x/examples/t5/layers.py:821-884 without packing/prefix-LM inputs:
  causal AND target-padding."""
  causal = make_causal_mask(decoder_target_tokens)
  padding = make_attention_mask(decoder_target_tokens > 0,
                                decoder_target_tokens > 0)
  return combine_masks(causal, padding)


def softmax(x):
  x = np.asarray(x, dtype=_F32)
  e = np.exp(x - np.max(x, axis=-1, keepdims=True))
  return (e / np.sum(e, axis=-1, keepdims=True, dtype=_F32)).astype(_F32)


def dot_product_attention(query, key, value, bias, dtype: str):
  """t5x/examples/t5/layers.py:52-129.  q [b,q,h,d]; k,v [b,k,h,d]."""
  attn_weights = cast(np.einsum('bqhd,bkhd->bhqk', query, key), dtype)
  if bias is not None:
    attn_weights = cast(attn_weights + cast(bias, dtype), dtype)
  attn_weights = cast(softmax(attn_weights), dtype)
  return cast(np.einsum('bhqk,bkhd->bqhd', attn_weights, value), dtype)


def multi_head_attention(params, inputs_q, inputs_kv, mask, bias, *,
                         num_heads, head_dim, dtype, decode=False, cache=None,
                         projected_kv=None):
  """t5x/examples/t5/layers.py:137-346.

  Returns (out, new_cache).  `cache` is the layer's
  {'cached_key','cached_value','cache_index'} dict when `decode`.
  `projected_kv`, if given, is the (key, value) pair the projection of
  `inputs_kv` would produce (cross-attention K/V are the same every step).
  """
  b, ql = inputs_q.shape[:2]
  query = dense_general(inputs_q, params['query']['kernel'], dtype).reshape(
      b, ql, num_heads, head_dim)
  if projected_kv is not None:
    key, value = projected_kv
  else:
    kl = inputs_kv.shape[1]
    key = dense_general(inputs_kv, params['key']['kernel'], dtype).reshape(
        b, kl, num_heads, head_dim)
    value = dense_general(inputs_kv, params['value']['kernel'], dtype).reshape(
        b, kl, num_heads, head_dim)

  new_cache = None
  if decode:
    cached_key = np.asarray(cache['cached_key'])  # [b, h, d, L]
    cached_value = np.asarray(cache['cached_value'])
    length = cached_key.shape[-1]
    if query.shape != (b, 1, num_heads, head_dim):  # :250-256
      raise ValueError('Autoregressive cache shape error, expected query shape '
                       '%s instead got %s.' %
                       ((b, 1, num_heads, head_dim), query.shape))
    cur_index = np.asarray(cache['cache_index'])
    one_hot = cast((np.arange(length) == cur_index).astype(_F32), dtype)
    one_token_key = np.moveaxis(key, -3, -1)  # [b, h, d, 1]
    one_token_value = np.moveaxis(value, -3, -1)
    key = cast(cached_key + one_token_key * one_hot, dtype)  # :271-272
    value = cast(cached_value + one_token_value * one_hot, dtype)
    new_cache = {'cached_key': key, 'cached_value': value,
                 'cache_index': (cur_index + 1).astype(np.int32)}
    key = np.moveaxis(key, -1, -3)  # back to [b, L, h, d]
    value = np.moveaxis(value, -1, -3)
    mask = combine_masks(
        mask,
        np.broadcast_to(np.arange(length) <= cur_index, (b, 1, 1, length)))
    if bias is not None:  # :297-303 row `cur_index` of the bias matrix
      # lax.dynamic_slice_in_dim (:132-134) clamps a start beyond the last
      # row to the last row; jax.nn.one_hot above is all zeros there, so a
      # step past the end of the cache inserts nothing and attends to all of
      # it.  (No reference test goes there: parity unpinned for that case.)
      ci = min(max(int(cur_index), 0), bias.shape[2] - 1)
      bias = bias[:, :, ci:ci + 1, :]

  if mask is not None:  # :306-314
    attention_bias = np.where(mask > 0, cast(_F32(0.0), dtype),
                              cast(_F32(-1e10), dtype)).astype(_F32)
  else:
    attention_bias = None
  if bias is not None:  # :317-318
    attention_bias = (bias if attention_bias is None else cast(
        attention_bias + bias, dtype))

  x = dot_product_attention(query, key, value, attention_bias, dtype)
  out = dense_general(x.reshape(b, ql, num_heads * head_dim),
                      params['out']['kernel'], dtype)
  return out, new_cache


def mlp_block(params, x, activations, dtype: str):
  """t5x/examples/t5/layers.py:434-487."""
  acts = []
  for idx, name in enumerate(activations):
    dense_name = 'wi' if len(activations) == 1 else f'wi_{idx}'
    h = dense_general(x, params[dense_name]['kernel'], dtype)
    acts.append(cast(activation(name)(h), dtype))
  h = acts[0]
  for other in acts[1:]:
    h = cast(h * other, dtype)
  return dense_general(h, params['wo']['kernel'], dtype)


def embed(table, ids, dtype: str):
  """t5x/examples/t5/layers.py:520-541 (one-hot dot == exact row pick)."""
  ids = np.asarray(ids)
  if not np.issubdtype(ids.dtype, np.integer):
    raise ValueError('Input type must be an integer or unsigned integer.')
  return cast(table, dtype)[ids]


# ------------------------------------------------------------------------------
# network.py
# ------------------------------------------------------------------------------


def encoder_layer(p, cfg, inputs, encoder_mask, encoder_bias):
  """t5x/examples/t5/network.py:47-96."""
  A = cfg.dtype
  x = layer_norm(inputs, p['pre_attention_layer_norm']['scale'], A)
  x, _ = multi_head_attention(p['attention'], x, x, encoder_mask, encoder_bias,
                              num_heads=cfg.num_heads, head_dim=cfg.head_dim,
                              dtype=A)
  x = cast(x + inputs, A)
  y = layer_norm(x, p['pre_mlp_layer_norm']['scale'], A)
  y = mlp_block(p['mlp'], y, cfg.mlp_activations, A)
  return cast(y + x, A)


def encode(params, cfg: T5Config, encoder_input_tokens):
  """Transformer.encode + Encoder, t5x/examples/t5/network.py:182-219,315-343."""
  A = cfg.dtype
  tokens = np.asarray(encoder_input_tokens)
  encoder_mask = make_attention_mask(tokens > 0, tokens > 0)
  p = params['encoder']
  n = tokens.shape[-1]
  bias = relpos_bias(p['relpos_bias']['rel_embedding'], n, n, True, A)
  x = embed(params['token_embedder']['embedding'], tokens.astype(np.int32), A)
  for lyr in range(cfg.num_encoder_layers):
    x = encoder_layer(p[f'layers_{lyr}'], cfg, x, encoder_mask, bias)
  return layer_norm(x, p['encoder_norm']['scale'], A)


def decoder_layer(p, cfg, inputs, encoded, decoder_mask, encoder_decoder_mask,
                  decoder_bias, decode, cache, cross_kv):
  """t5x/examples/t5/network.py:99-179."""
  A = cfg.dtype
  kw = dict(num_heads=cfg.num_heads, head_dim=cfg.head_dim, dtype=A)
  x = layer_norm(inputs, p['pre_self_attention_layer_norm']['scale'], A)
  x, new_cache = multi_head_attention(
      p['self_attention'], x, x, decoder_mask, decoder_bias, decode=decode,
      cache=cache['self_attention'] if decode else None, **kw)
  x = cast(x + inputs, A)
  y = layer_norm(x, p['pre_cross_attention_layer_norm']['scale'], A)
  y, _ = multi_head_attention(p['encoder_decoder_attention'], y, encoded,
                              encoder_decoder_mask, None,
                              projected_kv=cross_kv, **kw)
  y = cast(y + x, A)
  z = layer_norm(y, p['pre_mlp_layer_norm']['scale'], A)
  z = mlp_block(p['mlp'], z, cfg.mlp_activations, A)
  z = cast(z + y, A)
  return z, ({'self_attention': new_cache} if decode else None)


def project_cross_kv(params, cfg: T5Config, encoded):
  """K/V that `encoder_decoder_attention` re-derives from `encoded` on every
  step (t5x/examples/t5/network.py:152-159 -> layers.py:216-217).  Returned
  per layer as ([b, E, h, d], [b, E, h, d])."""
  A = cfg.dtype
  out = []
  b, e = encoded.shape[:2]
  for lyr in range(cfg.num_decoder_layers):
    p = params['decoder'][f'layers_{lyr}']['encoder_decoder_attention']
    k = dense_general(encoded, p['key']['kernel'], A).reshape(
        b, e, cfg.num_heads, cfg.head_dim)
    v = dense_general(encoded, p['value']['kernel'], A).reshape(
        b, e, cfg.num_heads, cfg.head_dim)
    out.append((k, v))
  return out


def decode(params, cfg: T5Config, encoded, encoder_input_tokens,
           decoder_input_tokens, decoder_target_tokens, *, decode=False,
           cache=None, max_decode_length=None, cross_kv=None,
           return_hidden=False):
  """Transformer.decode + Decoder, t5x/examples/t5/network.py:222-292,345-409.

  Returns logits [b, len, V] float32, and the new cache when `decode`.
  """
  A = cfg.dtype
  enc_tokens = np.asarray(encoder_input_tokens)
  dec_in = np.asarray(decoder_input_tokens)
  dec_tgt = np.asarray(decoder_target_tokens)
  if decode:  # :362-370
    decoder_mask = None
    encoder_decoder_mask = make_attention_mask(np.ones_like(dec_tgt),
                                               enc_tokens > 0)
  else:  # :372-379
    decoder_mask = make_decoder_mask(dec_tgt)
    encoder_decoder_mask = make_attention_mask(dec_tgt > 0, enc_tokens > 0)

  p = params['decoder']
  y = embed(params['token_embedder']['embedding'], dec_in.astype(np.int32), A)
  l = max_decode_length if decode and max_decode_length else dec_in.shape[-1]
  decoder_bias = relpos_bias(p['relpos_bias']['rel_embedding'], l, l, False, A)
  new_cache = {'decoder': {}} if decode else None
  for lyr in range(cfg.num_decoder_layers):
    name = f'layers_{lyr}'
    y, c = decoder_layer(
        p[name], cfg, y, encoded, decoder_mask, encoder_decoder_mask,
        decoder_bias, decode, cache['decoder'][name] if decode else None,
        cross_kv[lyr] if cross_kv is not None else None)
    if decode:
      new_cache['decoder'][name] = c
  y = layer_norm(y, p['decoder_norm']['scale'], A)
  if return_hidden:
    return y
  if cfg.logits_via_embedding:  # :280-284
    emb = np.asarray(params['token_embedder']['embedding'], _F32)
    logits = (y @ emb.T) / np.sqrt(_F32(y.shape[-1]))
  else:  # :286-291 float32 dense
    logits = dense_general(y, p['logits_dense']['kernel'], 'float32')
  if decode:
    return logits.astype(_F32), new_cache
  return logits.astype(_F32)


def init_cache(cfg: T5Config, batch: int, max_decode_length: int):
  """Cache tree of t5x/examples/t5/layers.py:231-244 for every decoder layer."""
  def leaf():
    return {
        'cached_key': np.zeros(
            (batch, cfg.num_heads, cfg.head_dim, max_decode_length), _F32),
        'cached_value': np.zeros(
            (batch, cfg.num_heads, cfg.head_dim, max_decode_length), _F32),
        'cache_index': np.array(0, dtype=np.int32)}
  return {'decoder': {f'layers_{i}': {'self_attention': leaf()}
                      for i in range(cfg.num_decoder_layers)}}


# ------------------------------------------------------------------------------
# synthetic parameters shared with the HIP path
# ------------------------------------------------------------------------------


def init_params(cfg: T5Config, seed: int = 0, with_encoder: bool = True):
  """normal(0, 1/sqrt(fan_in)) float32 parameters from PCG64(seed), in the
  reference's parameter-tree layout (names: layers.py:403-410,512-518,651-657,
  697-699; shapes witnessed by t5x/testdata/test_t5_tiny.checkpoint_0)."""
  gen = np.random.Generator(np.random.PCG64(seed))
  d, hd, f = cfg.emb_dim, cfg.num_heads * cfg.head_dim, cfg.mlp_dim

  def w(k, n, fan_in=None):
    fan_in = fan_in or k
    return (gen.standard_normal((k, n), dtype=_F32) /
            _F32(np.sqrt(fan_in))).astype(_F32)

  def norm():
    return {'scale': (1.0 + 0.1 * gen.standard_normal((d,), dtype=_F32)
                     ).astype(_F32)}

  def attn():
    return {'query': {'kernel': w(d, hd) / _F32(np.sqrt(cfg.head_dim))},
            'key': {'kernel': w(d, hd)}, 'value': {'kernel': w(d, hd)},
            'out': {'kernel': w(hd, d)}}

  def mlp():
    return {'wi_0': {'kernel': w(d, f)}, 'wi_1': {'kernel': w(d, f)},
            'wo': {'kernel': w(f, d)}}

  params = {'token_embedder': {
      'embedding': gen.standard_normal((cfg.vocab_size, d), dtype=_F32)}}
  if with_encoder:
    enc = {'relpos_bias': {'rel_embedding': w(cfg.num_heads, 32, fan_in=1) *
                           _F32(0.5)},
           'encoder_norm': norm()}
    for i in range(cfg.num_encoder_layers):
      enc[f'layers_{i}'] = {'pre_attention_layer_norm': norm(),
                            'attention': attn(),
                            'pre_mlp_layer_norm': norm(), 'mlp': mlp()}
    params['encoder'] = enc
  dec = {'relpos_bias': {'rel_embedding': w(cfg.num_heads, 32, fan_in=1) *
                         _F32(0.5)},
         'decoder_norm': norm(), 'logits_dense': {'kernel': w(d,
                                                              cfg.vocab_size)}}
  for i in range(cfg.num_decoder_layers):
    dec[f'layers_{i}'] = {
        'pre_self_attention_layer_norm': norm(), 'self_attention': attn(),
        'pre_cross_attention_layer_norm': norm(),
        'encoder_decoder_attention': attn(),
        'pre_mlp_layer_norm': norm(), 'mlp': mlp()}
  params['decoder'] = dec
  return params


def quantize_int8(kernel):
  """Per-output-channel symmetric int8: scale = max|w| / 127 over the input
  axis, q = round(w / scale) clipped to [-127, 127]."""
  kernel = np.asarray(kernel, _F32)
  scale = np.maximum(np.max(np.abs(kernel), axis=0), _F32(1e-30)) / _F32(127.0)
  q = np.clip(np.rint(kernel / scale), -127, 127).astype(np.int8)
  return {'q': q, 'scale': scale.astype(_F32)}
