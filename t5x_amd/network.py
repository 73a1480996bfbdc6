"""T5.1.1 encoder-decoder behind a flax-like `module.apply`, with the decoder's
single-step (decode=True) forward running on the HIP kernels.

Mirrors t5x/examples/t5/network.py (Transformer.encode / decode, :295-409) and
the layers it uses (t5x/examples/t5/layers.py).  What runs where:
  * decode step (the hot path): embedding gather, RMS norms, all dense layers,
    cached self-attention, cross-attention and the float32 logits layer are
    t5d kernels; weights are cast/packed once per parameter tree;
  * once per batch, outside the step loop: the encoder forward and the
    projection of its output to per-layer cross-attention K/V use library
    GEMMs through torch (the reference recomputes that projection every step,
    network.py:152-159 — the values are identical).
"""

import dataclasses
from typing import Any, Mapping, Optional, Sequence

import numpy as np
import torch

from t5x_amd import ops


@dataclasses.dataclass(frozen=True)
class T5Config:
  """t5x/examples/t5/network.py:25-44."""
  vocab_size: int = 32128
  dtype: str = 'bfloat16'
  emb_dim: int = 512
  num_heads: int = 8
  num_encoder_layers: int = 6
  num_decoder_layers: int = 6
  head_dim: int = 64
  mlp_dim: int = 2048
  mlp_activations: Sequence[str] = ('gelu', 'linear')
  dropout_rate: float = 0.0
  logits_via_embedding: bool = False
  float32_attention_logits: bool = False
  # Not in the reference config: storage type of the dense kernels on the
  # decode path ('int8' = weight-only, per-output-channel symmetric scales).
  weight_dtype: Optional[str] = None


# t5x/examples/t5/t5_1_1/{small,base,large,xl,xxl}.gin
T5_1_1 = {
    'small': dict(emb_dim=512, num_heads=6, num_encoder_layers=8,
                  num_decoder_layers=8, head_dim=64, mlp_dim=1024),
    'base': dict(emb_dim=768, num_heads=12, num_encoder_layers=12,
                 num_decoder_layers=12, head_dim=64, mlp_dim=2048),
    'large': dict(emb_dim=1024, num_heads=16, num_encoder_layers=24,
                  num_decoder_layers=24, head_dim=64, mlp_dim=2816),
    'xl': dict(emb_dim=2048, num_heads=32, num_encoder_layers=24,
               num_decoder_layers=24, head_dim=64, mlp_dim=5120),
    'xxl': dict(emb_dim=4096, num_heads=64, num_encoder_layers=24,
                num_decoder_layers=24, head_dim=64, mlp_dim=10240),
}


def t5_1_1_config(size: str, **overrides) -> T5Config:
  kw = dict(T5_1_1[size])
  kw.update(overrides)
  return T5Config(**kw)


_TORCH_DTYPE = {'float32': torch.float32, 'bfloat16': torch.bfloat16,
                'int8': torch.int8}


def relative_position_bucket(relative_position, bidirectional=True,
                             num_buckets=32, max_distance=128):
  """t5x/examples/t5/layers.py:580-625 (host-side NumPy, as in the
  reference)."""
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


class BeamShared:
  """An array that is logically `flat_batch_beam_expand(x, beams)` but stored
  once per batch item.  `EncoderDecoderModel.predict_batch_with_aux` hands the
  encoder output to the decode step this way so cross-attention K/V are
  projected and streamed once per item instead of once per beam."""

  def __init__(self, x, beams: int):
    self.x, self.beams = x, int(beams)

  @property
  def shape(self):
    return (self.x.shape[0] * self.beams,) + tuple(self.x.shape[1:])


def _leaf(tree, *path):
  for p in path:
    tree = tree[p]
  return tree


def _f32(x, device):
  if isinstance(x, torch.Tensor):
    return x.to(device=device, dtype=torch.float32).contiguous()
  return torch.as_tensor(np.asarray(x, dtype=np.float32), device=device)


class DecoderWeights:
  """Decode-path parameters, cast and packed once on the device.

  Parameter names follow the reference tree (t5x/examples/t5/layers.py:403-410,
  512-518,651-657,697-699): params['decoder']['layers_i'][...]['kernel'] etc.
  """

  def __init__(self, cfg: T5Config, params, device):
    act = _TORCH_DTYPE[cfg.dtype]
    wdt = _TORCH_DTYPE[cfg.weight_dtype or cfg.dtype]
    self.act_dtype = act
    dec = params['decoder']
    g = lambda *p: _f32(_leaf(dec, *p), device)
    self.embedding = _f32(params['token_embedder']['embedding'],
                          device).to(act).contiguous()
    self.rel_embedding = g('relpos_bias', 'rel_embedding')  # [H, 32] f32
    self.layers = []
    for i in range(cfg.num_decoder_layers):
      n = f'layers_{i}'
      sa, ca, mlp = 'self_attention', 'encoder_decoder_attention', 'mlp'
      qkv = torch.cat([g(n, sa, 'query', 'kernel'), g(n, sa, 'key', 'kernel'),
                       g(n, sa, 'value', 'kernel')], dim=1).contiguous()
      layer = dict(
          ln_self=g(n, 'pre_self_attention_layer_norm', 'scale').to(act),
          qkv=ops.pack_weight(qkv, act, wdt),
          self_out=ops.pack_weight(g(n, sa, 'out', 'kernel'), act, wdt),
          ln_cross=g(n, 'pre_cross_attention_layer_norm', 'scale').to(act),
          cross_q=ops.pack_weight(g(n, ca, 'query', 'kernel'), act, wdt),
          cross_out=ops.pack_weight(g(n, ca, 'out', 'kernel'), act, wdt),
          ln_mlp=g(n, 'pre_mlp_layer_norm', 'scale').to(act),
          wi=ops.pack_weight(g(n, mlp, 'wi_0', 'kernel'), act, wdt,
                             gate_kernel=g(n, mlp, 'wi_1', 'kernel')),
          wo=ops.pack_weight(g(n, mlp, 'wo', 'kernel'), act, wdt),
          # once-per-batch cross K/V projection (library GEMM)
          cross_k=self._dense_for_library(g(n, ca, 'key', 'kernel'), act, wdt),
          cross_v=self._dense_for_library(g(n, ca, 'value', 'kernel'), act,
                                          wdt),
      )
      self.layers.append(layer)
    self.ln_final = g('decoder_norm', 'scale').to(act)
    # Logits layer: float32 in the reference; bf16 configs stream it as bf16
    # (or int8) with float32 accumulation and float32 output.
    self.logits = ops.pack_weight(g('logits_dense', 'kernel'), act, wdt)
    self._rel_bias = {}

  @staticmethod
  def _dense_for_library(kernel, act, wdt):
    if wdt == torch.int8:
      scale = kernel.abs().amax(dim=0).clamp_min(1e-30) / 127.0
      q = torch.clamp(torch.round(kernel / scale), -127, 127)
      return (q.to(act), scale.to(torch.float32))
    return (kernel.to(act), None)

  def rel_bias(self, length: int):
    """[H, L] table: bias for distance n = query_pos - key_pos >= 0
    (RelativePositionBiases with bidirectional=False, layers.py:627-677)."""
    if length not in self._rel_bias:
      bucket = relative_position_bucket(-np.arange(length),
                                        bidirectional=False)
      idx = torch.as_tensor(bucket.astype(np.int64),
                            device=self.rel_embedding.device)
      self._rel_bias[length] = self.rel_embedding.to(
          self.act_dtype)[:, idx].contiguous()
    return self._rel_bias[length]

  def nbytes_per_step(self):
    """Weight bytes one decode step streams."""
    n = 0
    for l in self.layers:
      for k in ('qkv', 'self_out', 'cross_q', 'cross_out', 'wi', 'wo'):
        n += l[k].nbytes()
    return n + self.logits.nbytes()


class _StepBuffers:
  """Activations of one decode step for R rows."""

  def __init__(self, cfg: T5Config, R, device, act):
    d, hd, f = cfg.emb_dim, cfg.num_heads * cfg.head_dim, cfg.mlp_dim
    e = lambda *s: torch.empty(s, dtype=act, device=device)
    self.ids = torch.empty((R,), dtype=torch.int32, device=device)
    self.x, self.x1, self.x2 = e(R, d), e(R, d), e(R, d)
    self.xn = e(R, d)
    self.qkv = e(R, 3 * hd)
    self.q = e(R, hd)
    self.ao = e(R, hd)
    self.h = e(R, f)
    self.logits = torch.empty((R, cfg.vocab_size), dtype=torch.float32,
                              device=device)


class Transformer:
  """network.Transformer with `apply(variables, *args, method=..., **kwargs)`.

  `variables['params']` is the reference parameter tree (NumPy or torch
  float32 leaves); it is cast/packed on first use and cached by identity.
  """

  scan_layers = False

  def __init__(self, config: T5Config, device=None):
    if config.head_dim != 64:
      raise ValueError('the attention kernels are specialised for head_dim 64')
    if tuple(config.mlp_activations) != ('gelu', 'linear'):
      raise ValueError('the MLP kernel implements T5.1.1 gated-GELU only')
    if config.logits_via_embedding:
      raise ValueError('T5.1.1 uses a separate logits layer')
    self.config = config
    self.dtype = config.dtype
    self.device = device
    self._weights = {}
    self._enc_weights = {}
    self._bufs = {}
    self._cross = None

  # -- plumbing ---------------------------------------------------------------
  def _dev(self):
    if self.device is None:
      if not torch.cuda.is_available():
        raise RuntimeError('t5x_amd needs a GPU (no CPU fallback)')
      self.device = torch.device('cuda')
    return self.device

  def decoder_weights(self, params) -> DecoderWeights:
    key = id(params)
    if key not in self._weights:
      self._weights[key] = (params, DecoderWeights(self.config, params,
                                                   self._dev()))
    return self._weights[key][1]

  def apply(self, variables, *args, method=None, mutable=False, **kwargs):
    name = 'call' if method is None else method.__name__
    return getattr(self, '_' + name)(variables, *args, mutable=mutable,
                                     **kwargs)

  def encode(self, *a, **k):
    raise TypeError('call through apply(..., method=module.encode)')

  def decode(self, *a, **k):
    raise TypeError('call through apply(..., method=module.decode)')

  # -- encoder (once per batch; library GEMMs) ----------------------------------
  def _encode(self, variables, encoder_input_tokens, encoder_segment_ids=None,
              enable_dropout=False, mutable=False):
    del encoder_segment_ids, enable_dropout, mutable
    from t5x_amd import encoder
    return encoder.encode(self, variables['params'], encoder_input_tokens)

  # -- cache --------------------------------------------------------------------
  def init_cache(self, batch: int, max_decode_length: int):
    """Zero cache tree of t5x/examples/t5/layers.py:231-244.  All layers' K/V
    live in one allocation [layers, 2, batch, H, 64, L] and all cache_index
    leaves in one int32 vector, so whole-model kernels can address them with
    a stride."""
    cfg, dev = self.config, self._dev()
    act = _TORCH_DTYPE[cfg.dtype]
    # Rows are read in 16-byte chunks: a length that is not a multiple of 8
    # (bf16) / 4 (f32) positions is padded up; the extra columns are never
    # attended to (they lie beyond every cache_index).
    el = 16 // torch.empty((), dtype=act).element_size()
    length = (max_decode_length + el - 1) // el * el
    kv = torch.zeros((cfg.num_decoder_layers, 2, batch, cfg.num_heads,
                      cfg.head_dim, length), dtype=act, device=dev)
    idx = torch.zeros((cfg.num_decoder_layers,), dtype=torch.int32, device=dev)
    return {'decoder': {
        f'layers_{i}': {'self_attention': {
            'cached_key': kv[i, 0], 'cached_value': kv[i, 1],
            'cache_index': idx[i]}}
        for i in range(cfg.num_decoder_layers)}}

  def _call(self, variables, encoder_input_tokens, decoder_input_tokens,
            decoder_target_tokens, enable_dropout=False, decode=False,
            mutable=False):
    if decode and 'cache' not in variables:
      # cache initialisation pass (t5x/models.py:542-552): shapes only
      b, l = decoder_input_tokens.shape
      return None, {'cache': self.init_cache(b, l)}
    raise NotImplementedError(
        'only the inference entry points (encode / decode(decode=True) / cache '
        'initialisation) are implemented')

  # -- cross-attention K/V, once per batch ---------------------------------------
  def _cross_kv(self, w: DecoderWeights, encoded, enc_tokens, beams):
    key = (encoded.data_ptr(), tuple(encoded.shape), enc_tokens.data_ptr(),
           id(w), encoded._version)
    if self._cross is not None and self._cross[0] == key:
      return self._cross[1]
    cfg = self.config
    B, E, d = encoded.shape
    H, D = cfg.num_heads, cfg.head_dim
    el = 16 // encoded.element_size()
    Ep = (E + el - 1) // el * el  # rows padded to 16-byte multiples
    x = encoded.reshape(B * E, d)
    ks, vs = [], []
    for l in w.layers:
      for (kern, scale), dst in ((l['cross_k'], ks), (l['cross_v'], vs)):
        y = torch.matmul(x, kern)  # float32 accumulate, one rounding
        if scale is not None:
          y = (torch.matmul(x.float(), kern.float()) * scale).to(x.dtype)
        y = y.view(B, E, H, D).permute(0, 2, 3, 1)  # [B, H, D, E]
        buf = torch.zeros((B, H, D, Ep), dtype=x.dtype, device=x.device)
        buf[..., :E] = y
        dst.append(buf)
    tok = enc_tokens.reshape(B, E)
    valid = tok > 0
    # The mask keeps exactly the positions with token > 0 (network.py:366-370).
    # The kernel takes a prefix length; inputs are right-padded.
    lens = valid.sum(dim=1).to(torch.int32)
    prefix = (torch.arange(E, device=tok.device)[None, :] <
              lens[:, None])
    if not bool((prefix == valid).all()):
      raise ValueError('encoder padding must be a suffix of zeros')
    out = dict(k=ks, v=vs, enc_len=lens.contiguous(), B=B, beams=beams, E=Ep)
    self._cross = (key, out, encoded)
    return out

  # -- the decode step -------------------------------------------------------------
  def _decode(self, variables, encoded, encoder_input_tokens,
              decoder_input_tokens, decoder_target_tokens,
              enable_dropout=False, decode=False, max_decode_length=None,
              mutable=False):
    del decoder_target_tokens, enable_dropout
    if not decode:
      raise NotImplementedError('only decode=True (single-step) is implemented')
    cfg, dev = self.config, self._dev()
    w = self.decoder_weights(variables['params'])
    cache = variables['cache']
    if isinstance(encoded, BeamShared):
      beams, enc = encoded.beams, encoded.x
      enc_tok = encoder_input_tokens.x
    else:
      beams, enc, enc_tok = 1, encoded, encoder_input_tokens
    enc_tok = torch.as_tensor(np.asarray(enc_tok), device=dev) if not isinstance(
        enc_tok, torch.Tensor) else enc_tok.to(dev)
    cross = self._cross_kv(w, enc, enc_tok, beams)
    ids = decoder_input_tokens
    if not isinstance(ids, torch.Tensor):
      ids = torch.as_tensor(np.asarray(ids), device=dev)
    R = ids.shape[0]
    if ids.dim() != 2 or ids.shape[1] != 1:
      raise ValueError('Autoregressive cache shape error, expected query shape '
                       '%s instead got %s.' % ((R, 1), tuple(ids.shape)))
    if R != cross['B'] * beams:
      raise ValueError(f'{R} decoder rows vs {cross["B"]} x {beams} encoder rows')
    key = (R,)
    if key not in self._bufs:
      self._bufs[key] = _StepBuffers(cfg, R, dev, w.act_dtype)
    b = self._bufs[key]
    b.ids.copy_(ids.reshape(R).to(torch.int32))

    ops.embed(w.embedding, b.ids, b.x)
    x = b.x
    index_leaves = []
    for i, lw in enumerate(w.layers):
      c = cache['decoder'][f'layers_{i}']['self_attention']
      ck, cv, ci = c['cached_key'], c['cached_value'], c['cache_index']
      L = ck.shape[-1]
      if max_decode_length and L < max_decode_length:
        raise ValueError(f'cache length {L} < max_decode_length '
                         f'{max_decode_length}')
      index_leaves.append(ci)
      ops.rmsnorm(x, lw['ln_self'], b.xn)
      ops.gemm(b.xn, lw['qkv'], b.qkv)
      ops.self_attention_step(b.qkv, ck, cv, w.rel_bias(L), ci, b.ao)
      ops.gemm(b.ao, lw['self_out'], b.x1, residual=x)
      ops.rmsnorm(b.x1, lw['ln_cross'], b.xn)
      ops.gemm(b.xn, lw['cross_q'], b.q)
      ops.cross_attention_step(b.q, cross['k'][i], cross['v'][i],
                               cross['enc_len'], beams, b.ao)
      ops.gemm(b.ao, lw['cross_out'], b.x2, residual=b.x1)
      ops.rmsnorm(b.x2, lw['ln_mlp'], b.xn)
      ops.gemm(b.xn, lw['wi'], b.h)
      ops.gemm(b.h, lw['wo'], b.x, residual=b.x2)
      x = b.x
    ops.rmsnorm(x, w.ln_final, b.xn)
    ops.gemm(b.xn, w.logits, b.logits, out_dtype=torch.float32)
    # cache_index += 1 for every layer (layers.py:275): one launch when the
    # leaves are consecutive elements of one vector.
    first = index_leaves[0]
    contiguous = all(
        ci.data_ptr() == first.data_ptr() + 4 * j
        for j, ci in enumerate(index_leaves))
    if contiguous:
      base = first.as_strided((len(index_leaves),), (1,))
      ops.add_i32(base, 1)
    else:
      for ci in index_leaves:
        ops.add_i32(ci, 1)
    logits = b.logits.view(R, 1, cfg.vocab_size)
    return (logits, {'cache': cache}) if mutable else logits


def init_params(cfg: T5Config, seed: int = 0, device=None,
                with_encoder: bool = True):
  """Synthetic random-init parameters in the reference tree layout, generated
  on the device: every dense kernel normal(0, 1/sqrt(fan_in)) (query kernels
  additionally / sqrt(head_dim), as the reference initialiser does,
  t5x/examples/t5/layers.py:207-211), embedding normal(0, 1), norm scales
  1 + 0.1 normal, relative-position table 0.5 normal."""
  device = device or torch.device('cuda')
  gen = torch.Generator(device=device)
  gen.manual_seed(seed)
  d, hd, f = cfg.emb_dim, cfg.num_heads * cfg.head_dim, cfg.mlp_dim

  def w(k, n, scale=None):
    t = torch.randn((k, n), generator=gen, device=device, dtype=torch.float32)
    return t * (scale if scale is not None else 1.0 / np.sqrt(k))

  def norm():
    return {'scale': 1.0 + 0.1 * torch.randn((d,), generator=gen,
                                             device=device)}

  def attn():
    return {'query': {'kernel': w(d, hd) / np.sqrt(cfg.head_dim)},
            'key': {'kernel': w(d, hd)}, 'value': {'kernel': w(d, hd)},
            'out': {'kernel': w(hd, d)}}

  def mlp():
    return {'wi_0': {'kernel': w(d, f)}, 'wi_1': {'kernel': w(d, f)},
            'wo': {'kernel': w(f, d)}}

  params = {'token_embedder': {'embedding': w(cfg.vocab_size, d, 1.0)}}
  if with_encoder:
    enc = {'relpos_bias': {'rel_embedding': w(cfg.num_heads, 32, 0.5)},
           'encoder_norm': norm()}
    for i in range(cfg.num_encoder_layers):
      enc[f'layers_{i}'] = {'pre_attention_layer_norm': norm(),
                            'attention': attn(), 'pre_mlp_layer_norm': norm(),
                            'mlp': mlp()}
    params['encoder'] = enc
  dec = {'relpos_bias': {'rel_embedding': w(cfg.num_heads, 32, 0.5)},
         'decoder_norm': norm(),
         'logits_dense': {'kernel': w(d, cfg.vocab_size)}}
  for i in range(cfg.num_decoder_layers):
    dec[f'layers_{i}'] = {
        'pre_self_attention_layer_norm': norm(), 'self_attention': attn(),
        'pre_cross_attention_layer_norm': norm(),
        'encoder_decoder_attention': attn(),
        'pre_mlp_layer_norm': norm(), 'mlp': mlp()}
  params['decoder'] = dec
  return params
