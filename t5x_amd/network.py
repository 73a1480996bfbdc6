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
import weakref
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


def cache_tree(keys, values, index, scanned: bool):
  """The cache tree of t5x/examples/t5/layers.py:231-244 over per-layer K/V
  `keys[i]` / `values[i]` [rows, H, 64, L] and the int32 vector `index`
  [layers]: one scope per layer, or (scanned) one 'decoder' scope with the
  layer axis leading (t5x/examples/scalable_t5/network.py:324-352)."""
  if scanned:
    return {'decoder': {'decoder': {'self_attention': {
        'cached_key': keys, 'cached_value': values, 'cache_index': index}}}}
  return {'decoder': {
      f'layers_{i}': {'self_attention': {
          'cached_key': keys[i], 'cached_value': values[i],
          'cache_index': index[i]}} for i in range(index.shape[0])}}


class FreshCache(dict):
  """The zero cache as returned by cache initialisation.  While `fresh` is set
  a decode loop that owns its (beam-expanded) caches may skip expanding this
  one and start from zero caches of its own; the first decode step that writes
  into the tree clears the flag, and any tree derived from it through
  cache_map is a plain dict."""

  def __init__(self, *args, **kw):
    super().__init__(*args, **kw)
    self.fresh = True


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
          # once-per-batch cross K/V projection (t5d_gemm_rows / t5d_gemm)
          cross_k_packed=ops.pack_weight(g(n, ca, 'key', 'kernel'), act, wdt),
          cross_v_packed=ops.pack_weight(g(n, ca, 'value', 'kernel'), act,
                                         wdt),
      )
      self.layers.append(layer)
    self.ln_final = g('decoder_norm', 'scale').to(act)
    # Logits layer: float32 in the reference; bf16 configs stream it as bf16
    # (or int8) with float32 accumulation and float32 output.
    self.logits = ops.pack_weight(g('logits_dense', 'kernel'), act, wdt)
    self._rel_bias = {}

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


# device index -> the decode streams of that device (Transformer.decode_stream)
_DECODE_STREAMS = {}
# device index -> how many of them (the first n) were measured to run side by
# side, or None where that could not be measured
_DECODE_STREAMS_SIDE_BY_SIDE = {}


def _measure_side_by_side(streams):
  """The largest n for which busy kernels on the first n streams overlap: n
  kernels of about half a millisecond, one per stream, must finish in less
  than 1.5 times what one takes (the shortest of three runs each; on a busy
  device a single run can read long).  The whole measurement is taken twice;
  None when the two disagree or when there is no busy kernel to use: the
  caller then goes by the number of hardware queues instead."""
  import time
  sleep = getattr(torch.cuda, '_sleep', None)
  if sleep is None:
    return None

  def timed(group, cycles):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for stream in group:
      with torch.cuda.stream(stream):
        sleep(cycles)
    for stream in group:
      stream.synchronize()
    return time.perf_counter() - t0

  cycles = 100_000
  one = timed(streams[:1], cycles)
  for _ in range(8):  # the unit of `cycles` is the device's business
    if one >= 4e-4:
      break
    cycles *= 4
    one = timed(streams[:1], cycles)
  if one < 4e-4:
    return None

  def count():
    alone = min(timed(streams[:1], cycles) for _ in range(3))
    n = 1
    while n < len(streams):
      together = min(timed(streams[:n + 1], cycles) for _ in range(3))
      if together > 1.5 * alone:
        break
      n += 1
    return n

  first, second = count(), count()
  return first if first == second else None


def decode_cache_layout(act_dtype, beams, length):
  """The layout a decode loop keeps the self-attention caches it owns in, as
  t5d_self_attention_step_gather names them, and the cache length to use.
  bfloat16 caches are kept for the loop's access pattern — 3: keys by
  position, values in finished blocks of 32 positions plus a position-major
  tail, so that the column a step appends is two full cache lines instead of
  128 two-byte stores into 128 lines (the kernels cover 256 positions);
  2: keys and values in blocks of 32 positions, for longer caches — and
  converted back by cache_tree().
  float32 caches stay in the reference layout (0)."""
  if act_dtype != torch.bfloat16:
    return 0, (length + 3) // 4 * 4
  L = (length + 31) // 32 * 32
  if beams <= 8 and L <= 256:
    return 3, L
  return 2, L


def _plain_caches(kv, layout, n):
  """[2, R, H, 64, L(+32)] keys and values of one layer in `layout`, holding n
  positions -> the pair in the reference layout [R, H, 64, L]."""
  from t5x_amd import ops
  if layout == 3:
    return (ops.untail_cached_key(kv[0].reshape(*kv.shape[1:3], -1, 64)),
            ops.untail_cached_value(kv[1], n))
  if layout == 2:
    return ops.unblock_cached_value(kv[0]), ops.unblock_cached_value(kv[1])
  return kv[0], kv[1]


class Transformer:
  """network.Transformer with `apply(variables, *args, method=..., **kwargs)`.

  `variables['params']` is the reference parameter tree (NumPy or torch
  float32 leaves); it is cast/packed on first use and cached by identity.
  """

  # Batch slices ("lanes") that a fused beam search steps on separate streams.
  # A decode step is a chain of dependent kernels that leaves most of the
  # device waiting, so two half-batches side by side finish an iteration
  # sooner than the whole batch in one chain (measured: base beam 4
  # 0.789 -> 0.738 ms, XL int8 2.61 -> 2.46 ms; three lanes are slower
  # again, and a fourth stream shares a hardware queue).  None: 2 lanes for a
  # decode on its own, 1 when several batches are in flight (those fill the
  # device better than lanes do, and streams that run side by side are few).
  decode_lanes = None

  # How many decode streams the device runs side by side.  None: the
  # environment variable T5X_AMD_STREAMS_SIDE_BY_SIDE if set, else measured
  # once per device and process (streams_side_by_side).  A fixed value makes
  # the number of batch lanes and of batches in flight, hence what is
  # captured and held, the same in every run; results never depend on it.
  side_by_side = None

  def __init__(self, config: T5Config, device=None, scan_layers: bool = False):
    """scan_layers: hand out and accept the cache in the layout of a scanned
    decoder stack (t5x/examples/scalable_t5/network.py:324-352): one 'decoder'
    scope whose leaves carry a leading layer axis, [layers, rows, H, 64, L] and
    cache_index [layers]; EncoderDecoderModel then decodes with
    cache_offset=1 (t5x/models.py:739-748).  The parameter tree and the layer
    arithmetic are the same."""
    self.scan_layers = bool(scan_layers)
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
    self._step_cache = None
    self._beam_ctx = {}

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
    nl = cfg.num_decoder_layers
    idx = torch.zeros((nl,), dtype=torch.int32, device=dev)
    if self.scan_layers:
      kv = torch.zeros((2, nl, batch, cfg.num_heads, cfg.head_dim, length),
                       dtype=act, device=dev)
      return FreshCache(cache_tree(kv[0], kv[1], idx, True))
    kv = torch.zeros((nl, 2, batch, cfg.num_heads, cfg.head_dim, length),
                     dtype=act, device=dev)
    return FreshCache(cache_tree(kv[:, 0], kv[:, 1], idx, False))

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
  def _cross_kv(self, w: DecoderWeights, encoded, enc_tokens, beams, out=None):
    """Projects the encoder output to every decoder layer's cross-attention
    K/V, once per batch.  `out`: a result of an earlier call with the same
    shapes whose tensors are to be (re)used — a decode context that has their
    addresses recorded in a captured graph passes its own."""
    key = (encoded.data_ptr(), tuple(encoded.shape), enc_tokens.data_ptr(),
           id(w), encoded._version)
    if self._cross is not None and self._cross[0] == key:
      res = self._cross[1]
      if out is None or res is out:
        return res
      for dst, src in zip(out['k'] + out['v'], res['k'] + res['v']):
        dst.copy_(src)
      out['enc_len'].copy_(res['enc_len'])
      if out.get('units') is not None:
        out['units'].copy_(res['units'])
      self._cross = (key, out, encoded)
      return out
    cfg = self.config
    B, E, d = encoded.shape
    H, D = cfg.num_heads, cfg.head_dim
    bf16 = encoded.dtype == torch.bfloat16
    # float32: [B, H, Ep, 64] / [B, H, 64, Ep], rows padded to 16 bytes;
    # bfloat16: [B, H, 2, Ep, 32] / [B, H, Ep/32, 64, 32] (blocks of 32
    # positions).  Padding positions e >= E stay zero.
    pad = 32 if bf16 else 16 // encoded.element_size()
    Ep = (E + pad - 1) // pad * pad
    if out is not None and (out['B'], out['E']) != (B, Ep):
      raise ValueError('cross K/V buffers of another shape')
    # The mask keeps exactly the keys whose token is > 0 (network.py:366-370).
    # Keys and values of a position depend on that position alone and
    # cross-attention has no position term, so masking a key equals leaving
    # it out: the kernels take a count of valid keys per item, and where the
    # padding is not a suffix of zeros (a padding token inside the text) the
    # valid positions' encoder outputs are moved to the front first, in order.
    tok = enc_tokens.reshape(B, E)
    valid = tok > 0
    lens = valid.sum(dim=1).to(torch.int32)
    prefix = torch.arange(E, device=tok.device)[None, :] < lens[:, None]
    if not bool((prefix == valid).all()):
      order = torch.sort((~valid).to(torch.int8), dim=1, stable=True).indices
      x = torch.gather(encoded, 1, order[:, :, None].expand(B, E, d))
    else:
      x = encoded
    x = x.reshape(B * E, d).contiguous()
    ks, vs = [], []
    hip = bf16 and E % 4 == 0
    for i, l in enumerate(w.layers):
      if hip:
        # straight from the dense kernel's epilogue
        from t5x_amd import _lib
        ks.append(ops.gemm_rows(x, l['cross_k_packed'],
                                out=out['k'][i] if out else None,
                                layout=_lib.OUT_HEADS_KEY, E=E, Ep=Ep))
        vs.append(ops.gemm_rows(x, l['cross_v_packed'],
                                out=out['v'][i] if out else None,
                                layout=_lib.OUT_HEADS_VALUE, E=E, Ep=Ep))
        continue
      # float32, or an encoder length the head-layout epilogue does not take:
      # rows from the dense kernel, brought into the head layouts by copies
      for packed, dst in ((l['cross_k_packed'], ks), (l['cross_v_packed'], vs)):
        y = (ops.gemm_rows(x, packed) if bf16 else ops.gemm(x, packed))
        y = y.view(B, E, H, D)
        if dst is ks:  # keys: [B, H, E, D], head dim contiguous
          buf = torch.zeros((B, H, Ep, D), dtype=x.dtype, device=x.device)
          buf[:, :, :E] = y.permute(0, 2, 1, 3)
          buf = ops.tile_cross_key(buf) if bf16 else buf
        else:  # values: [B, H, D, E], positions contiguous
          buf = torch.zeros((B, H, D, Ep), dtype=x.dtype, device=x.device)
          buf[..., :E] = y.permute(0, 2, 3, 1)
          buf = ops.tile_cross_value(buf) if bf16 else buf
        if out is not None:
          buf = (out['k'] if dst is ks else out['v'])[i].copy_(buf)
        dst.append(buf)
    if out is not None:
      out['enc_len'].copy_(lens)
      res = out
    else:
      res = dict(k=ks, v=vs, enc_len=lens.contiguous(), B=B, beams=beams,
                 E=Ep, units=None)
    # The order in which the cross-attention workgroups take the (item, head)
    # pairs, chosen from the valid lengths so that the CUs are evenly loaded.
    if bf16 and B <= 256 and H <= 256:
      res['units'] = ops.cross_attention_units(res['enc_len'], H, Ep,
                                               out=res.get('units'))
    self._cross = (key, res, encoded)
    return res

  # -- the decode step -------------------------------------------------------------
  def _model_step(self, w, cross, bufs, layer_caches, cache_index, R, beams,
                  L, gate=None, pending_src=None, cache_layout=0,
                  pending_dst=None):
    """Fills a t5d_model_step for one call of t5d_decoder_step."""
    from t5x_amd import _lib
    cfg = self.config
    P = _lib.ptr
    layers = (_lib.Layer * cfg.num_decoder_layers)()
    for i, lw in enumerate(w.layers):
      ck, cv = layer_caches[i]
      l = layers[i]
      l.ln_self, l.ln_cross, l.ln_mlp = (P(lw['ln_self']), P(lw['ln_cross']),
                                         P(lw['ln_mlp']))
      for name in ('qkv', 'self_out', 'cross_q', 'cross_out', 'wi', 'wo'):
        setattr(l, name, P(lw[name].data))
        setattr(l, name + '_scales', P(lw[name].scales))
      l.cached_key, l.cached_value = P(ck), P(cv)
      l.cross_key, l.cross_value = P(cross['k'][i]), P(cross['v'][i])
    m = _lib.ModelStep()
    m.dtype = _lib.dtype_code(w.act_dtype)
    m.w_dtype = w.layers[0]['qkv'].w_dtype
    m.d, m.H, m.F, m.V = (cfg.emb_dim, cfg.num_heads, cfg.mlp_dim,
                          cfg.vocab_size)
    m.L, m.E, m.NL = L, cross['E'], cfg.num_decoder_layers
    m.R, m.B, m.beams = R, cross['B'], beams
    m.embedding, m.rel_bias = P(w.embedding), P(w.rel_bias(L))
    m.ln_final, m.logits_w = P(w.ln_final), P(w.logits.data)
    m.logits_scales = P(w.logits.scales)
    m.layers = layers
    m.cache_index, m.enc_len = P(cache_index), P(cross['enc_len'])
    m.cross_units = P(cross.get('units'))
    for name in ('x', 'x1', 'x2', 'xn', 'qkv', 'q', 'ao', 'h', 'logits'):
      setattr(m, name, P(getattr(bufs, name)))
    m.gate = P(gate)
    m.pending_src, m.pending_dst = P(pending_src), P(pending_dst)
    # 0: the reference layout; 2: keys and values in blocks of 32 positions;
    # 3: the decode loops' own layout (decode_cache_layout)
    m.value_blocked = int(cache_layout)
    m._keepalive = (layers, w, cross, bufs, layer_caches, cache_index, gate,
                    pending_src, pending_dst)
    return m

  def _step_buffers(self, R, w):
    if R not in self._bufs:
      self._bufs[R] = _StepBuffers(self.config, R, self._dev(), w.act_dtype)
    return self._bufs[R]

  def _decode(self, variables, encoded, encoder_input_tokens,
              decoder_input_tokens, decoder_target_tokens,
              enable_dropout=False, decode=False, max_decode_length=None,
              mutable=False):
    del decoder_target_tokens, enable_dropout
    if not decode:
      raise NotImplementedError('only decode=True (single-step) is implemented')
    from t5x_amd import _lib
    cfg, dev = self.config, self._dev()
    w = self.decoder_weights(variables['params'])
    cache = variables['cache']
    if getattr(cache, 'fresh', False):
      cache.fresh = False  # this step writes into it
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
    b = self._step_buffers(R, w)
    b.ids.copy_(ids.reshape(R).to(torch.int32))

    layer_caches, index_leaves = [], []
    scanned = 'decoder' in cache['decoder']
    if scanned != self.scan_layers:
      raise ValueError('cache tree layout (scanned layers or one scope per '
                       'layer) does not match this module')
    for i in range(cfg.num_decoder_layers):
      if scanned:
        c = cache['decoder']['decoder']['self_attention']
        c = {k: v[i] for k, v in c.items()}
      else:
        c = cache['decoder'][f'layers_{i}']['self_attention']
      ck, cv = c['cached_key'], c['cached_value']
      for t in (ck, cv):
        if (not t.is_contiguous() or t.dtype != w.act_dtype or
            tuple(t.shape[:3]) != (R, cfg.num_heads, cfg.head_dim)):
          raise ValueError(f'cache leaf of layer {i}: shape {tuple(t.shape)} '
                           f'dtype {t.dtype} contiguous={t.is_contiguous()}')
      layer_caches.append((ck, cv))
      index_leaves.append(c['cache_index'])
    L = layer_caches[0][0].shape[-1]
    if max_decode_length and L < max_decode_length:
      raise ValueError(f'cache length {L} < max_decode_length '
                       f'{max_decode_length}')
    # cache_index leaves are consecutive elements of one int32 vector when the
    # tree came from init_cache; otherwise gather them into one.
    first = index_leaves[0]
    consecutive = all(ci.dtype == torch.int32 and ci.is_cuda and
                      ci.data_ptr() == first.data_ptr() + 4 * j
                      for j, ci in enumerate(index_leaves))
    if consecutive:
      index_vec = first.as_strided((len(index_leaves),), (1,))
    else:
      index_vec = torch.stack([ci.reshape(()).to(dev, torch.int32)
                               for ci in index_leaves])
    key = (id(w), R, beams, L, layer_caches[0][0].data_ptr(),
           layer_caches[-1][1].data_ptr(), index_vec.data_ptr(),
           cross['k'][0].data_ptr())
    if self._step_cache is None or self._step_cache[0] != key:
      self._step_cache = (key, self._model_step(w, cross, b, layer_caches,
                                                index_vec, R, beams, L))
    m = self._step_cache[1]
    _lib.call('t5d_decoder_step', _lib.stream_handle(), m, b.ids.data_ptr())
    if not consecutive:
      if scanned:
        cache['decoder']['decoder']['self_attention']['cache_index'] = index_vec
      else:
        for j, name in enumerate(cache['decoder']):
          cache['decoder'][name]['self_attention']['cache_index'] = index_vec[j]
    logits = b.logits.view(R, 1, cfg.vocab_size)
    return (logits, {'cache': cache}) if mutable else logits

  # -- fused beam search: one graph replay per loop iteration ------------------------
  def make_fused_beam_step(self, loop, params, encoded, enc_tokens,
                           in_flight=False):
    """Returns a FusedBeamStep driving `loop` (a decoding.BeamLoop), or None
    when this configuration has to use the generic per-call path.  The step
    object (caches, cross K/V buffers, state, captured graphs) is kept and
    re-bound to the next loop of the same shape and options, so a stream of
    batches pays for allocation and graph capture once.  in_flight: the
    caller keeps several decodes running at once (see decode_lanes)."""
    if (not isinstance(encoded, BeamShared) or
        loop.cache_offset != int(self.scan_layers)):
      return None
    if loop.beam_size > 8:
      return None
    w = self.decoder_weights(params)
    lanes = self.decode_lanes or (
        1 if in_flight or self.streams_side_by_side() < 2 else 2)
    lanes = max(1, min(int(lanes), loop.batch_size))
    key = (id(w), tuple(encoded.x.shape), encoded.x.dtype, encoded.beams,
           loop.batch_size, loop.beam_size, loop.max_decode_len,
           tuple(loop.inputs_dev.shape), tuple(loop.brevity.shape),
           int(loop.eos_id), float(loop.min_brevity), float(loop.min_log_prob),
           int(loop.max_decode_step), int(loop.min_initial), lanes)
    return self._decode_context(
        key, w, loop,
        make=lambda slot: FusedBeamStep(self, loop, params, encoded,
                                        enc_tokens, lanes=lanes, slot=slot),
        rebind=lambda ctx: ctx.rebind(loop, encoded, enc_tokens))

  # Decode contexts of one (weights, shapes, options) key that are kept for
  # re-binding: more than one only when several decodes are in flight at once.
  MAX_CONTEXTS_PER_KEY = 4

  def _decode_context(self, key, w, owner, make, rebind):
    """A decode context for `owner` (the loop object that will drive it): a
    kept one of this key that no live, unfinished loop owns any more, re-bound,
    or a new one.  Contexts are kept in small pools per key, so that a caller
    who keeps several decodes in flight (each on its own stream) pays for
    their allocation and graph capture once.  make(slot) builds a context for
    pool slot `slot`, whose stream is decode_stream(slot)."""
    pool = self._beam_ctx.get(key)
    if pool and pool[0].w is not w:  # an id reused by other weights
      del self._beam_ctx[key]
      pool = None
    if pool is None:
      if len(self._beam_ctx) >= 2:  # a context holds the caches: keep few
        self._beam_ctx.pop(next(iter(self._beam_ctx)))
      pool = self._beam_ctx[key] = []
    for ctx in pool:
      if ctx.is_free():
        rebind(ctx)
        ctx.claim(owner)
        return ctx
    ctx = make(len(pool))
    ctx.claim(owner)
    if len(pool) < self.MAX_CONTEXTS_PER_KEY:
      pool.append(ctx)
    return ctx

  def streams_side_by_side(self) -> int:
    """How many decode streams the device runs side by side.  One hardware
    queue of the process serves the default stream, the others are dealt to
    the streams in turn, and queues beyond the fourth share command
    processors (3 decodes in flight pay with the runtime's default of 4
    queues, 4 with GPU_MAX_HW_QUEUES=8 or more, a fifth never).  Which queue a
    stream got cannot be asked, so it is measured once per device when the
    decode streams are made: the first n streams count when n short busy
    kernels, one per stream, take about as long as one."""
    import os
    fixed = self.side_by_side
    if fixed is None and os.environ.get('T5X_AMD_STREAMS_SIDE_BY_SIDE'):
      fixed = int(os.environ['T5X_AMD_STREAMS_SIDE_BY_SIDE'])
    if fixed is not None:
      return max(1, min(int(fixed), self.MAX_CONTEXTS_PER_KEY))
    self.decode_stream(0, measure=True)
    key = self._stream_key()
    measured = _DECODE_STREAMS_SIDE_BY_SIDE.get(key)
    if measured is not None:
      return measured
    try:
      queues = int(os.environ.get('GPU_MAX_HW_QUEUES', '4'))
    except ValueError:
      queues = 4
    return 4 if queues >= 8 else 3

  def _stream_key(self):
    key = torch.device(self._dev()).index
    return torch.cuda.current_device() if key is None else key

  def decode_context_bytes(self, batch_size, num_decodes, enc_len,
                           decode_len) -> int:
    """What one decode in flight keeps on the device besides the shared
    weights: its beam-expanded self-attention caches and the cross K/V of its
    batch (activations and beam state are small beside them)."""
    cfg = self.config
    el = 2 if self.dtype == 'bfloat16' else 4
    per_position = cfg.num_decoder_layers * 2 * cfg.num_heads * cfg.head_dim * el
    return per_position * (batch_size * num_decodes * decode_len +
                           batch_size * enc_len)

  def batches_in_flight(self, batch_size, num_decodes, enc_len,
                        decode_len) -> int:
    """How many batches of this shape to keep decoding at once: as many as the
    device runs side by side, fewer when their caches and cross K/V would
    take more than half of the free device memory."""
    n = self.streams_side_by_side()
    need = self.decode_context_bytes(batch_size, num_decodes, enc_len,
                                     decode_len)
    free, _ = torch.cuda.mem_get_info(self._dev())
    return max(1, min(n, int(free // 2 // max(1, need))))

  def decode_stream(self, slot, measure=False):
    """The stream of the decode contexts in pool slot `slot` (with batch
    lanes: of lane l of the context in slot s, at s * lanes + l).  The device
    runs streams side by side only when they sit on different hardware
    queues, of which a process has few (4 by default) and which streams are
    given in turn as they are first used; so the decode streams of a device
    are made once per process, together, and each is used once right away:
    consecutive slots then sit on different queues whatever streams the
    caller, or another model on the same device, makes later."""
    dev, key = self._dev(), self._stream_key()
    streams = _DECODE_STREAMS.get(key)
    if streams is None:
      streams = [torch.cuda.Stream(device=dev)
                 for _ in range(self.MAX_CONTEXTS_PER_KEY)]
      touch = torch.zeros((16,), dtype=torch.int32, device=dev)
      torch.cuda.current_stream().synchronize()
      for stream in streams:
        with torch.cuda.stream(stream):
          touch.zero_()
        stream.synchronize()
      _DECODE_STREAMS[key] = streams
    if measure and key not in _DECODE_STREAMS_SIDE_BY_SIDE:
      _DECODE_STREAMS_SIDE_BY_SIDE[key] = _measure_side_by_side(streams)
    return streams[slot % len(streams)]

  # -- fused sampling: one graph replay per loop iteration --------------------------
  def make_fused_sample_step(self, params, encoded, enc_tokens, owner=None,
                             **kw):
    """Returns a FusedSampleStep (see there for the arguments).  Like the beam
    contexts, the step object is kept per (weights, shapes, options) and
    re-bound to the next call's state; `owner` is the loop object that drives
    it (a context without owner is free for the next call at once)."""
    beams = encoded.beams if isinstance(encoded, BeamShared) else 1
    enc = encoded.x if isinstance(encoded, BeamShared) else encoded
    rows = kw['sequences'].shape[0]
    if rows != enc.shape[0] * beams:
      raise ValueError(f'{rows} decoder rows vs {enc.shape[0]} x {beams} '
                       'encoder rows')
    w = self.decoder_weights(params)
    key = ('sample', id(w), tuple(enc.shape), enc.dtype, beams,
           tuple(kw['sequences'].shape), int(kw['eos_id']), int(kw['topk']),
           float(kw['topp']), bool(kw['rescale']),
           kw.get('noise_source') is not None)
    return self._decode_context(
        key, w, owner,
        make=lambda slot: FusedSampleStep(self, params, encoded, enc_tokens,
                                          slot=slot, **kw),
        rebind=lambda ctx: ctx.rebind(encoded, enc_tokens, **kw))


class _OwnedContext:
  """What the kept decode contexts share: who drives them, and chunks of
  iterations whose end the host can ask about without waiting.

  A context is free for the next decode when nothing owns it, its owner is
  gone, or its owner has finished (`owner.finished`); contexts never keep
  their loop alive."""

  CHUNK_SLOTS = 4  # chunks a caller may have outstanding per context
  _owner = None
  _flag_host = None
  _n_chunks = 0

  def claim(self, owner):
    self._owner = None if owner is None else weakref.ref(owner)

  def is_free(self) -> bool:
    if self._owner is None:
      return True
    owner = self._owner()
    return owner is None or bool(getattr(owner, 'finished', False))

  def _end_chunk(self, flag, stream):
    """After a chunk of iterations was enqueued on `stream`: copies the
    device flag to pinned host memory and records an event behind it.
    Returns the ticket for _chunk_flag()."""
    if self._flag_host is None:
      self._flag_host = torch.zeros((self.CHUNK_SLOTS,), dtype=torch.int32,
                                    pin_memory=True)
      self._chunk_events = [torch.cuda.Event()
                            for _ in range(self.CHUNK_SLOTS)]
    slot = self._n_chunks % self.CHUNK_SLOTS
    self._n_chunks += 1
    with torch.cuda.stream(stream):
      self._flag_host[slot:slot + 1].copy_(flag.reshape(1), non_blocking=True)
    self._chunk_events[slot].record(stream)
    return slot

  def _chunk_flag(self, ticket, block=False):
    """The flag as the chunk left it, or None while the chunk is running
    (block: wait for it)."""
    event = self._chunk_events[ticket]
    if block:
      event.synchronize()
    elif not event.query():
      return None
    return int(self._flag_host[ticket])


class FusedSampleStep(_OwnedContext):
  """Whole temperature_sample iterations as replays of one captured HIP graph
  (decoder step on the current tokens, token choice, bookkeeping, loop flag).
  Owns the self-attention caches of its rows as one block
  [layers, 2, rows, H, 64, L].  The host refills a ring of Gumbel noise for
  the next `ring` steps, enqueues that many replays, and only then reads the
  flag back; replays enqueued after the last row ended change nothing."""

  def __init__(self, module, params, encoded, enc_tokens, *, sequences,
               cur_index, cur_token, ended, log_prob, max_decode_len,
               initial_eos_count, temperature, all_ended, eos_id, topk, topp,
               rescale, noise_source=None, ring=8, slot=0):
    from t5x_amd import _lib
    self._lib = _lib
    cfg, dev = module.config, module._dev()
    self.module, self.device = module, dev
    w = module.decoder_weights(params)
    if isinstance(encoded, BeamShared):
      beams, enc, enc_tok = encoded.beams, encoded.x, enc_tokens.x
    else:
      beams, enc, enc_tok = 1, encoded, enc_tokens
    enc_tok = torch.as_tensor(np.asarray(enc_tok), device=dev) if not isinstance(
        enc_tok, torch.Tensor) else enc_tok.to(dev)
    cross = module._cross_kv(w, enc, enc_tok, beams)
    self.w, self.cross = w, cross
    # The state the captured graph addresses; a later call is re-bound onto it
    # and reads its results (sequences, log_prob) from here.
    self.sequences, self.cur_index, self.cur_token = (sequences, cur_index,
                                                      cur_token)
    self.ended, self.log_prob = ended, log_prob
    self.max_decode_len, self.initial_eos_count = (max_decode_len,
                                                   initial_eos_count)
    self.temperature = temperature
    R, S = sequences.shape
    act = w.act_dtype
    # bfloat16: the caches are kept in a layout of the loop's own
    # (decode_cache_layout); cache_tree() converts back.
    self.cache_layout, self.L = decode_cache_layout(act, 1, S - 2)
    L = self.L
    nl = cfg.num_decoder_layers
    self.kv = torch.zeros((nl, 2, R, cfg.num_heads, cfg.head_dim,
                           L + (32 if self.cache_layout == 3 else 0)),
                          dtype=act, device=dev)
    self.cache_index = torch.zeros((nl,), dtype=torch.int32, device=dev)
    self.bufs = _StepBuffers(cfg, R, dev, act)
    self.keep_going = torch.ones((), dtype=torch.int32, device=dev)
    self.step_count = torch.zeros((), dtype=torch.int32, device=dev)
    self.tokens = torch.empty((R,), dtype=torch.int32, device=dev)
    self.tok_lp = torch.empty((R,), dtype=torch.float32, device=dev)
    self.all_ended = all_ended
    self.noise_source, self.ring = noise_source, int(ring)
    # A row ends at the latest in the iteration that writes its last position,
    # so no more than max(max_decode_len) iterations ever run (and no noise is
    # asked for beyond them).
    self.max_steps = int(max_decode_len.max().item())
    self.noise = None
    if noise_source is not None:
      self.noise = torch.empty((self.ring, R, cfg.vocab_size),
                               dtype=torch.float32, device=dev)
    layer_caches = [(self.kv[i, 0], self.kv[i, 1]) for i in range(nl)]
    self.model = module._model_step(w, cross, self.bufs, layer_caches,
                                    self.cache_index, R, beams, L,
                                    gate=self.keep_going,
                                    cache_layout=self.cache_layout)
    P = _lib.ptr
    st = _lib.SampleStep()
    st.sequences, st.cur_index, st.cur_token = (P(sequences), P(cur_index),
                                                P(cur_token))
    st.ended, st.log_prob = P(ended), P(log_prob)
    st.max_decode_len, st.initial_eos_count = (P(max_decode_len),
                                               P(initial_eos_count))
    st.temperature, st.gumbel = P(temperature), P(self.noise)
    st.noise_ring = self.ring
    st.step_count, st.tokens, st.token_logprobs = (
        P(self.step_count), P(self.tokens), P(self.tok_lp))
    from t5x_amd import ops
    self.sample_ws = ops.sample_tokens_workspace(R, dev)
    st.workspace = P(self.sample_ws)
    st.all_ended, st.keep_going = P(all_ended), P(self.keep_going)
    st.S, st.eos_id, st.topk = S, int(eos_id), int(topk)
    st.rescale, st.topp = int(bool(rescale)), float(topp)
    self.sample = st
    self._keepalive = (sequences, cur_index, cur_token, ended, log_prob,
                       max_decode_len, initial_eos_count, temperature)
    self.stream = module.decode_stream(slot)
    self.graph = None
    self.step = 0
    self._capture()

  _STATE = ('sequences', 'cur_index', 'cur_token', 'ended', 'log_prob',
            'max_decode_len', 'initial_eos_count', 'temperature')

  def rebind(self, encoded, enc_tokens, *, noise_source=None, **state):
    """Starts another call of the same shape and options on this context: the
    new state is copied into the buffers the graph addresses, the new encoder
    output is projected into the same cross K/V buffers, caches and counters
    restart."""
    module, dev = self.module, self.device
    cur = torch.cuda.current_stream()
    cur.wait_stream(self.stream)
    if isinstance(encoded, BeamShared):
      beams, enc, enc_tok = encoded.beams, encoded.x, enc_tokens.x
    else:
      beams, enc, enc_tok = 1, encoded, enc_tokens
    enc_tok = torch.as_tensor(np.asarray(enc_tok), device=dev) if not isinstance(
        enc_tok, torch.Tensor) else enc_tok.to(dev)
    cross = module._cross_kv(self.w, enc, enc_tok, beams, out=self.cross)
    assert cross is self.cross
    for name in self._STATE:
      getattr(self, name).copy_(state[name])
    self.all_ended.zero_()
    self.keep_going.fill_(1)
    self.step_count.zero_()
    self.kv.zero_()
    self.cache_index.zero_()
    self.noise_source = noise_source
    self.max_steps = int(self.max_decode_len.max().item())
    self.step = 0
    self.stream.wait_stream(cur)

  def _enqueue(self):
    self._lib.call('t5d_temperature_sample_step', self.stream.cuda_stream,
                   self.model, self.sample)

  def _record(self):
    lib = self._lib
    lib.call('t5d_graph_begin', self.stream.cuda_stream)
    try:
      self._enqueue()
    finally:
      handle = ctypes_void_p()
      lib.call('t5d_graph_end', self.stream.cuda_stream, handle_ref(handle))
    return handle

  def _capture(self):
    self.stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(self.stream):
      # First launches load the code objects; with the gate closed they
      # compute nothing.
      self.keep_going.zero_()
      self._enqueue()
      self.stream.synchronize()
      self.graph = self._record()
      self.keep_going.fill_(1)
    self.stream.synchronize()

  def iteration_graph(self, leave_out=0):
    """A graph of one iteration enqueued without the kernel families in the
    `leave_out` mask (t5d_measure_leave_out; 0: the full iteration), for
    timing a family by difference.  The caller replays it with launch_graph
    and destroys it with t5d_graph_destroy."""
    self.stream.synchronize()
    before = self._lib.measure_leave_out(int(leave_out))
    try:
      with torch.cuda.stream(self.stream):
        return self._record()
    finally:
      self._lib.measure_leave_out(before)

  def launch_graph(self, graph, n):
    for _ in range(n):
      self._lib.call('t5d_graph_launch', graph, self.stream.cuda_stream)

  def advance(self, n, wait=True):
    """Enqueues n more iterations (fewer when the longest row ends sooner),
    refilling the noise ring for each group of `ring` steps.  The refills are
    enqueued on the loop's stream, behind the iterations that read the slots
    they overwrite; with `wait` the host also stays at most one ring ahead of
    the device."""
    lib = self._lib
    with torch.cuda.stream(self.stream):
      todo = min(int(n), self.max_steps - self.step)
      while todo > 0:
        m = min(todo, self.ring - self.step % self.ring)
        if self.noise is not None:
          if wait and self.step % self.ring == 0:
            self.stream.synchronize()
          for step in range(self.step, self.step + m):
            g = self.noise_source.noise(step, tuple(self.noise.shape[1:]))
            self.noise[step % self.ring].copy_(
                torch.as_tensor(g, device=self.device).to(torch.float32))
        for _ in range(m):
          lib.call('t5d_graph_launch', self.graph, self.stream.cuda_stream)
        self.step += m
        todo -= m

  def running(self) -> bool:
    """The loop condition (not every row ended), read back from the device."""
    self.stream.synchronize()
    return not bool(self.all_ended.item())

  def launch_chunk(self, n):
    """Enqueues up to n iterations without waiting for anything and returns a
    ticket for chunk_running(); None when the loop has no iterations left."""
    if self.step >= self.max_steps:
      return None
    self.advance(n, wait=False)
    return self._end_chunk(self.all_ended, self.stream)

  def chunk_running(self, ticket, block=False):
    """Whether the loop condition still held after that chunk; None while the
    chunk is running (block: wait for it)."""
    flag = self._chunk_flag(ticket, block)
    return None if flag is None else flag == 0

  def finish(self):
    self.stream.synchronize()
    torch.cuda.current_stream().wait_stream(self.stream)

  def run(self):
    """Runs the loop to its end (every row ended); returns the number of
    iterations executed."""
    while self.step < self.max_steps:
      self.advance(self.ring - self.step % self.ring)
      if not self.running():
        break
    self.finish()
    return int(self.step_count.item())

  def cache_tree(self):
    """The caches in the reference's tree layout."""
    self.stream.synchronize()
    from t5x_amd import ops
    nl = self.kv.shape[0]
    held = self.cache_index.tolist()
    plain = [_plain_caches(self.kv[i], self.cache_layout, held[i])
             for i in range(nl)]
    return cache_tree(torch.stack([k for k, _ in plain]),
                      torch.stack([v for _, v in plain]),
                      self.cache_index, self.module.scan_layers)

  def __del__(self):
    try:
      if self.graph is not None:
        self._lib.call('t5d_graph_destroy', self.graph)
    except Exception:  # pylint: disable=broad-except
      pass


class _BeamLane:
  """One independent slice [b0, b1) of the batch: its own caches, activations,
  loop flag, position counter, stream and captured graph."""

  def __init__(self, owner, index, b0, b1, w, cross):
    from t5x_amd import _lib
    module, loop = owner.module, owner.loop
    cfg, dev = module.config, owner.device
    B, K = b1 - b0, loop.beam_size
    self.b0, self.b1 = b0, b1
    R, S, L = B * K, loop.max_decode_len, owner.L
    act = w.act_dtype
    nl = cfg.num_decoder_layers
    self.kv = torch.zeros((nl, 2, R, cfg.num_heads, cfg.head_dim,
                           L + (32 if owner.cache_layout == 3 else 0)),
                          dtype=act, device=dev)
    self.cache_index = torch.zeros((nl,), dtype=torch.int32, device=dev)
    self.bufs = _StepBuffers(cfg, R, dev, act)
    self.keep_going = loop.keep_going      # one flag for the whole batch
    self.cur_index = owner.lane_cur_index[index]
    k2 = 2 * K
    f32, i32 = torch.float32, torch.int32
    self.topk_vals = torch.empty((B, k2), dtype=f32, device=dev)
    self.topk_idx = torch.empty((B, k2), dtype=i32, device=dev)
    self.row_max = torch.empty((R,), dtype=f32, device=dev)
    self.row_lse = torch.empty((R,), dtype=f32, device=dev)
    self.scratch = torch.empty((2 * R * k2,), dtype=i32, device=dev)
    self.top_alive = loop.top_alive[b0:b1]
    # where the beams' cache rows live: slot of beam e, and for the reorder in
    # flight the slot each new beam reads and the slot it keeps
    self.cache_slot, self.cache_src, self.cache_dst = (
        owner.cache_slots[i, b0:b1] for i in range(3))
    lane_cross = dict(k=[t[b0:b1] for t in cross['k']],
                      v=[t[b0:b1] for t in cross['v']],
                      enc_len=cross['enc_len'][b0:b1], B=B, beams=K,
                      E=cross['E'],
                      units=cross.get('units') if owner.n_lanes == 1 else None)
    layer_caches = [(self.kv[i, 0], self.kv[i, 1]) for i in range(nl)]
    self.model = module._model_step(
        w, lane_cross, self.bufs, layer_caches, self.cache_index, R, K, L,
        gate=self.keep_going,
        pending_src=self.cache_src if owner.deferred_gather else None,
        pending_dst=self.cache_dst if owner.deferred_gather else None,
        cache_layout=owner.cache_layout)
    st = loop.cur
    P = _lib.ptr
    ptrs = _lib.BeamStatePtrs()
    ptrs.cur_index = P(self.cur_index)
    ptrs.live_logprobs = P(st.live_logprobs[b0:b1])
    ptrs.finished_scores = P(st.finished_scores[b0:b1])
    ptrs.live_seqs = P(st.live_seqs[b0:b1])
    ptrs.finished_seqs = P(st.finished_seqs[b0:b1])
    ptrs.finished_flags = P(st.finished_flags[b0:b1])
    self.state_ptrs = ptrs
    bs = _lib.BeamStep()
    bs.state = ptrs
    bs.inputs = P(loop.inputs_dev[b0:b1])
    bs.initial_index = P(loop.init_idx_dev[b0:b1])
    bs.brevity, bs.top_alive = P(loop.brevity), P(self.top_alive)
    bs.topk_vals, bs.topk_idx = P(self.topk_vals), P(self.topk_idx)
    bs.row_max, bs.row_lse = P(self.row_max), P(self.row_lse)
    bs.scratch, bs.ids = P(self.scratch), P(self.bufs.ids)
    bs.keep_going = P(self.keep_going)
    bs.S, bs.Lin, bs.eos_id = S, loop.inputs_dev.shape[1], int(loop.eos_id)
    bs.min_brevity, bs.min_log_prob = loop.min_brevity, loop.min_log_prob
    bs.max_decode_step = int(loop.max_decode_step)
    bs.min_initial_index = loop.min_initial
    bs.kv_base = P(self.kv)
    bs.kv_tensor_stride_bytes = self.kv[0, 0].numel() * self.kv.element_size()
    bs.n_kv_tensors = 2 * nl
    bs.skip_cond = 1 if owner.n_lanes > 1 else 0
    if owner.deferred_gather:
      bs.cache_slot, bs.cache_src, bs.cache_dst = (
          P(self.cache_slot), P(self.cache_src), P(self.cache_dst))
    self.beam = bs
    self.stream = module.decode_stream(owner.slot * owner.n_lanes + index)
    self.event = torch.cuda.Event()
    self.graph = None
    self.graph_long = None


class FusedBeamStep(_OwnedContext):
  """Whole beam-search iterations as replays of captured HIP graphs.

  The batch is cut into lanes (batch items never interact in beam search).
  Each lane owns its beam-expanded self-attention caches as one block
  [layers, 2, rows, H, 64, L], its activations and its position counter, and
  replays its own graph on its own stream, so the lanes' kernels overlap on
  the device: while one lane sits in a latency-bound phase another one
  streams.  The loop condition stays the reference's single whole-batch
  condition: after every iteration the lanes' streams join, one kernel
  evaluates it over the whole (contiguous) beam state into the one device
  flag that gates every kernel of every lane, and the lanes fork again, all
  without the host.  Iterations enqueued after the flag turned 0 change
  nothing, so the host may look at it only every few iterations."""

  def __init__(self, module, loop, params, encoded, enc_tokens, lanes=None,
               slot=0):
    from t5x_amd import _lib
    self._lib = _lib
    cfg, dev = module.config, module._dev()
    self.module, self.device = module, dev
    self.loop = loop
    w = module.decoder_weights(params)
    enc_tok = enc_tokens.x
    enc_tok = torch.as_tensor(np.asarray(enc_tok), device=dev) if not isinstance(
        enc_tok, torch.Tensor) else enc_tok.to(dev)
    cross = module._cross_kv(w, encoded.x, enc_tok, encoded.beams)
    B, K = loop.batch_size, loop.beam_size
    if cross['B'] != B or encoded.beams != K:
      raise ValueError('encoder batch / beams do not match the decode loop')
    S = loop.max_decode_len
    act = w.act_dtype
    el = 16 // torch.empty((), dtype=act).element_size()
    L = (S - 1 + el - 1) // el * el
    # With bfloat16 caches the reorder of a step is deferred into the next
    # step's self-attention kernels, which read each row's cache from its
    # source beam anyway.  Beams do not own fixed cache rows: a new beam
    # inherits the slot of its parent (only a parent's further children are
    # copied), so the reorder in flight is a pair of slot maps, cache_slots.
    self.deferred_gather = (K > 1 and act == torch.bfloat16 and
                            K * ((L + 127) // 128) <= 16)
    # The caches are then kept in a layout of the loop's own
    # (decode_cache_layout); cache_tree() converts back.  (The stand-alone
    # reorder kernel of the other path copies row prefixes, which only the
    # reference layout has.)
    self.cache_layout = 0
    if self.deferred_gather or (K == 1 and act == torch.bfloat16):
      layout, L32 = decode_cache_layout(act, K, S - 1)
      if K * ((L32 + 127) // 128) <= 16:
        self.cache_layout, L = layout, L32
      else:
        self.deferred_gather = False
    self.L = L
    loop.top_alive.copy_(torch.arange(K, dtype=torch.int32,
                                      device=dev).expand(B, K))
    # [0]: slot of beam e; [1], [2]: source / destination slots in flight
    self.cache_slots = torch.arange(K, dtype=torch.int32, device=dev).expand(
        3, B, K).contiguous()
    n = max(1, min(int(lanes or 1), B))
    self.n_lanes = n
    self.slot = slot
    bounds = [B * i // n for i in range(n + 1)]
    self.lane_cur_index = loop.cur.cur_index.to(torch.int32).reshape(1).repeat(n)
    self.cond_event = torch.cuda.Event()
    # What the captured graphs hold addresses of, beyond the lanes' own
    # buffers: the loop's state.  A later loop is re-bound onto these.
    self.w, self.cross = w, cross
    self.state = loop.cur
    self.inputs_dev, self.init_idx_dev = loop.inputs_dev, loop.init_idx_dev
    self.brevity, self.flag = loop.brevity, loop.keep_going
    self.top_alive = loop.top_alive
    self.lanes = [_BeamLane(self, i, bounds[i], bounds[i + 1], w, cross)
                  for i in range(n)]
    self._capture()

  @property
  def loop(self):
    """The loop bound to this context (None once it is gone)."""
    return self._loop()

  @loop.setter
  def loop(self, loop):
    self._loop = weakref.ref(loop)

  _STATE_FIELDS = ('cur_index', 'live_logprobs', 'finished_scores', 'live_seqs',
                   'finished_seqs', 'finished_flags')

  def rebind(self, loop, encoded, enc_tokens):
    """Takes over a freshly initialised loop of the same shape and options:
    its initial state is copied into the buffers the captured graphs address
    (which the loop then uses as its own), the new encoder output is projected
    into the same cross K/V buffers, caches and counters start from zero."""
    module, dev = self.module, self.device
    cur = torch.cuda.current_stream()
    for lane in self.lanes:  # whatever the previous loop left in flight
      cur.wait_stream(lane.stream)
    enc_tok = enc_tokens.x
    enc_tok = torch.as_tensor(np.asarray(enc_tok), device=dev) if not isinstance(
        enc_tok, torch.Tensor) else enc_tok.to(dev)
    cross = module._cross_kv(self.w, encoded.x, enc_tok, encoded.beams,
                             out=self.cross)
    assert cross is self.cross
    for name in self._STATE_FIELDS:
      getattr(self.state, name).copy_(getattr(loop.cur, name))
    self.inputs_dev.copy_(loop.inputs_dev)
    self.init_idx_dev.copy_(loop.init_idx_dev)
    self.brevity.copy_(loop.brevity)
    K = loop.beam_size
    self.top_alive.copy_(torch.arange(K, dtype=torch.int32, device=dev).expand(
        loop.batch_size, K))
    self.cache_slots.copy_(torch.arange(K, dtype=torch.int32,
                                        device=dev).expand_as(self.cache_slots))
    self.lane_cur_index.copy_(
        loop.cur.cur_index.to(torch.int32).reshape(1).expand(self.n_lanes))
    for lane in self.lanes:
      lane.kv.zero_()
      lane.cache_index.zero_()
    loop.cur = loop.nxt = self.state
    loop.inputs_dev, loop.init_idx_dev = self.inputs_dev, self.init_idx_dev
    loop.brevity, loop.keep_going = self.brevity, self.flag
    loop.top_alive = self.top_alive
    self.loop = loop
    for lane in self.lanes:
      lane.stream.wait_stream(cur)
    self._cond(self.lanes[0].stream)
    self.lanes[0].stream.synchronize()

  def _enqueue(self, lane):
    self._lib.call('t5d_beam_search_step', lane.stream.cuda_stream,
                   lane.model, lane.beam)

  def _cond(self, stream):
    """The whole-batch loop condition -> loop.keep_going, on `stream`."""
    loop = self.loop
    st = self._lib.BeamStatePtrs()
    P = self._lib.ptr
    st.cur_index = P(self.lane_cur_index)  # lane 0's counter; all are equal
    st.live_logprobs = P(loop.cur.live_logprobs)
    st.finished_scores = P(loop.cur.finished_scores)
    st.live_seqs = P(loop.cur.live_seqs)
    st.finished_seqs = P(loop.cur.finished_seqs)
    st.finished_flags = P(loop.cur.finished_flags)
    self._lib.call('t5d_beam_cond', stream.cuda_stream, handle_ref(st),
                   loop.batch_size, loop.beam_size, loop.max_decode_len,
                   float(loop.min_brevity), float(loop.min_log_prob),
                   int(loop.max_decode_step), int(loop.min_initial),
                   loop.keep_going.data_ptr())

  # Iterations recorded in the long graph of a single-lane loop: one launch
  # (and one gap between launches) per that many iterations.
  GRAPH_STEPS = 8

  def _record(self, lane, steps):
    lib = self._lib
    lib.call('t5d_graph_begin', lane.stream.cuda_stream)
    try:
      for _ in range(steps):
        self._enqueue(lane)
    finally:
      handle = ctypes_void_p()
      lib.call('t5d_graph_end', lane.stream.cuda_stream, handle_ref(handle))
    return handle

  def iteration_graph(self, leave_out=0):
    """A graph of one iteration enqueued without the kernel families in the
    `leave_out` mask (t5d_measure_leave_out; 0: the full iteration), for
    timing a family by difference.  Single-lane loops.  The caller replays it
    with launch_graph and destroys it with t5d_graph_destroy."""
    if self.n_lanes != 1:
      raise ValueError('iteration graphs are for the single-lane loop')
    lane = self.lanes[0]
    lane.stream.synchronize()
    before = self._lib.measure_leave_out(int(leave_out))
    try:
      with torch.cuda.stream(lane.stream):
        return self._record(lane, 1)
    finally:
      self._lib.measure_leave_out(before)

  def launch_graph(self, graph, n):
    stream = self.lanes[0].stream.cuda_stream
    for _ in range(n):
      self._lib.call('t5d_graph_launch', graph, stream)

  @property
  def stream(self):
    return self.lanes[0].stream

  def _capture(self):
    loop = self.loop
    cur = torch.cuda.current_stream()
    for lane in self.lanes:
      lane.stream.wait_stream(cur)
      with torch.cuda.stream(lane.stream):
        # First launches load the code objects; do them with the gate closed
        # so nothing is computed, then open the gate with the real condition.
        loop.keep_going.zero_()
        self._enqueue(lane)
        lane.stream.synchronize()
        lane.graph = self._record(lane, 1)
        if self.n_lanes == 1:
          lane.graph_long = self._record(lane, self.GRAPH_STEPS)
      lane.stream.synchronize()
    self._cond(self.lanes[0].stream)
    self.lanes[0].stream.synchronize()

  def launch(self, n=1):
    lanes, lib = self.lanes, self._lib
    first = lanes[0].stream
    if len(lanes) == 1:
      lane = lanes[0]
      while n >= self.GRAPH_STEPS:
        lib.call('t5d_graph_launch', lane.graph_long, first.cuda_stream)
        n -= self.GRAPH_STEPS
      for _ in range(n):
        lib.call('t5d_graph_launch', lane.graph, first.cuda_stream)
      return
    for _ in range(n):
      for lane in lanes:
        lib.call('t5d_graph_launch', lane.graph, lane.stream.cuda_stream)
      # join -> one condition for the whole batch -> fork
      for lane in lanes[1:]:
        lane.event.record(lane.stream)
        first.wait_event(lane.event)
      self._cond(first)
      self.cond_event.record(first)
      for lane in lanes[1:]:
        lane.stream.wait_event(self.cond_event)

  def launch_chunk(self, n):
    """launch(n), and a ticket for chunk_running().  (The loop condition
    bounds the loop: there is always a next iteration to enqueue.)"""
    self.launch(n)
    # the last condition of a chunk is evaluated on the first lane's stream
    # after all lanes joined; a single lane's kernels are on that stream too
    return self._end_chunk(self.flag, self.lanes[0].stream)

  def chunk_running(self, ticket, block=False):
    """Whether the loop condition still held after that chunk; None while the
    chunk is running (block: wait for it)."""
    flag = self._chunk_flag(ticket, block)
    return None if flag is None else flag != 0

  def synchronize(self):
    for lane in self.lanes:
      lane.stream.synchronize()
    # the lanes advance in lock step
    self.loop.cur.cur_index.copy_(self.lane_cur_index[0])

  def keep_going(self) -> bool:
    self.synchronize()
    return bool(self.loop.keep_going.item())

  def finish(self):
    self.synchronize()

  def cache_tree(self):
    """The caches in the reference's tree layout (copies; pending reorders
    are applied first)."""
    self.synchronize()
    from t5x_amd import ops
    K = self.loop.beam_size
    for lane in self.lanes:
      if self.deferred_gather:
        # Beam e's rows are in slot cache_src[b, e] (the copy into its own
        # slot is still in flight): bring every beam to slot e, then mark all
        # of it done.
        nl = lane.kv.shape[0]
        B = lane.b1 - lane.b0
        ops.cache_gather_beams(
            lane.kv[0, 0].view(B, K, *lane.kv.shape[3:]), lane.cache_src,
            n_tensors=2 * nl,
            tensor_stride_bytes=lane.kv[0, 0].numel() * lane.kv.element_size())
        identity = torch.arange(K, dtype=torch.int32,
                                device=self.device).expand(B, K)
        for t in (lane.top_alive, lane.cache_slot, lane.cache_src,
                  lane.cache_dst):
          t.copy_(identity)
    torch.cuda.synchronize()
    nl = self.lanes[0].kv.shape[0]
    kv = torch.cat([lane.kv for lane in self.lanes], dim=2)
    idx = self.lanes[0].cache_index
    held = idx.tolist()
    plain = [_plain_caches(kv[i], self.cache_layout, held[i])
             for i in range(nl)]
    return cache_tree(torch.stack([k for k, _ in plain]),
                      torch.stack([v for _, v in plain]), idx,
                      self.module.scan_layers)

  def __del__(self):
    try:
      for lane in self.lanes:
        for g in (lane.graph, lane.graph_long):
          if g is not None:
            self._lib.call('t5d_graph_destroy', g)
    except Exception:  # pylint: disable=broad-except
      pass


def ctypes_void_p():
  import ctypes
  return ctypes.c_void_p()


def handle_ref(h):
  import ctypes
  return ctypes.byref(h)


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
