"""T5.1.1 encoder forward (t5x/examples/t5/network.py:47-96,182-219,315-343),
run once per batch before the decode loop.

bfloat16: hand-written HIP kernels — the many-row dense kernel
(t5d_gemm_rows: fused residual / gated-GELU epilogues, value projection written
transposed), whole-sequence self-attention on the matrix cores
(t5d_encoder_attention), the embedding gather and the RMS norm of the decode
path.  float32 (the exactness-test dtype): library GEMMs and softmax through
torch with the reference's rounding points.  The decode step never calls into
this module.
"""

import numpy as np
import torch

from t5x_amd import network


def _dense(x, w):
  kern, scale = w
  if scale is None:
    return torch.matmul(x, kern)
  return (torch.matmul(x.float(), kern.float()) * scale).to(x.dtype)


def _prep(kernel, act, wdt, device):
  k = network._f32(kernel, device)
  return network.DecoderWeights._dense_for_library(k, act, wdt)


class EncoderWeights:

  def __init__(self, cfg, params, device):
    act = network._TORCH_DTYPE[cfg.dtype]
    wdt = network._TORCH_DTYPE[cfg.weight_dtype or cfg.dtype]
    enc = params['encoder']
    self.embedding = network._f32(params['token_embedder']['embedding'],
                                  device).to(act)
    self.rel_embedding = network._f32(enc['relpos_bias']['rel_embedding'],
                                      device).to(act)
    self.layers = []
    for i in range(cfg.num_encoder_layers):
      p = enc[f'layers_{i}']
      a, m = p['attention'], p['mlp']
      self.layers.append(dict(
          ln_attn=network._f32(p['pre_attention_layer_norm']['scale'],
                               device).to(act),
          q=_prep(a['query']['kernel'], act, wdt, device),
          k=_prep(a['key']['kernel'], act, wdt, device),
          v=_prep(a['value']['kernel'], act, wdt, device),
          o=_prep(a['out']['kernel'], act, wdt, device),
          ln_mlp=network._f32(p['pre_mlp_layer_norm']['scale'],
                              device).to(act),
          wi_0=_prep(m['wi_0']['kernel'], act, wdt, device),
          wi_1=_prep(m['wi_1']['kernel'], act, wdt, device),
          wo=_prep(m['wo']['kernel'], act, wdt, device)))
    self.ln_final = network._f32(enc['encoder_norm']['scale'], device).to(act)


def _rms(x, scale, eps=1e-6):
  xf = x.float()
  y = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype)
  return y * scale


class EncoderKernelWeights:
  """Encoder parameters packed for the HIP kernels (bfloat16 activations)."""

  def __init__(self, cfg, params, device):
    from t5x_amd import ops
    act = torch.bfloat16
    wdt = network._TORCH_DTYPE[cfg.weight_dtype or cfg.dtype]
    enc = params['encoder']
    f = lambda x: network._f32(x, device)
    self.embedding = f(params['token_embedder']['embedding']).to(act).contiguous()
    self.rel_embedding = f(enc['relpos_bias']['rel_embedding']).to(act)
    self.layers = []
    for i in range(cfg.num_encoder_layers):
      p = enc[f'layers_{i}']
      a, m = p['attention'], p['mlp']
      qk = torch.cat([f(a['query']['kernel']), f(a['key']['kernel'])],
                     dim=1).contiguous()
      self.layers.append(dict(
          ln_attn=f(p['pre_attention_layer_norm']['scale']).to(act),
          qk=ops.pack_weight(qk, act, wdt),
          v=ops.pack_weight(f(a['value']['kernel']), act, wdt),
          o=ops.pack_weight(f(a['out']['kernel']), act, wdt),
          ln_mlp=f(p['pre_mlp_layer_norm']['scale']).to(act),
          wi=ops.pack_weight(f(m['wi_0']['kernel']), act, wdt,
                             gate_kernel=f(m['wi_1']['kernel'])),
          wo=ops.pack_weight(f(m['wo']['kernel']), act, wdt)))
    self.ln_final = f(enc['encoder_norm']['scale']).to(act)
    self._bias = {}

  def rel_bias(self, E):
    """[H, 2E-1] bias by (key - query + E - 1), bidirectional buckets."""
    if E not in self._bias:
      bucket = network.relative_position_bucket(np.arange(-(E - 1), E),
                                                bidirectional=True)
      idx = torch.as_tensor(bucket.astype(np.int64),
                            device=self.rel_embedding.device)
      self._bias[E] = self.rel_embedding[:, idx].contiguous()
    return self._bias[E]


def _encode_hip(module, params, tokens):
  """bfloat16 encoder on the HIP kernels; tokens [B, E] int64 on the device."""
  from t5x_amd import _lib, ops
  cfg, dev = module.config, module._dev()
  key = ('hip', id(params))
  if key not in module._enc_weights:
    module._enc_weights[key] = (params, EncoderKernelWeights(cfg, params, dev))
  w = module._enc_weights[key][1]
  B, E = tokens.shape
  H = cfg.num_heads
  HD = H * 64
  valid = tokens > 0
  lens = valid.sum(dim=1).to(torch.int32)
  prefix = torch.arange(E, device=dev)[None, :] < lens[:, None]
  if not bool((prefix == valid).all()):
    raise ValueError('encoder padding must be a suffix of zeros')
  lens = lens.contiguous()
  Ep = (E + 31) // 32 * 32  # values are stored in blocks of 32 positions
  bias = w.rel_bias(E)
  ids = tokens.reshape(-1).to(torch.int32).contiguous()
  x = ops.embed(w.embedding, ids)
  M = B * E
  v_t = torch.zeros((B, H, Ep // 32, 64, 32), dtype=x.dtype, device=dev)
  for l in w.layers:
    xn = ops.rmsnorm(x, l['ln_attn'])
    qk = ops.gemm_rows(xn, l['qk'])                       # [M, q | k]
    ops.gemm_rows(xn, l['v'], out=v_t, layout=_lib.OUT_HEADS_VALUE, E=E, Ep=Ep)
    attn = ops.encoder_attention(qk[:, :HD], qk[:, HD:], v_t, bias, lens)
    x = ops.gemm_rows(attn, l['o'], residual=x)
    y = ops.rmsnorm(x, l['ln_mlp'])
    h = ops.gemm_rows(y, l['wi'])
    x = ops.gemm_rows(h, l['wo'], residual=x)
  return ops.rmsnorm(x, w.ln_final).view(B, E, cfg.emb_dim)


def encode(module, params, encoder_input_tokens):
  cfg, dev = module.config, module._dev()
  tokens = encoder_input_tokens
  if not isinstance(tokens, torch.Tensor):
    tokens = torch.as_tensor(np.asarray(tokens), device=dev)
  tokens = tokens.to(dev).long()
  B, E = tokens.shape
  if cfg.dtype == 'bfloat16' and E % 4 == 0:
    return _encode_hip(module, params, tokens)
  key = id(params)
  if key not in module._enc_weights:
    module._enc_weights[key] = (params, EncoderWeights(cfg, params, dev))
  w = module._enc_weights[key][1]
  H, D = cfg.num_heads, cfg.head_dim
  act = w.embedding.dtype
  bucket = network.relative_position_bucket(
      np.arange(E)[None, :] - np.arange(E)[:, None], bidirectional=True)
  rel = w.rel_embedding[:, torch.as_tensor(bucket, device=dev)][None]
  valid = tokens > 0
  zero = torch.zeros((), dtype=act, device=dev)
  neg = torch.full((), -1e10, dtype=act, device=dev)
  out = torch.empty((B, E, cfg.emb_dim), dtype=act, device=dev)
  # bound the [b, H, E, E] score tensor to ~1 GiB per chunk
  chunk = max(1, min(B, (1 << 30) // max(1, H * E * E * 4)))
  for s in range(0, B, chunk):
    tok = tokens[s:s + chunk]
    v = valid[s:s + chunk]
    mask = (v[:, None, :, None] & v[:, None, None, :])
    bias = torch.where(mask, zero, neg) + rel
    x = w.embedding[tok]
    b = tok.shape[0]
    for l in w.layers:
      xn = _rms(x, l['ln_attn'])
      q = _dense(xn, l['q']).view(b, E, H, D).transpose(1, 2)
      k = _dense(xn, l['k']).view(b, E, H, D).transpose(1, 2)
      vv = _dense(xn, l['v']).view(b, E, H, D).transpose(1, 2)
      scores = torch.matmul(q, k.transpose(-1, -2)) + bias
      p = torch.softmax(scores, dim=-1)
      o = torch.matmul(p, vv).transpose(1, 2).reshape(b, E, H * D)
      x = _dense(o, l['o']) + x
      y = _rms(x, l['ln_mlp'])
      h = torch.nn.functional.gelu(_dense(y, l['wi_0']), approximate='tanh')
      h = h * _dense(y, l['wi_1'])
      x = _dense(h, l['wo']) + x
    out[s:s + chunk] = _rms(x, w.ln_final)
  return out
