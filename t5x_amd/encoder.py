"""T5.1.1 encoder forward (t5x/examples/t5/network.py:47-96,182-219,315-343),
run once per batch before the decode loop, on hand-written HIP kernels.

bfloat16: the many-row dense kernel (t5d_gemm_rows: fused residual /
gated-GELU epilogues, value projection written transposed), whole-sequence
self-attention on the matrix cores (t5d_encoder_attention), the embedding
gather and the RMS norm of the decode path.  float32 (the exactness-test
dtype): the float32 dense kernel with the layer norms riding inside it
(t5d_gemm / t5d_norm_gemm) and a vector-ALU attention kernel
(t5d_encoder_attention_f32).  The decode step never calls into this module.
"""

import numpy as np
import torch

from t5x_amd import network


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
  lens, bits = _key_mask(tokens, dev)
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
    attn = ops.encoder_attention(qk[:, :HD], qk[:, HD:], v_t, bias, lens,
                                 valid_bits=bits)
    x = ops.gemm_rows(attn, l['o'], residual=x)
    y = ops.rmsnorm(x, l['ln_mlp'])
    h = ops.gemm_rows(y, l['wi'])
    x = ops.gemm_rows(h, l['wo'], residual=x)
  return ops.rmsnorm(x, w.ln_final).view(B, E, cfg.emb_dim)


class EncoderKernelWeightsF32:
  """Encoder parameters for the float32 kernels: row-major [K, N] kernels,
  query | key | value fused into one projection."""

  def __init__(self, cfg, params, device):
    from t5x_amd import ops
    f32 = torch.float32
    enc = params['encoder']
    f = lambda x: network._f32(x, device)
    self.embedding = f(params['token_embedder']['embedding']).contiguous()
    self.rel_embedding = f(enc['relpos_bias']['rel_embedding'])
    self.layers = []
    for i in range(cfg.num_encoder_layers):
      p = enc[f'layers_{i}']
      a, m = p['attention'], p['mlp']
      qkv = torch.cat([f(a['query']['kernel']), f(a['key']['kernel']),
                       f(a['value']['kernel'])], dim=1).contiguous()
      self.layers.append(dict(
          ln_attn=f(p['pre_attention_layer_norm']['scale']).contiguous(),
          qkv=ops.pack_weight(qkv, f32),
          o=ops.pack_weight(f(a['out']['kernel']), f32),
          ln_mlp=f(p['pre_mlp_layer_norm']['scale']).contiguous(),
          wi=ops.pack_weight(f(m['wi_0']['kernel']), f32,
                             gate_kernel=f(m['wi_1']['kernel'])),
          wo=ops.pack_weight(f(m['wo']['kernel']), f32)))
    self.ln_final = f(enc['encoder_norm']['scale']).contiguous()
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


def _key_mask(tokens, dev):
  """The padding mask of t5x/examples/t5/network.py:325-328 (token > 0,
  element-wise) as the kernels take it: (lengths, bits).  Padding that is a
  suffix of zeros, the usual case, is a length per row and bits None; a
  padding token inside the text gives the last valid position + 1 and one bit
  per position (ops.pack_valid_bits)."""
  from t5x_amd import ops
  B, E = tokens.shape
  valid = tokens > 0
  lens = valid.sum(dim=1).to(torch.int32)
  prefix = torch.arange(E, device=dev)[None, :] < lens[:, None]
  if bool((prefix == valid).all()):
    return lens.contiguous(), None
  last = (valid * torch.arange(1, E + 1, device=dev)[None, :]).max(dim=1).values
  return last.to(torch.int32).contiguous(), ops.pack_valid_bits(valid)


def _encode_hip_f32(module, params, tokens):
  """float32 encoder on the HIP kernels; tokens [B, E] int64 on the device."""
  from t5x_amd import ops
  cfg, dev = module.config, module._dev()
  key = ('hip_f32', id(params))
  if key not in module._enc_weights:
    module._enc_weights[key] = (params,
                                EncoderKernelWeightsF32(cfg, params, dev))
  w = module._enc_weights[key][1]
  B, E = tokens.shape
  H = cfg.num_heads
  lens, bits = _key_mask(tokens, dev)
  bias = w.rel_bias(E)
  x = ops.embed(w.embedding, tokens.reshape(-1).to(torch.int32).contiguous())
  for l in w.layers:
    qkv = ops.gemm(x, l['qkv'], norm_scale=l['ln_attn'])
    attn = ops.encoder_attention_f32(qkv, bias, lens, H, valid_bits=bits)
    x = ops.gemm(attn, l['o'], residual=x)
    h = ops.gemm(x, l['wi'], norm_scale=l['ln_mlp'])
    x = ops.gemm(h, l['wo'], residual=x)
  return ops.rmsnorm(x, w.ln_final).view(B, E, cfg.emb_dim)


def encode(module, params, encoder_input_tokens):
  cfg, dev = module.config, module._dev()
  tokens = encoder_input_tokens
  if not isinstance(tokens, torch.Tensor):
    tokens = torch.as_tensor(np.asarray(tokens), device=dev)
  tokens = tokens.to(dev).long()
  B, E = tokens.shape
  if cfg.dtype == 'float32':
    return _encode_hip_f32(module, params, tokens)
  if cfg.dtype != 'bfloat16':
    raise ValueError(f'unsupported encoder dtype {cfg.dtype}')
  if E % 4 == 0:
    return _encode_hip(module, params, tokens)
  # The dense kernel's head-layout epilogue takes lengths in multiples of 4:
  # pad with padding tokens (masked keys; their own rows are dropped again).
  E4 = (E + 3) // 4 * 4
  padded = torch.zeros((B, E4), dtype=tokens.dtype, device=dev)
  padded[:, :E] = tokens
  return _encode_hip(module, params, padded)[:, :E].contiguous()
