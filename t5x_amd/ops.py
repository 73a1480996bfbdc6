"""Tensor-level wrappers over the t5d C ABI.

Each function takes torch device tensors, checks what the kernel assumes
(shape, dtype, contiguity, device) and enqueues the kernel on the current
torch stream.  No function here computes anything in torch.
"""

import ctypes

import torch

from t5x_amd import _lib
from t5x_amd._lib import BF16, EPI_GEGLU, EPI_NONE, EPI_RESIDUAL, F32, I8

__all__ = [
    'PackedWeight', 'pack_weight', 'embed', 'rmsnorm', 'gemm',
    'self_attention_step', 'cross_attention_step', 'add_i32',
    'cache_gather_beams', 'gather_beams', 'top_k', 'beam_topk', 'BeamBuffers',
    'beam_update', 'beam_cond', 'sample_tokens', 'sample_update',
]


def _chk(t, name, dtype=None, ndim=None):
  if not isinstance(t, torch.Tensor):
    raise TypeError(f'{name}: expected a torch tensor, got {type(t)}')
  if not t.is_cuda:
    raise ValueError(f'{name}: tensor must live on the GPU')
  if not t.is_contiguous():
    raise ValueError(f'{name}: tensor must be contiguous')
  if dtype is not None and t.dtype != dtype:
    raise ValueError(f'{name}: dtype {t.dtype}, expected {dtype}')
  if ndim is not None and t.dim() != ndim:
    raise ValueError(f'{name}: rank {t.dim()}, expected {ndim}')
  return t


def _s():
  return _lib.stream_handle()


class PackedWeight:
  """A dense kernel in the layout t5d_gemm streams.

  dtype float32: row-major [K, N] (or [K, 2F] = wi_0 | wi_1 for geglu).
  dtype bfloat16 / int8: 32x16 MFMA tiles (see include/t5d.h), `scales` holds
  the per-output-channel float32 scales of int8 weights in packed column order.
  """

  def __init__(self, data, K, N, w_dtype, geglu=False, scales=None):
    self.data, self.K, self.N = data, K, N
    self.w_dtype, self.geglu, self.scales = w_dtype, geglu, scales

  @property
  def out_features(self):
    return self.N // 2 if self.geglu else self.N

  def nbytes(self):
    n = self.data.numel() * self.data.element_size()
    if self.scales is not None:
      n += self.scales.numel() * 4
    return n


def _quantize(w):
  """Per-output-channel symmetric int8 (scale = max|w| / 127).  The divisor is
  a tensor: dividing by a Python scalar multiplies by its rounded reciprocal,
  which moves some scales by an ulp and with them a few weights by one step."""
  amax = w.abs().amax(dim=0).clamp_min(1e-30)
  scale = amax / torch.full_like(amax, 127.0)
  q = torch.clamp(torch.round(w / scale), -127, 127).to(torch.int8)
  return q, scale.to(torch.float32)


def pack_weight(kernel, act_dtype, weight_dtype=None, gate_kernel=None):
  """kernel: float32 [K, N] device tensor (reference layout).  `gate_kernel`
  (wi_1) makes a geglu-packed pair with `kernel` as wi_0."""
  _chk(kernel, 'kernel', torch.float32, 2)
  K, N = kernel.shape
  geglu = gate_kernel is not None
  if geglu:
    _chk(gate_kernel, 'gate_kernel', torch.float32, 2)
    if gate_kernel.shape != kernel.shape:
      raise ValueError('wi_0 / wi_1 shapes differ')
  weight_dtype = weight_dtype or act_dtype
  if act_dtype == torch.float32:
    if weight_dtype != torch.float32:
      raise ValueError('float32 activations need float32 weights')
    data = torch.cat([kernel, gate_kernel], dim=1) if geglu else kernel.clone()
    return PackedWeight(data.contiguous(), K, data.shape[1], F32, geglu)
  if act_dtype != torch.bfloat16:
    raise ValueError(f'unsupported activation dtype {act_dtype}')
  Np = 2 * N if geglu else N
  scales = None
  if weight_dtype == torch.bfloat16:
    src = kernel.to(torch.bfloat16).contiguous()
    src2 = gate_kernel.to(torch.bfloat16).contiguous() if geglu else None
    code = BF16
  elif weight_dtype == torch.int8:
    src, s0 = _quantize(kernel)
    src = src.contiguous()
    if geglu:
      src2, s1 = _quantize(gate_kernel)
      src2 = src2.contiguous()
      # packed column 16*nt + c <- wi_0[8*nt + c] (c < 8) | wi_1[8*nt + c - 8]
      scales = torch.stack([s0.view(-1, 8), s1.view(-1, 8)], dim=1).reshape(-1)
    else:
      src2, scales = None, s0
    scales = scales.contiguous()
    code = I8
  else:
    raise ValueError(f'unsupported weight dtype {weight_dtype}')
  nbytes = _lib.load().t5d_packed_weight_bytes(code, K, Np)
  if nbytes < 0:
    raise ValueError(f'kernel [{K}, {Np}] does not tile 32x16')
  dst = torch.empty(nbytes, dtype=torch.uint8, device=kernel.device)
  _lib.call('t5d_pack_weight', _s(), code, src.data_ptr(), _lib.ptr(src2),
            dst.data_ptr(), K, N, int(geglu))
  return PackedWeight(dst, K, Np, code, geglu, scales)


def embed(table, ids, out=None):
  _chk(table, 'table', ndim=2)
  _chk(ids, 'ids', torch.int32)
  V, d = table.shape
  R = ids.numel()
  if out is None:
    out = torch.empty((R, d), dtype=table.dtype, device=table.device)
  _chk(out, 'out', table.dtype)
  _lib.call('t5d_embed', _s(), _lib.dtype_code(table.dtype), table.data_ptr(),
            ids.data_ptr(), out.data_ptr(), R, d, V)
  return out


def rmsnorm(x, scale, out=None, eps=1e-6):
  _chk(x, 'x', ndim=2)
  _chk(scale, 'scale', x.dtype, 1)
  R, d = x.shape
  if scale.shape[0] != d:
    raise ValueError('scale length mismatch')
  if out is None:
    out = torch.empty_like(x)
  _chk(out, 'out', x.dtype)
  _lib.call('t5d_rmsnorm', _s(), _lib.dtype_code(x.dtype), x.data_ptr(),
            scale.data_ptr(), out.data_ptr(), R, d, float(eps))
  return out


def gemm(a, w: PackedWeight, out=None, residual=None, out_dtype=None,
         norm_scale=None, eps=1e-6):
  """C = epilogue(a @ W).  a [M, K]; geglu weights give [M, F].  With
  norm_scale [K] the rows of a are RMS-normalised first, in the same kernel."""
  _chk(a, 'a', ndim=2)
  M, K = a.shape
  if K != w.K:
    raise ValueError(f'a is [{M}, {K}] but the kernel has K={w.K}')
  epi = EPI_GEGLU if w.geglu else (EPI_RESIDUAL if residual is not None
                                   else EPI_NONE)
  out_dtype = out_dtype or a.dtype
  n_out = w.out_features
  if out is None:
    out = torch.empty((M, n_out), dtype=out_dtype, device=a.device)
  _chk(out, 'out', out_dtype, 2)
  if tuple(out.shape) != (M, n_out):
    raise ValueError(f'out shape {tuple(out.shape)} != {(M, n_out)}')
  if residual is not None:
    _chk(residual, 'residual', a.dtype, 2)
    if tuple(residual.shape) != (M, n_out):
      raise ValueError('residual shape mismatch')
  dt = _lib.dtype_code(a.dtype)
  if norm_scale is not None:
    _chk(norm_scale, 'norm_scale', a.dtype, 1)
    if norm_scale.numel() != K or residual is not None:
      raise ValueError('norm_scale must be [K]; no residual with a fused norm')
    _lib.call('t5d_norm_gemm', _s(), dt, w.w_dtype,
              _lib.dtype_code(out_dtype), a.data_ptr(), norm_scale.data_ptr(),
              float(eps), w.data.data_ptr(), _lib.ptr(w.scales),
              out.data_ptr(), M, K, w.N, epi)
    return out
  _lib.call('t5d_gemm', _s(), dt, w.w_dtype, _lib.dtype_code(out_dtype),
            a.data_ptr(), w.data.data_ptr(), _lib.ptr(w.scales),
            _lib.ptr(residual), out.data_ptr(), M, K, w.N, epi, None, None)
  return out


def gemm_tiled(a, w: PackedWeight, mp, nt, k_parts=1, out=None, residual=None,
               out_dtype=None):
  """gemm on the large-tile kernel (mp*16 rows x nt*16 columns per workgroup,
  K split over k_parts workgroups)."""
  _chk(a, 'a', torch.bfloat16, 2)
  M, K = a.shape
  if K != w.K:
    raise ValueError(f'a is [{M}, {K}] but the kernel has K={w.K}')
  epi = EPI_GEGLU if w.geglu else (EPI_RESIDUAL if residual is not None
                                   else EPI_NONE)
  out_dtype = out_dtype or a.dtype
  if out is None:
    out = torch.empty((M, w.out_features), dtype=out_dtype, device=a.device)
  _chk(out, 'out', out_dtype, 2)
  if residual is not None:
    _chk(residual, 'residual', a.dtype, 2)
    if tuple(residual.shape) != (M, w.out_features):
      raise ValueError('residual shape mismatch')
  ws = None
  if k_parts > 1:
    ws = torch.empty((k_parts, M, w.N), dtype=torch.float32, device=a.device)
  _lib.call('t5d_gemm_tiled', _s(), _lib.dtype_code(a.dtype), w.w_dtype,
            _lib.dtype_code(out_dtype), a.data_ptr(), w.data.data_ptr(),
            _lib.ptr(w.scales), _lib.ptr(residual), out.data_ptr(), M, K, w.N,
            epi, _lib.ptr(ws), int(mp), int(nt), int(k_parts))
  return out


def block_cached_value(v):
  """[R, H, 64, L] value (or key) cache -> the blocked [R, H, L/32, 64, 32]
  layout (same bytes count; L a multiple of 32)."""
  R, H, D, L = v.shape
  return v.reshape(R, H, D, L // 32, 32).permute(0, 1, 3, 2, 4).contiguous()


def unblock_cached_value(v):
  """Inverse of block_cached_value: [R, H, L/32, 64, 32] (or the same memory
  viewed as [R, H, 64, L]) -> [R, H, 64, L]."""
  R, H = v.shape[:2]
  L = v.numel() // (R * H * 64)
  return v.reshape(R, H, L // 32, 64, 32).permute(0, 1, 3, 2, 4).reshape(
      R, H, 64, L)


def tail_cached_key(k):
  """[R, H, 64, L] key cache -> the decode loops' [R, H, L + 32, 64]
  (position-major; the last 32 rows are unused)."""
  R, H, D, L = k.shape
  out = k.new_zeros((R, H, L + 32, D))
  out[:, :, :L] = k.transpose(2, 3)
  return out


def untail_cached_key(k):
  """Inverse of tail_cached_key -> [R, H, 64, L]."""
  return k[:, :, :-32].transpose(2, 3).contiguous()


def tail_cached_value(v, n):
  """[R, H, 64, L] value cache holding n positions -> the decode loops'
  [R, H, L/32 + 1, 64, 32]: the finished blocks of 32 positions, and in the
  last block the n % 32 positions of the block being filled as [32, 64]
  position-major."""
  R, H, D, L = v.shape
  n = int(n)
  out = v.new_zeros((R, H, L // 32 + 1, D, 32))
  full = n // 32
  out[:, :, :full] = block_cached_value(v)[:, :, :full]
  rest = n - 32 * full
  if rest:
    tail = out[:, :, -1].reshape(R, H, 32, D)  # a view: same memory
    tail[:, :, :rest] = v[:, :, :, 32 * full:n].transpose(2, 3)
  return out


def untail_cached_value(v, n):
  """Inverse of tail_cached_value for a cache holding n positions ->
  [R, H, 64, L]; positions n and beyond read zero."""
  R, H = v.shape[:2]
  v = v.reshape(R, H, -1, 64, 32)
  L = (v.shape[2] - 1) * 32
  n = int(n)
  full = min(n // 32, L // 32)
  out = v.new_zeros((R, H, 64, L))
  if full:
    out[:, :, :, :32 * full] = unblock_cached_value(
        v[:, :, :full].contiguous())
  rest = n - 32 * full
  if rest > 0 and full < L // 32:
    tail = v[:, :, -1].reshape(R, H, 32, 64)
    out[:, :, :, 32 * full:n] = tail[:, :, :rest].transpose(2, 3)
  return out


def self_attention_step(qkv, cached_key, cached_value, rel_bias, cache_index,
                        out=None, pending_src=None, value_blocked=False,
                        pending_dst=None, key_blocked=False, tail=False):
  """One cached self-attention step; with pending_src [B, beams] the rows'
  caches are first gathered from their source beams inside the kernel, into
  slot e of row (b, e) or, with pending_dst [B, beams], into slot
  pending_dst[b, e].  value_blocked: cached_value holds the blocked layout
  (see block_cached_value) in a tensor of the usual [R, H, 64, L] shape;
  key_blocked (with value_blocked): cached_key as well.  tail: both caches in
  the decode loops' layout (tail_cached_key / tail_cached_value), as tensors
  of [R, H, 64, L + 32] elements."""
  if key_blocked and not value_blocked:
    raise ValueError('key_blocked goes with value_blocked')
  if tail and (value_blocked or key_blocked):
    raise ValueError('tail is a layout of its own')
  _chk(qkv, 'qkv', ndim=2)
  _chk(rel_bias, 'rel_bias', qkv.dtype, 2)
  _chk(cache_index, 'cache_index', torch.int32)
  if tail:
    _chk(cached_key, 'cached_key', qkv.dtype)
    _chk(cached_value, 'cached_value', qkv.dtype)
    R, H = cached_key.shape[:2]
    D = 64
    L = cached_key.numel() // (R * H * D) - 32
    if cached_value.numel() != cached_key.numel() or L <= 0 or L % 32:
      raise ValueError('tail layout: both caches hold [R, H, (L + 32) * 64] '
                       'elements, L a multiple of 32')
  else:
    _chk(cached_key, 'cached_key', qkv.dtype, 4)
    _chk(cached_value, 'cached_value', qkv.dtype, 4)
    R, H, D, L = cached_key.shape
  if D != 64:
    raise ValueError('head_dim must be 64')
  if not tail and cached_value.shape != cached_key.shape:
    raise ValueError('cached_key / cached_value shapes differ')
  if tuple(qkv.shape) != (R, 3 * H * D):
    raise ValueError(f'qkv shape {tuple(qkv.shape)} != {(R, 3 * H * D)}')
  if tuple(rel_bias.shape) != (H, L):
    raise ValueError(f'rel_bias shape {tuple(rel_bias.shape)} != {(H, L)}')
  if cache_index.numel() != 1:
    raise ValueError('cache_index must be a scalar')
  if out is None:
    out = torch.empty((R, H * D), dtype=qkv.dtype, device=qkv.device)
  _chk(out, 'out', qkv.dtype, 2)
  if pending_src is not None or value_blocked or tail:
    B, beams = R, 1
    if pending_src is not None:
      _chk(pending_src, 'pending_src', torch.int32, 2)
      B, beams = pending_src.shape
      if B * beams != R:
        raise ValueError(f'pending_src {(B, beams)} does not cover {R} rows')
    if pending_dst is not None:
      _chk(pending_dst, 'pending_dst', torch.int32, 2)
      if pending_src is None or pending_dst.shape != pending_src.shape:
        raise ValueError('pending_dst goes with a pending_src of its shape')
    _lib.call('t5d_self_attention_step_gather', _s(),
              _lib.dtype_code(qkv.dtype), qkv.data_ptr(),
              cached_key.data_ptr(), cached_value.data_ptr(),
              rel_bias.data_ptr(), cache_index.data_ptr(), out.data_ptr(), B,
              beams, H, L, _lib.ptr(pending_src), _lib.ptr(pending_dst),
              3 if tail else 2 if key_blocked else int(bool(value_blocked)))
    return out
  _lib.call('t5d_self_attention_step', _s(), _lib.dtype_code(qkv.dtype),
            qkv.data_ptr(), cached_key.data_ptr(), cached_value.data_ptr(),
            rel_bias.data_ptr(), cache_index.data_ptr(), out.data_ptr(), R, H,
            L)
  return out


def tile_cross_key(k):
  """[B, H, E, 64] keys -> the bfloat16 kernels' [B, H, 2, E, 32] (the two
  halves of the head dim as planes).  E must be a multiple of 32."""
  B, H, E, D = k.shape
  return k.reshape(B, H, E, 2, 32).permute(0, 1, 3, 2, 4).contiguous()


def tile_cross_value(v):
  """[B, H, 64, E] values -> the bfloat16 kernels' [B, H, E/32, 64, 32]
  (blocks of 32 positions).  E must be a multiple of 32."""
  B, H, D, E = v.shape
  return v.reshape(B, H, D, E // 32, 32).permute(0, 1, 3, 2, 4).contiguous()


def _cross_kv_dims(cross_key, cross_value):
  """(B, H, E) of a cross K/V pair in the layout of its dtype: float32
  [B, H, E, 64] / [B, H, 64, E]; bfloat16 [B, H, 2, E, 32] /
  [B, H, E/32, 64, 32]."""
  if cross_key.dtype == torch.float32:
    _chk(cross_key, 'cross_key', torch.float32, 4)
    _chk(cross_value, 'cross_value', torch.float32, 4)
    B, H, E, D = cross_key.shape
    if D != 64 or tuple(cross_value.shape) != (B, H, D, E):
      raise ValueError(f'float32 cross_key must be [B, H, E, 64] and '
                       f'cross_value [B, H, 64, E], got '
                       f'{tuple(cross_key.shape)} / {tuple(cross_value.shape)}')
    return B, H, E
  _chk(cross_key, 'cross_key', torch.bfloat16, 5)
  _chk(cross_value, 'cross_value', torch.bfloat16, 5)
  B, H, two, E, w = cross_key.shape
  if (two, w) != (2, 32) or E % 32 or tuple(cross_value.shape) != (
      B, H, E // 32, 64, 32):
    raise ValueError(f'bfloat16 cross_key must be [B, H, 2, E, 32] and '
                     f'cross_value [B, H, E/32, 64, 32] (E %% 32 == 0), got '
                     f'{tuple(cross_key.shape)} / {tuple(cross_value.shape)}')
  return B, H, E


def cross_attention_units(enc_len, H, E, out=None):
  """The work order of the bfloat16 cross-attention launches for a batch with
  these valid lengths: int32 [B * H] (t5d_cross_attention_units)."""
  _chk(enc_len, 'enc_len', torch.int32, 1)
  B = enc_len.shape[0]
  if out is None:
    out = torch.empty((B * H,), dtype=torch.int32, device=enc_len.device)
  _chk(out, 'units', torch.int32, 1)
  if out.shape[0] != B * H:
    raise ValueError(f'units must have {B * H} entries')
  _lib.call('t5d_cross_attention_units', _s(), enc_len.data_ptr(), B, H, E,
            out.data_ptr())
  return out


def _units_ptr(units, B, H):
  if units is None:
    return None
  _chk(units, 'units', torch.int32, 1)
  if units.shape[0] != B * H:
    raise ValueError(f'units must have {B * H} entries')
  return units.data_ptr()


def cross_attention_step(q, cross_key, cross_value, enc_len, beams, out=None,
                         units=None):
  _chk(q, 'q', ndim=2)
  _chk(cross_key, 'cross_key', q.dtype)
  _chk(enc_len, 'enc_len', torch.int32, 1)
  B, H, E = _cross_kv_dims(cross_key, cross_value)
  D = 64
  if tuple(q.shape) != (B * beams, H * D):
    raise ValueError(f'q shape {tuple(q.shape)} != {(B * beams, H * D)}')
  if enc_len.shape[0] != B:
    raise ValueError('enc_len length mismatch')
  if out is None:
    out = torch.empty_like(q)
  _chk(out, 'out', q.dtype, 2)
  _lib.call('t5d_cross_attention_step', _s(), _lib.dtype_code(q.dtype),
            q.data_ptr(), cross_key.data_ptr(), cross_value.data_ptr(),
            enc_len.data_ptr(), out.data_ptr(), B, beams, H, E,
            _units_ptr(units, B, H))
  return out


def cross_attention_step_norm_q(x, ln_scale, wq: PackedWeight, cross_key,
                                cross_value, enc_len, beams, out=None,
                                eps=1e-6, units=None):
  """rmsnorm(x, ln_scale) @ wq followed by cross_attention_step, one kernel."""
  _chk(x, 'x', torch.bfloat16, 2)
  _chk(ln_scale, 'ln_scale', torch.bfloat16, 1)
  _chk(cross_key, 'cross_key', x.dtype)
  _chk(enc_len, 'enc_len', torch.int32, 1)
  B, H, E = _cross_kv_dims(cross_key, cross_value)
  D = 64
  R, d = x.shape
  if R != B * beams or ln_scale.shape[0] != d or enc_len.shape[0] != B:
    raise ValueError('x / ln_scale / enc_len do not match the batch')
  if wq.K != d or wq.N != H * D or wq.geglu:
    raise ValueError(f'query kernel must be [{d}, {H * D}]')
  if out is None:
    out = torch.empty((R, H * D), dtype=x.dtype, device=x.device)
  _chk(out, 'out', x.dtype, 2)
  _lib.call('t5d_cross_attention_step_norm_q', _s(), _lib.dtype_code(x.dtype),
            wq.w_dtype, x.data_ptr(), ln_scale.data_ptr(), float(eps),
            wq.data.data_ptr(), cross_key.data_ptr(), cross_value.data_ptr(),
            enc_len.data_ptr(), out.data_ptr(), B, beams, H, E, d,
            _units_ptr(units, B, H))
  return out


def gemm_rows(a, w: PackedWeight, out=None, residual=None,
              layout=_lib.OUT_ROWS, E=0, Ep=0, tile=0):
  """Dense layer over any number of rows (bfloat16).  layout OUT_HEADS_KEY /
  OUT_HEADS_VALUE writes [B, H, 2, Ep, 32] / [B, H, Ep/32, 64, 32] (rows
  m = b*E + e; Ep a multiple of 32, positions e >= E stay zero).  tile: 0 =
  chosen from the shape, 1 = 256 x 128, 2 = 256 x 256, 3 = 256 x 192
  (t5d_gemm_rows_tiled)."""
  _chk(a, 'a', torch.bfloat16, 2)
  M, K = a.shape
  if K != w.K or w.w_dtype == F32:
    raise ValueError(f'a is [{M}, {K}]; kernel K={w.K}, packed weights only')
  epi = EPI_GEGLU if w.geglu else (EPI_RESIDUAL if residual is not None
                                   else EPI_NONE)
  if layout == _lib.OUT_ROWS:
    if out is None:
      out = torch.empty((M, w.out_features), dtype=a.dtype, device=a.device)
    if tuple(out.shape) != (M, w.out_features):
      raise ValueError(f'out shape {tuple(out.shape)}')
  else:
    B, H = M // max(E, 1), w.N // 64
    want = ((B, H, 2, Ep, 32) if layout == _lib.OUT_HEADS_KEY else
            (B, H, Ep // 32, 64, 32))
    if out is None:
      # positions e >= E are not written: they start at zero (none if Ep == E)
      make = torch.empty if Ep == E else torch.zeros
      out = make(want, dtype=a.dtype, device=a.device)
    if tuple(out.shape) != want:
      raise ValueError(f'out shape {tuple(out.shape)} != {want}')
  _chk(out, 'out', a.dtype)
  if residual is not None:
    _chk(residual, 'residual', a.dtype, 2)
    if tuple(residual.shape) != (M, w.N):
      raise ValueError('residual shape mismatch')
  _lib.call('t5d_gemm_rows_tiled', _s(), w.w_dtype, a.data_ptr(),
            w.data.data_ptr(), _lib.ptr(w.scales), _lib.ptr(residual),
            out.data_ptr(), M, K, w.N, epi, int(layout), int(E), int(Ep),
            int(tile))
  return out


def _valid_bits(valid_bits, B, E):
  if valid_bits is None:
    return None
  _chk(valid_bits, 'valid_bits', torch.int32, 2)
  if tuple(valid_bits.shape) != (B, (E + 31) // 32):
    raise ValueError(f'valid_bits {tuple(valid_bits.shape)}, expected '
                     f'{(B, (E + 31) // 32)}')
  return valid_bits.data_ptr()


def pack_valid_bits(valid):
  """[B, E] bool -> [B, (E + 31) / 32] int32 words, bit e % 32 of word e / 32
  = valid[b, e] (what the encoder attention kernels take as valid_bits)."""
  B, E = valid.shape
  words = (E + 31) // 32
  padded = torch.zeros((B, words * 32), dtype=torch.int64, device=valid.device)
  padded[:, :E] = valid.to(torch.int64)
  weights = (1 << torch.arange(32, device=valid.device, dtype=torch.int64))
  packed = (padded.view(B, words, 32) * weights).sum(-1)
  packed = torch.where(packed >= 2**31, packed - 2**32, packed)
  return packed.to(torch.int32).contiguous()


def encoder_attention(q, k, v_t, rel_bias, enc_len, out=None, valid_bits=None,
                      variant=0):
  """q, k: [B*E, >= H*64] row-major views (row stride = stride(0)); v_t
  [B, H, Ep/32, 64, 32] (tile_cross_value of [B, H, 64, Ep]); rel_bias
  [H, 2E-1]; enc_len [B]; valid_bits: None or pack_valid_bits of the
  per-position mask -> out [B*E, H*64].  variant: 0 = chosen from E, 1 / 2 =
  the kernel that forms the scores twice / keeps them in registers
  (t5d_encoder_attention_variant)."""
  _chk(v_t, 'v_t', torch.bfloat16, 5)
  _chk(rel_bias, 'rel_bias', torch.bfloat16, 2)
  _chk(enc_len, 'enc_len', torch.int32, 1)
  B, H, blocks, D, w = v_t.shape
  if w != 32:
    raise ValueError('v_t must be [B, H, Ep/32, 64, 32]')
  Ep = blocks * 32
  E = (rel_bias.shape[1] + 1) // 2
  for name, t in (('q', q), ('k', k)):
    if (not t.is_cuda or t.dtype != torch.bfloat16 or t.dim() != 2 or
        t.stride(1) != 1 or t.shape[0] != B * E or t.shape[1] != H * 64):
      raise ValueError(f'{name} must be a [B*E, H*64] bfloat16 view with unit '
                       f'column stride, got {tuple(t.shape)}')
  if D != 64 or rel_bias.shape[0] != H or enc_len.shape[0] != B:
    raise ValueError('v_t [B, H, Ep/32, 64, 32], rel_bias [H, 2E-1], '
                     'enc_len [B]')
  if out is None:
    out = torch.empty((B * E, H * 64), dtype=torch.bfloat16, device=v_t.device)
  _chk(out, 'out', torch.bfloat16, 2)
  _lib.call('t5d_encoder_attention_variant', _s(), q.data_ptr(), k.data_ptr(),
            v_t.data_ptr(), rel_bias.data_ptr(), enc_len.data_ptr(),
            _valid_bits(valid_bits, B, E), out.data_ptr(), B, H, E, Ep,
            q.stride(0), k.stride(0), int(variant))
  return out


def encoder_attention_f32(qkv, rel_bias, enc_len, H, out=None,
                          valid_bits=None):
  """float32 encoder self-attention from the fused projection: qkv
  [B*E, 3*H*64] (q | k | v), rel_bias [H, 2E-1], enc_len [B], valid_bits as
  encoder_attention -> [B*E, H*64]."""
  _chk(qkv, 'qkv', torch.float32, 2)
  _chk(rel_bias, 'rel_bias', torch.float32, 2)
  _chk(enc_len, 'enc_len', torch.int32, 1)
  B = enc_len.shape[0]
  E = (rel_bias.shape[1] + 1) // 2
  if (tuple(qkv.shape) != (B * E, 3 * H * 64) or rel_bias.shape[0] != H or
      rel_bias.shape[1] != 2 * E - 1):
    raise ValueError(f'qkv {tuple(qkv.shape)} / rel_bias {tuple(rel_bias.shape)}'
                     f' do not match B={B}, E={E}, H={H}')
  if out is None:
    out = torch.empty((B * E, H * 64), dtype=torch.float32, device=qkv.device)
  _chk(out, 'out', torch.float32, 2)
  _lib.call('t5d_encoder_attention_f32', _s(), qkv.data_ptr(),
            rel_bias.data_ptr(), enc_len.data_ptr(),
            _valid_bits(valid_bits, B, E), out.data_ptr(), B, H, E)
  return out


def add_i32(x, delta):
  _chk(x, 'x', torch.int32)
  _lib.call('t5d_add_i32', _s(), x.data_ptr(), x.numel(), int(delta))
  return x


def cache_gather_beams(cache, beam_indices, valid_len=None, valid_offset=0,
                       n_tensors=1, tensor_stride_bytes=0):
  """In-place gather of [.., B, beams, inner.., L] cache tensors.

  `cache` is [B, beams, ..., L] (n_tensors == 1) or the first of n_tensors
  such tensors spaced tensor_stride_bytes apart."""
  _chk(cache, 'cache')
  _chk(beam_indices, 'beam_indices', torch.int32, 2)
  B, beams = beam_indices.shape
  if cache.shape[0] != B or cache.shape[1] != beams:
    raise ValueError(f'cache {tuple(cache.shape)} vs indices {(B, beams)}')
  L = cache.shape[-1]
  inner = 1
  for s in cache.shape[2:-1]:
    inner *= s
  if valid_len is not None:
    _chk(valid_len, 'valid_len', torch.int32)
  _lib.call('t5d_cache_gather_beams', _s(), cache.data_ptr(),
            int(tensor_stride_bytes), int(n_tensors), cache.element_size(), B,
            beams, inner, L, beam_indices.data_ptr(), _lib.ptr(valid_len),
            int(valid_offset))
  return cache


def gather_beams(x, beam_indices, out=None):
  """out[b, e] = x[b, beam_indices[b, e]] (out of place)."""
  _chk(x, 'x')
  _chk(beam_indices, 'beam_indices', torch.int32, 2)
  B, new_beams = beam_indices.shape
  if x.dim() < 2 or x.shape[0] != B:
    raise ValueError(f'x {tuple(x.shape)} vs indices {(B, new_beams)}')
  old_beams = x.shape[1]
  inner = x[0, 0].numel() * x.element_size()
  if out is None:
    out = torch.empty((B, new_beams) + tuple(x.shape[2:]), dtype=x.dtype,
                      device=x.device)
  if inner == 0 or B == 0:
    return out
  _lib.call('t5d_gather_beams', _s(), x.data_ptr(), out.data_ptr(),
            beam_indices.data_ptr(), B, old_beams, new_beams, inner)
  return out


def top_k(x, k):
  _chk(x, 'x', torch.float32, 2)
  rows, n = x.shape
  vals = torch.empty((rows, k), dtype=torch.float32, device=x.device)
  idx = torch.empty((rows, k), dtype=torch.int32, device=x.device)
  _lib.call('t5d_top_k', _s(), x.data_ptr(), vals.data_ptr(), idx.data_ptr(),
            rows, n, k)
  return vals, idx


def beam_topk(logits, live_logprobs, k, bufs=None):
  """-> (topk_vals [B, k], topk_idx [B, k], row_max [R], row_lse [R])."""
  _chk(logits, 'logits', torch.float32, 2)
  _chk(live_logprobs, 'live_logprobs', torch.float32, 2)
  B, beams = live_logprobs.shape
  R, V = logits.shape
  if R != B * beams:
    raise ValueError(f'logits rows {R} != {B}*{beams}')
  dev = logits.device
  if bufs is None:
    bufs = (torch.empty((B, k), dtype=torch.float32, device=dev),
            torch.empty((B, k), dtype=torch.int32, device=dev),
            torch.empty((R,), dtype=torch.float32, device=dev),
            torch.empty((R,), dtype=torch.float32, device=dev),
            torch.empty((2 * R * k,), dtype=torch.int32, device=dev))
  vals, idx, row_max, row_lse, scratch = bufs
  _lib.call('t5d_beam_topk', _s(), logits.data_ptr(), live_logprobs.data_ptr(),
            vals.data_ptr(), idx.data_ptr(), row_max.data_ptr(),
            row_lse.data_ptr(), scratch.data_ptr(), B, beams, V, k)
  return vals, idx, row_max, row_lse


class BeamBuffers:
  """Device arrays of one BeamState (t5x/decoding.py:1002-1021)."""

  def __init__(self, B, K, S, device):
    self.B, self.K, self.S = B, K, S
    self.cur_index = torch.zeros((), dtype=torch.int32, device=device)
    self.live_logprobs = torch.zeros((B, K), dtype=torch.float32,
                                     device=device)
    self.finished_scores = torch.zeros((B, K), dtype=torch.float32,
                                       device=device)
    self.live_seqs = torch.zeros((B, K, S), dtype=torch.int32, device=device)
    self.finished_seqs = torch.zeros((B, K, S), dtype=torch.int32,
                                     device=device)
    self.finished_flags = torch.zeros((B, K), dtype=torch.uint8, device=device)
    self._ptrs = _lib.BeamStatePtrs(
        self.cur_index.data_ptr(), self.live_logprobs.data_ptr(),
        self.finished_scores.data_ptr(), self.live_seqs.data_ptr(),
        self.finished_seqs.data_ptr(), self.finished_flags.data_ptr())

  def ptrs(self):
    return ctypes.byref(self._ptrs)


def beam_update(cur: BeamBuffers, nxt: BeamBuffers, topk_vals, topk_idx,
                inputs, initial_index, brevity, top_alive_indices, V, eos_id):
  _chk(topk_vals, 'topk_vals', torch.float32, 2)
  _chk(topk_idx, 'topk_idx', torch.int32, 2)
  _chk(inputs, 'inputs', torch.int32, 2)
  _chk(initial_index, 'initial_index', torch.int32, 1)
  _chk(brevity, 'brevity', torch.float32, 1)
  _chk(top_alive_indices, 'top_alive_indices', torch.int32, 2)
  B, K, S = cur.B, cur.K, cur.S
  if tuple(topk_vals.shape) != (B, 2 * K) or topk_idx.shape != topk_vals.shape:
    raise ValueError('top-k buffers must be [B, 2K]')
  if inputs.shape[0] != B or initial_index.shape[0] != B:
    raise ValueError('inputs / initial_index batch mismatch')
  if tuple(top_alive_indices.shape) != (B, K):
    raise ValueError('top_alive_indices must be [B, K]')
  _lib.call('t5d_beam_update', _s(), cur.ptrs(), nxt.ptrs(),
            topk_vals.data_ptr(), topk_idx.data_ptr(), inputs.data_ptr(),
            initial_index.data_ptr(), brevity.data_ptr(),
            top_alive_indices.data_ptr(), B, K, S, inputs.shape[1], V,
            int(eos_id))


def beam_cond(state: BeamBuffers, min_brevity, min_log_prob, max_decode_step,
              min_initial_index, keep_going):
  _chk(keep_going, 'keep_going', torch.int32)
  _lib.call('t5d_beam_cond', _s(), state.ptrs(), state.B, state.K, state.S,
            float(min_brevity), float(min_log_prob), int(max_decode_step),
            int(min_initial_index), keep_going.data_ptr())


def sample_tokens_workspace(R, device):
  """Scratch memory that lets sample_tokens cut a top-k choice into two
  launches (t5d_sample_tokens_workspace_bytes)."""
  n = int(_lib.load().t5d_sample_tokens_workspace_bytes(int(R)))
  return torch.empty(((n + 3) // 4,), dtype=torch.int32, device=device)


def sample_tokens(logits, gumbel, temperature, topk, topp, rescale, tokens=None,
                  logprobs=None, workspace=None):
  _chk(logits, 'logits', torch.float32, 2)
  _chk(temperature, 'temperature', torch.float32, 1)
  R, V = logits.shape
  if temperature.shape[0] != R:
    raise ValueError('temperature must be [R]')
  if gumbel is not None:
    _chk(gumbel, 'gumbel', torch.float32, 2)
    if gumbel.shape != logits.shape:
      raise ValueError('gumbel shape mismatch')
  if tokens is None:
    tokens = torch.empty((R,), dtype=torch.int32, device=logits.device)
  if logprobs is None:
    logprobs = torch.empty((R,), dtype=torch.float32, device=logits.device)
  if workspace is not None:
    _chk(workspace, 'workspace', torch.int32, 1)
    need = int(_lib.load().t5d_sample_tokens_workspace_bytes(R))
    if workspace.numel() * 4 < need:
      raise ValueError(f'workspace of {workspace.numel() * 4} bytes, need {need}')
  _lib.call('t5d_sample_tokens', _s(), logits.data_ptr(), _lib.ptr(gumbel),
            temperature.data_ptr(), tokens.data_ptr(), logprobs.data_ptr(), R,
            V, int(topk), float(topp), int(bool(rescale)),
            _lib.ptr(workspace))
  return tokens, logprobs


def sample_update(tokens, token_logprobs, sequences, cur_index, cur_token,
                  ended, log_prob, max_decode_len, initial_eos_count,
                  all_ended, eos_id):
  R, S = sequences.shape
  for t, name, dt in ((tokens, 'tokens', torch.int32),
                      (token_logprobs, 'token_logprobs', torch.float32),
                      (sequences, 'sequences', torch.int32),
                      (cur_index, 'cur_index', torch.int32),
                      (cur_token, 'cur_token', torch.int32),
                      (ended, 'ended', torch.uint8),
                      (log_prob, 'log_prob', torch.float32),
                      (max_decode_len, 'max_decode_len', torch.int32),
                      (initial_eos_count, 'initial_eos_count', torch.int32),
                      (all_ended, 'all_ended', torch.int32)):
    _chk(t, name, dt)
    if name not in ('sequences', 'all_ended') and t.numel() != R:
      raise ValueError(f'{name} must have {R} elements')
  _lib.call('t5d_sample_update', _s(), tokens.data_ptr(),
            token_logprobs.data_ptr(), sequences.data_ptr(),
            cur_index.data_ptr(), cur_token.data_ptr(), ended.data_ptr(),
            log_prob.data_ptr(), max_decode_len.data_ptr(),
            initial_eos_count.data_ptr(), all_ended.data_ptr(), R, S,
            int(eos_id))
