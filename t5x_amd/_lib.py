"""ctypes binding of libt5d.so (the HIP kernels behind include/t5d.h).

There is no fallback: if the shared library has not been built, anything that
needs a kernel raises.  Pointers are passed as plain integers
(`tensor.data_ptr()`), the stream as the current torch stream's handle.
"""

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_float, c_int, c_int32,
                    c_int64, c_uint, c_uint8, c_void_p)

F32, BF16, I8 = 0, 1, 2
EPI_NONE, EPI_RESIDUAL, EPI_GEGLU = 0, 1, 2
OUT_ROWS, OUT_HEADS_KEY, OUT_HEADS_VALUE = 0, 1, 2
LEAVE_OUT_CROSS_ATTENTION, LEAVE_OUT_SELF_ATTENTION = 1, 2

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'csrc', 'libt5d.so')


class BeamStatePtrs(Structure):
  """t5d_beam_state."""
  _fields_ = [('cur_index', c_void_p), ('live_logprobs', c_void_p),
              ('finished_scores', c_void_p), ('live_seqs', c_void_p),
              ('finished_seqs', c_void_p), ('finished_flags', c_void_p)]


class Layer(Structure):
  """t5d_layer."""
  _fields_ = [(n, c_void_p) for n in (
      'ln_self', 'qkv', 'self_out', 'ln_cross', 'cross_q', 'cross_out',
      'ln_mlp', 'wi', 'wo', 'qkv_scales', 'self_out_scales', 'cross_q_scales',
      'cross_out_scales', 'wi_scales', 'wo_scales', 'cached_key',
      'cached_value', 'cross_key', 'cross_value')]


class ModelStep(Structure):
  """t5d_model_step."""
  _fields_ = ([(n, c_int) for n in (
      'dtype', 'w_dtype', 'd', 'H', 'F', 'V', 'L', 'E', 'NL', 'R', 'B',
      'beams')] + [(n, c_void_p) for n in (
          'embedding', 'rel_bias', 'ln_final', 'logits_w', 'logits_scales')] +
              [('layers', POINTER(Layer))] + [(n, c_void_p) for n in (
                  'cache_index', 'enc_len', 'cross_units', 'x', 'x1', 'x2',
                  'xn', 'qkv', 'q',
                  'ao', 'h', 'logits', 'gate', 'pending_src',
                  'pending_dst')] +
              [('value_blocked', c_int)])


class BeamStep(Structure):
  """t5d_beam_step."""
  _fields_ = ([('state', BeamStatePtrs)] + [(n, c_void_p) for n in (
      'inputs', 'initial_index', 'brevity', 'top_alive', 'topk_vals',
      'topk_idx', 'row_max', 'row_lse', 'scratch', 'ids', 'keep_going')] +
              [('S', c_int), ('Lin', c_int), ('eos_id', c_int),
               ('min_brevity', c_float), ('min_log_prob', c_float),
               ('max_decode_step', c_int), ('min_initial_index', c_int),
               ('kv_base', c_void_p), ('kv_tensor_stride_bytes', c_int64),
               ('n_kv_tensors', c_int), ('skip_cond', c_int),
               ('cache_slot', c_void_p), ('cache_src', c_void_p),
               ('cache_dst', c_void_p)])


class SampleStep(Structure):
  """t5d_sample_step."""
  _fields_ = ([(n, c_void_p) for n in (
      'sequences', 'cur_index', 'cur_token', 'ended', 'log_prob',
      'max_decode_len', 'initial_eos_count', 'temperature', 'gumbel')] +
              [('noise_ring', c_int)] + [(n, c_void_p) for n in (
                  'step_count', 'tokens', 'token_logprobs', 'workspace',
                  'all_ended', 'keep_going')] +
              [('S', c_int), ('eos_id', c_int), ('topk', c_int),
               ('rescale', c_int), ('topp', c_float)])


_P = c_void_p
_SIGNATURES = {
    't5d_gather_step_ids': (c_int, [_P, _P, _P, _P, c_int, c_int]),
    't5d_decoder_step': (c_int, [_P, POINTER(ModelStep), _P]),
    't5d_beam_search_step': (c_int, [_P, POINTER(ModelStep),
                                     POINTER(BeamStep)]),
    't5d_temperature_sample_step': (c_int, [_P, POINTER(ModelStep),
                                            POINTER(SampleStep)]),
    't5d_graph_begin': (c_int, [_P]),
    't5d_graph_end': (c_int, [_P, POINTER(c_void_p)]),
    't5d_graph_launch': (c_int, [_P, _P]),
    't5d_graph_destroy': (c_int, [_P]),
    't5d_version': (c_int, []),
    't5d_measure_leave_out': (c_int, [c_int]),
    't5d_measure_fill': (c_int, [_P, _P, c_int64, c_uint, c_int]),
    't5d_measure_read': (c_int, [_P, _P, c_int64, c_int, c_int, _P, c_int]),
    't5d_last_error': (c_char_p, []),
    't5d_packed_weight_bytes': (c_int64, [c_int, c_int, c_int]),
    't5d_pack_weight': (c_int, [_P, c_int, _P, _P, _P, c_int, c_int, c_int]),
    't5d_embed': (c_int, [_P, c_int, _P, _P, _P, c_int, c_int, c_int]),
    't5d_rmsnorm': (c_int, [_P, c_int, _P, _P, _P, c_int, c_int, c_float]),
    't5d_gemm_workspace_bytes': (c_int64, [c_int] * 5),
    't5d_gemm': (c_int, [_P, c_int, c_int, c_int, _P, _P, _P, _P, _P, c_int,
                         c_int, c_int, c_int, _P, _P]),
    't5d_encoder_attention': (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int,
                                      c_int, c_int, c_int, c_int, c_int]),
    't5d_encoder_attention_variant': (c_int, [_P, _P, _P, _P, _P, _P, _P, _P,
                                              c_int, c_int, c_int, c_int,
                                              c_int, c_int, c_int]),
    't5d_encoder_attention_f32': (c_int, [_P, _P, _P, _P, _P, _P, c_int,
                                          c_int, c_int]),
    't5d_gemm_rows': (c_int, [_P, c_int, _P, _P, _P, _P, _P, c_int64, c_int,
                              c_int, c_int, c_int, c_int, c_int]),
    't5d_gemm_rows_tiled': (c_int, [_P, c_int, _P, _P, _P, _P, _P, c_int64,
                                    c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_int]),
    't5d_gemm_rows_tile': (c_int, [c_int, c_int64, c_int, c_int]),
    't5d_gemm_tiled': (c_int, [_P, c_int, c_int, c_int, _P, _P, _P, _P, _P,
                               c_int, c_int, c_int, c_int, _P, c_int, c_int,
                               c_int]),
    't5d_norm_gemm': (c_int, [_P, c_int, c_int, c_int, _P, _P, c_float, _P, _P,
                              _P, c_int, c_int, c_int, c_int]),
    't5d_self_attention_step': (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P,
                                        c_int, c_int, c_int]),
    't5d_self_attention_step_gather': (c_int, [_P, c_int, _P, _P, _P, _P, _P,
                                               _P, c_int, c_int, c_int, c_int,
                                               _P, _P, c_int]),
    't5d_cross_attention_step': (c_int, [_P, c_int, _P, _P, _P, _P, _P, c_int,
                                         c_int, c_int, c_int, _P]),
    't5d_cross_attention_units': (c_int, [_P, _P, c_int, c_int, c_int, _P]),
    't5d_cross_attention_step_norm_q': (c_int, [_P, c_int, c_int, _P, _P,
                                                c_float, _P, _P, _P, _P, _P,
                                                c_int, c_int, c_int, c_int,
                                                c_int, _P]),
    't5d_add_i32': (c_int, [_P, _P, c_int, c_int]),
    't5d_cache_gather_beams': (c_int, [_P, _P, c_int64, c_int, c_int, c_int,
                                       c_int, c_int, c_int, _P, _P, c_int]),
    't5d_gather_beams': (c_int, [_P, _P, _P, _P, c_int, c_int, c_int,
                                 c_int64]),
    't5d_top_k': (c_int, [_P, _P, _P, _P, c_int, c_int, c_int]),
    't5d_beam_topk': (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int,
                              c_int, c_int]),
    't5d_beam_topk_static': (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int,
                                     c_int, c_int]),
    't5d_beam_update': (c_int, [_P, POINTER(BeamStatePtrs),
                                POINTER(BeamStatePtrs), _P, _P, _P, _P, _P, _P,
                                c_int, c_int, c_int, c_int, c_int, c_int]),
    't5d_beam_cond': (c_int, [_P, POINTER(BeamStatePtrs), c_int, c_int, c_int,
                              c_float, c_float, c_int, c_int, _P]),
    't5d_sample_tokens_workspace_bytes': (c_int64, [c_int]),
    't5d_sample_tokens': (c_int, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int,
                                  c_float, c_int, _P]),
    't5d_sample_update': (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,
                                  c_int, c_int, c_int]),
}

_lib = None


class T5DError(RuntimeError):
  pass


def load():
  """Loads libt5d.so once and declares every entry point's signature."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise T5DError(
        f'{LIB_PATH} is missing: build the HIP kernels first '
        '(python -c "import __graft_entry__ as g; g.build()" or '
        '`make -C t5x_amd/csrc`). There is no CPU fallback.')
  lib = ctypes.CDLL(LIB_PATH)
  for name, (restype, argtypes) in _SIGNATURES.items():
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = argtypes
  _lib = lib
  return lib


def exported_names():
  return sorted(_SIGNATURES)


def measure_leave_out(mask: int) -> int:
  """t5d_measure_leave_out (include/t5d_measure.h, a measurement aid that is
  not part of the boundary): sets the calling thread's mask of kernel
  families that fused steps are enqueued without; returns the previous one."""
  return int(load().t5d_measure_leave_out(int(mask)))


def last_error() -> str:
  return load().t5d_last_error().decode('utf-8', 'replace')


def call(name, *args):
  """Calls entry point `name`; raises on a non-zero status."""
  rc = getattr(load(), name)(*args)
  if rc != 0:
    msg = last_error()
    if rc == -1:
      raise ValueError(msg)
    raise T5DError(f'{name} failed ({rc}): {msg}')


def stream_handle():
  import torch
  return torch.cuda.current_stream().cuda_stream


def ptr(t):
  """Device pointer of a torch tensor (None -> NULL)."""
  return None if t is None else t.data_ptr()


def dtype_code(torch_dtype):
  import torch
  if torch_dtype == torch.float32:
    return F32
  if torch_dtype == torch.bfloat16:
    return BF16
  if torch_dtype == torch.int8:
    return I8
  raise ValueError(f'unsupported dtype {torch_dtype}')
