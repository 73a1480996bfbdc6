"""The C-ABI library loads and exports every entry point include/*.h
declare (no compute calls: this runs without a GPU)."""

import ctypes
import os
import re

import pytest

from t5x_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_names():
  inc = os.path.join(ROOT, 'include')
  text = ''.join(open(os.path.join(inc, f)).read()
                 for f in sorted(os.listdir(inc)) if f.endswith('.h'))
  text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
  return sorted(set(re.findall(r'\b(t5d_[a-z0-9_]+)\s*\(', text)))


def test_header_declares_entry_points():
  names = declared_names()
  assert 't5d_gemm' in names and 't5d_self_attention_step' in names
  assert len(names) >= 18


def test_library_exports_every_declared_symbol():
  if not os.path.exists(_lib.LIB_PATH):
    pytest.fail(f'{_lib.LIB_PATH} not built: run __graft_entry__.build()')
  lib = ctypes.CDLL(_lib.LIB_PATH)
  missing = [n for n in declared_names() if not hasattr(lib, n)]
  assert not missing, missing


def test_binding_covers_every_declared_symbol():
  assert set(declared_names()) == set(_lib.exported_names())


def test_measurement_aids_stay_out_of_the_boundary():
  """The work-skipping switch bench.py uses lives in its own header and entry
  point; the boundary's structs and declarations carry none."""
  boundary = open(os.path.join(ROOT, 'include', 't5d.h')).read()
  assert 'leave_out' not in boundary and 'LEAVE_OUT' not in boundary
  aids = open(os.path.join(ROOT, 'include', 't5d_measure.h')).read()
  assert 't5d_measure_leave_out' in aids
  if not os.path.exists(_lib.LIB_PATH):
    pytest.fail(f'{_lib.LIB_PATH} not built: run __graft_entry__.build()')
  assert hasattr(ctypes.CDLL(_lib.LIB_PATH), 't5d_measure_leave_out')
  assert _lib.measure_leave_out(0) == 0
  # no product module calls it
  pkg = os.path.join(ROOT, 't5x_amd')
  users = [f for f in os.listdir(pkg) if f.endswith('.py') and
           'measure_leave_out(' in open(os.path.join(pkg, f)).read()]
  assert sorted(users) == ['_lib.py', 'network.py']  # iteration_graph only


def test_static_entry_point_calls_no_allocator():
  """Source check: neither the entry point nor its address look-up names an
  allocating or freeing HIP call."""
  src = open(os.path.join(ROOT, 't5x_amd', 'csrc', 'select.hip')).read()
  start = src.index('static int static_topk_scratch(')
  entry = src.index('extern "C" int t5d_beam_topk_static(')
  end = src.index('\n}\n', entry)
  body = src[start:end]
  assert 'hipGetSymbolAddress' in body
  assert not re.search(r'hipMalloc|hipFree|hipMallocAsync|hipHostMalloc|'
                       r'hipExtMalloc|hipMemPool', body)


def test_version_and_error_string_without_gpu():
  lib = _lib.load()
  assert lib.t5d_version() == 1
  # shape validation happens on the host before any launch
  assert lib.t5d_packed_weight_bytes(_lib.BF16, 768, 2304) == 768 * 2304 * 2
  assert lib.t5d_packed_weight_bytes(_lib.I8, 768, 2304) == 768 * 2304
  assert lib.t5d_packed_weight_bytes(_lib.BF16, 40, 32) == -1
  rc = lib.t5d_rmsnorm(None, 7, None, None, None, 1, 1, 1e-6)
  assert rc == -1
  assert b'dtype' in lib.t5d_last_error()


def test_many_row_tile_choice_without_gpu():
  """t5d_gemm_rows_tile: which workgroup tile the many-row dense kernel runs a
  shape on (1: 256 x 128, 2: 256 x 256, 3: 256 x 192), by the rounds of
  workgroups on 256 CUs.  The T5.1.1-base encoder over 32 x 512 positions:"""
  lib = _lib.load()
  pick = lambda M, K, N, w=_lib.BF16: lib.t5d_gemm_rows_tile(w, M, K, N)
  assert pick(16384, 768, 768) == 3     # 192 tiles of 256 x 256, 256 of 256 x 192
  assert pick(16384, 2048, 768) == 3
  assert pick(16384, 768, 4096) == 2    # 4 full rounds of 256 x 256
  assert pick(16384, 768, 1536) == 3    # 2 rounds of 512 tiles of 256 x 192
  assert pick(16384, 4096, 4096) == 2
  assert pick(300, 96, 80) == 1         # one small workgroup
  # int8 weights and K < 64 run on the staging-register kernel: 256 x 128
  assert pick(16384, 768, 768, _lib.I8) == 1
  assert pick(16384, 32, 768) == 1


def test_product_path_has_no_cpu_fallback():
  import torch
  if torch.cuda.is_available():
    pytest.skip('GPU present')
  from t5x_amd import decoding
  with pytest.raises(RuntimeError, match='no CPU fallback'):
    decoding.beam_search([[0, 0]], {}, lambda s: None, 1)


def test_product_does_not_import_oracle():
  pkg = os.path.join(ROOT, 't5x_amd')
  for dirpath, _, files in os.walk(pkg):
    for f in files:
      if f.endswith('.py'):
        src = open(os.path.join(dirpath, f)).read()
        assert not re.search(r'^\s*(from|import)\s+oracle\b', src, re.M), f
