"""The C-ABI library loads and exports every entry point include/t5d.h
declares (no compute calls: this runs without a GPU)."""

import ctypes
import os
import re

import pytest

from t5x_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_names():
  text = open(os.path.join(ROOT, 'include', 't5d.h')).read()
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
