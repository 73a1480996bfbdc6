"""The build's check that no kernel reads a matrix instruction's result too
early (t5x_amd/csrc/check_mfma_reads.py): unit tests on small listings, and
the check itself on the assembly that `make check` has written, when it is
there."""

import glob
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, 't5x_amd', 'csrc')


def _checker():
  spec = importlib.util.spec_from_file_location(
      'check_mfma_reads', os.path.join(CSRC, 'check_mfma_reads.py'))
  mod = importlib.util.module_from_spec(spec)
  spec.loader.exec_module(mod)
  return mod


_STRAIGHT = """
_Z6kernelv:
	v_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]
	v_mov_b32_e32 v10, v11
	s_nop 6
	v_accvgpr_read_b32 v12, a3
	s_endpgm
"""

# the fall-through side is long enough, the taken side is 4 slots
_TAKEN_SIDE_SHORT = """
_Z6kernelv:
	v_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]
	s_cbranch_vccnz .LBB0_2
	v_mov_b32_e32 v3, 0
	ds_read_b32 v3, v3 offset:25600
	s_mov_b64 s[8:9], 0
	s_waitcnt lgkmcnt(0)
	v_lshrrev_b32_e32 v3, 16, v3
	s_branch .LBB0_3
.LBB0_2:
	s_mov_b64 s[8:9], -1
.LBB0_3:
	s_nop 0
	v_accvgpr_read_b32 v29, a3
	s_endpgm
"""

_CHAIN_THEN_STORE = """
_Z6kernelv:
	v_mfma_f32_16x16x32_bf16 v[0:3], v[8:11], v[12:15], 0
	v_mfma_f32_16x16x32_bf16 v[0:3], v[16:19], v[20:23], v[0:3]
	s_nop 1
	global_store_dwordx4 v[30:31], v[0:3], off
	s_endpgm
"""

_OVERWRITTEN = """
_Z6kernelv:
	v_mfma_f32_16x16x32_bf16 v[0:3], v[8:11], v[12:15], 0
	v_mov_b32_e32 v0, 0
	v_add_f32_e32 v5, v0, v0
	s_endpgm
"""


def test_straight_line_with_padding_passes():
  found, hist = _checker().short_reads(_STRAIGHT)
  assert found == [] and hist == {9: 1}


def test_taken_side_of_a_branch_is_followed():
  found, _ = _checker().short_reads(_TAKEN_SIDE_SHORT)
  assert len(found) == 1
  kernel, mfma, slots, reader = found[0]
  assert kernel == '_Z6kernelv' and slots == 4
  assert reader.startswith('v_accvgpr_read_b32 v29, a3')


def test_matrix_chain_is_interlocked_but_its_store_is_a_reader():
  found, _ = _checker().short_reads(_CHAIN_THEN_STORE)
  # the second v_mfma may follow at once; the store 3 slots after it may not
  assert [(f[2], f[3].split()[0]) for f in found] == [(3, 'global_store_dwordx4')]


def test_overwritten_result_is_not_a_read():
  found, hist = _checker().short_reads(_OVERWRITTEN)
  assert found == [] and not hist


_RING_GUARDED = """
_Z6kernelv:
	global_load_lds_dwordx4 v[4:5], off
.LBB0_1:
	ds_read_b128 v[0:3], v8
	s_cbranch_scc1 .LBB0_3
	s_waitcnt vmcnt(2) lgkmcnt(0)
	s_branch .LBB0_4
.LBB0_3:
	s_waitcnt vmcnt(0) lgkmcnt(0)
.LBB0_4:
	s_add_i32 s6, s33, 4
	s_barrier
	global_load_lds_dwordx4 v[4:5], off
	s_cbranch_scc0 .LBB0_1
	s_endpgm
"""

# the operand read after the last full wait reaches the barrier unwaited
_RING_SUNK_READ = """
_Z6kernelv:
	global_load_lds_dwordx4 v[4:5], off
	s_waitcnt vmcnt(0) lgkmcnt(0)
	ds_read_b128 v[0:3], v8
	s_waitcnt vmcnt(2)
	s_barrier
	global_load_lds_dwordx4 v[4:5], off
	s_waitcnt lgkmcnt(0)
	s_endpgm
"""

_NO_DMA = """
_Z6kernelv:
	ds_read_b128 v[0:3], v8
	s_barrier
	s_endpgm
"""


def test_barriers_of_kernels_that_load_into_lds_need_a_wait_for_lds_reads():
  mod = _checker()
  assert mod.unguarded_barriers(_RING_GUARDED) == []
  assert mod.unguarded_barriers(_RING_SUNK_READ) == [('_Z6kernelv', 1)]
  assert mod.unguarded_barriers(_NO_DMA) == []   # other kernels: not checked


def test_built_kernels_have_no_early_read():
  files = sorted(glob.glob(os.path.join(CSRC, 'isa', '*.s')))
  if not files:
    pytest.skip('no assembly here: `make -C t5x_amd/csrc check` writes it')
  mod = _checker()
  for path in files:
    with open(path) as f:
      found, _ = mod.short_reads(f.read())
    assert found == [], (path, found[:3])
    assert mod.unguarded_barriers(open(path).read()) == [], path
