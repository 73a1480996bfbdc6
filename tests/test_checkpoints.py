"""T5X checkpoint reader (t5x/checkpoints.py:1803-1958) against the reference's
own checkpoint fixtures: `tiny_t5/checkpoint_1` (TensorStore/zarr leaves, copied
as data under tests/golden/) and, when the reference tree is present,
`test_t5_tiny.checkpoint_0` (inline msgpack arrays; 4 MB, read in place).  The
reference holds no expected VALUES for either, so values are pinned through
what the format fixes (dtype, shape, chunk grid, fill value) and a chunked
array written here and read back; the parameter names and shapes are those of
`get_t5_test_model` (t5x/test_utils.py:181-195)."""

import gzip
import os

import msgpack
import numpy as np
import pytest

from t5x_amd import checkpoints

HERE = os.path.dirname(os.path.abspath(__file__))
TINY_T5 = os.path.join(HERE, 'golden', 'tiny_t5')
REF_TINY = '/root/reference/t5x/testdata/test_t5_tiny.checkpoint_0'


def test_find_checkpoint_accepts_model_dir_step_dir_and_file():
  f = os.path.join(TINY_T5, 'checkpoint_1', 'checkpoint')
  assert checkpoints.find_checkpoint(TINY_T5) == f            # latest step
  assert checkpoints.find_checkpoint(TINY_T5, step=1) == f
  assert checkpoints.find_checkpoint(os.path.join(TINY_T5, 'checkpoint_1')) == f
  assert checkpoints.find_checkpoint(f) == f
  assert checkpoints.all_steps(TINY_T5) == [1]
  with pytest.raises(ValueError, match='Path is not a valid checkpoint'):
    checkpoints.find_checkpoint(TINY_T5, step=7)
  with pytest.raises(ValueError, match='Path is not a valid checkpoint'):
    checkpoints.find_checkpoint(os.path.join(TINY_T5, 'nope'))


def test_zarr_leaves_of_the_reference_fixture():
  state = checkpoints.load_t5x_checkpoint(TINY_T5)
  assert set(state) == {'state', 'target'} and state['target'] == {}
  ps = state['state']['param_states']
  # dtype and shape are what each leaf's TensorStore spec declares
  assert ps['bias'].dtype == np.float32 and ps['bias'].shape == (5,)
  assert ps['kernel'].dtype == np.float64 and ps['kernel'].shape == (10, 5)
  assert ps['step'].dtype == np.int32 and ps['step'].shape == ()
  assert int(state['state']['step']) == 1 and int(ps['step']) == 1
  np.testing.assert_array_equal(ps['bias'], np.ones(5, np.float32))
  k = ps['kernel']
  assert np.all((k > 0) & (k < 1)) and len(np.unique(k)) == 50
  # the chunk really is the gzip of the C-order buffer
  raw = gzip.decompress(open(os.path.join(
      TINY_T5, 'checkpoint_1', 'state.param_states.kernel', '0.0'), 'rb').read())
  assert raw == k.tobytes()


def _write_zarr(dirname, arr, chunks, skip=()):
  os.makedirs(dirname)
  grid = [range((s + c - 1) // c) for s, c in zip(arr.shape, chunks)]
  import itertools
  for idx in itertools.product(*grid):
    if idx in skip:
      continue
    block = np.zeros(chunks, arr.dtype)
    sel = tuple(slice(i * c, min((i + 1) * c, s))
                for i, c, s in zip(idx, chunks, arr.shape))
    part = arr[sel]
    block[tuple(slice(0, n) for n in part.shape)] = part
    with open(os.path.join(dirname, '.'.join(map(str, idx))), 'wb') as f:
      f.write(gzip.compress(block.tobytes()))


def test_chunked_arrays_edge_chunks_and_absent_chunks(tmp_path):
  rs = np.random.RandomState(0)
  arr = rs.randn(7, 10, 3).astype(np.float32)
  ck = tmp_path / 'checkpoint_5'
  _write_zarr(str(ck / 'target.w'), arr, (4, 4, 3), skip={(1, 2, 0)})
  spec = {'driver': 'zarr', 'dtype': 'float32',
          'kvstore': {'driver': 'file', 'path': 'target.w/'},
          'metadata': {'chunks': [4, 4, 3], 'shape': [7, 10, 3],
                       'compressor': {'id': 'gzip', 'level': 1}}}
  tree = {'version': 3, 'optimizer': {
      'state': {'step': 5}, 'target': {'w': spec, 'b': 2}}}
  (ck / 'checkpoint').write_bytes(msgpack.packb(tree))
  got = checkpoints.load_t5x_checkpoint(str(tmp_path))
  want = arr.copy()
  want[4:, 8:, :] = 0          # the absent chunk reads as fill_value 0
  np.testing.assert_array_equal(got['target']['w'], want)
  assert got['target']['b'] == 2 and got['state']['step'] == 5
  # restore_dtype casts target only
  got = checkpoints.load_t5x_checkpoint(str(tmp_path), restore_dtype=np.float64)
  assert got['target']['w'].dtype == np.float64 and got['state']['step'] == 5


def test_old_versions_are_refused(tmp_path):
  (tmp_path / 'checkpoint').write_bytes(msgpack.packb({'version': 1}))
  with pytest.raises(ValueError, match='earlier than 2 are not supported'):
    checkpoints.load_t5x_checkpoint(str(tmp_path / 'checkpoint'))


def test_inline_msgpack_arrays_bfloat16_and_scalars(tmp_path):
  def nd(a, code=1):
    return msgpack.ExtType(code, msgpack.packb(
        (list(a.shape), a.dtype.name, a.tobytes())))
  w = np.arange(6, dtype=np.float32).reshape(2, 3)
  bits = np.array([0x3F80, 0xC000, 0x3DCD], np.uint16)  # 1, -2, ~0.1 in bf16
  tree = {'version': 3, 'optimizer': {'state': {'step': nd(np.int32(9), 3)},
                                      'target': {
      'w': nd(w),
      'h': msgpack.ExtType(1, msgpack.packb(([3], 'bfloat16', bits.tobytes())))}}}
  (tmp_path / 'checkpoint').write_bytes(msgpack.packb(tree))
  got = checkpoints.load_t5x_checkpoint(str(tmp_path / 'checkpoint'))
  np.testing.assert_array_equal(got['target']['w'], w)
  np.testing.assert_array_equal(
      got['target']['h'], (bits.astype(np.uint32) << 16).view(np.float32))
  assert got['state']['step'] == 9


@pytest.mark.skipif(not os.path.exists(REF_TINY),
                    reason='reference testdata not present')
def test_reference_tiny_checkpoint_tree_and_a_decode_with_it():
  params = checkpoints.load_params(REF_TINY)
  # get_t5_test_model: emb 8, 4 heads x head_dim 3, mlp 16, 2 + 2 layers
  assert params['token_embedder']['embedding'].shape == (32128, 8)
  dec = params['decoder']
  assert sorted(dec) == ['decoder_norm', 'layers_0', 'layers_1',
                         'logits_dense', 'relpos_bias']
  assert dec['relpos_bias']['rel_embedding'].shape == (4, 32)
  assert dec['logits_dense']['kernel'].shape == (8, 32128)
  l0 = dec['layers_0']
  for name in ('self_attention', 'encoder_decoder_attention'):
    for proj in ('query', 'key', 'value'):
      assert l0[name][proj]['kernel'].shape == (8, 12)
    assert l0[name]['out']['kernel'].shape == (12, 8)
  assert l0['mlp']['wi_0']['kernel'].shape == (8, 16)
  assert l0['mlp']['wo']['kernel'].shape == (16, 8)
  for leaf in (l0['pre_mlp_layer_norm']['scale'],
               params['encoder']['encoder_norm']['scale']):
    assert leaf.dtype == np.float32 and leaf.shape == (8,)
  # the tree drives the oracle model end to end
  from oracle import decoding as odec
  from oracle import models as omodels
  from oracle import t5 as ot5
  cfg = ot5.T5Config(vocab_size=32128, dtype='float32', emb_dim=8, num_heads=4,
                     num_encoder_layers=2, num_decoder_layers=2, head_dim=3,
                     mlp_dim=16)
  model = omodels.EncoderDecoderModel(omodels.Transformer(cfg),
                                      decode_fn=odec.beam_search)
  batch = {'encoder_input_tokens': np.array([[5, 9, 13, 0]], np.int32),
           'decoder_input_tokens': np.zeros((1, 5), np.int32)}
  out, aux = model.predict_batch_with_aux(params, batch, num_decodes=2)
  assert out.shape == (1, 5) and np.isfinite(aux['scores']).all()
