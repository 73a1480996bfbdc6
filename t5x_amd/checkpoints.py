"""Reader for T5X checkpoints (`load_t5x_checkpoint`, t5x/checkpoints.py:1835-1958).

On disk a checkpoint is a directory `checkpoint_<step>/` holding a msgpack
file `checkpoint` (:1967) whose tree is
`{'version': int, 'optimizer': {'state': ..., 'target': ...}}` (:1887-1892).
A leaf is either an inline array — flax's msgpack extension type 1, a packed
`(shape, dtype name, bytes)` tuple; type 3 is a NumPy scalar in the same
packing, type 2 a complex number — or a dict that is a TensorStore spec
(`{'driver': 'zarr', 'kvstore': {'path': ...}, 'metadata': {...}}`) pointing at
a sibling directory (:1894-1905).  Such an array is stored as zarr v2 chunks:
one file per chunk named by its chunk coordinates joined with '.', C order,
compressed as `metadata.compressor` says (gzip here), edge chunks padded to
the full chunk shape.

Only non-executing decoders touch the file (msgpack, gzip/zlib, numpy
frombuffer).  `restore_dtype` casts `target` only, like the reference
(:1951-1952); nothing else of the checkpointing system (saving, datasets,
Orbax, partitioned reads) is provided.
"""

import glob
import gzip
import itertools
import os
import re
import zlib
from typing import Any, Optional

import msgpack
import numpy as np

_CHECKPOINT_FILE = 'checkpoint'  # t5x/checkpoints.py:1967


def _ext_hook(code, data):
  """flax.serialization's msgpack extension types."""
  if code == 1:  # ndarray: (shape, dtype name, buffer)
    shape, dtype_name, buf = msgpack.unpackb(data, raw=False)
    if dtype_name == 'bfloat16':
      # kept exact: widen the 16 stored bits to float32
      u = np.frombuffer(buf, dtype=np.uint16).astype(np.uint32) << 16
      return u.view(np.float32).reshape(shape)
    return np.frombuffer(buf, dtype=np.dtype(dtype_name)).reshape(shape).copy()
  if code == 2:  # native complex
    re_, im = msgpack.unpackb(data, raw=False)
    return complex(re_, im)
  if code == 3:  # numpy scalar, packed like an array
    shape, dtype_name, buf = msgpack.unpackb(data, raw=False)
    return np.frombuffer(buf, dtype=np.dtype(dtype_name)).reshape(shape)[()]
  return msgpack.ExtType(code, data)


def all_steps(checkpoints_dir: str):
  """t5x/checkpoints_utils.py:40-46."""
  pat = re.compile(r'.*/checkpoint_(\d+)$')
  hits = [pat.match(p) for p in glob.glob(
      os.path.join(checkpoints_dir, 'checkpoint_*'))]
  return sorted(int(m.group(1)) for m in hits if m)


def latest_step(checkpoints_dir: str) -> Optional[int]:
  """t5x/checkpoints_utils.py:60-65."""
  steps = all_steps(checkpoints_dir)
  return steps[-1] if steps else None


def find_checkpoint(path: str, step: Optional[int] = None) -> str:
  """t5x/checkpoints.py:1803-1832: `path` may be the model dir, a
  `checkpoint_<step>` dir, or the msgpack file itself."""
  path = os.fspath(path)
  if os.path.isdir(path):
    step = latest_step(path) if step is None else step
    if step is not None:
      path = os.path.join(path, f'checkpoint_{step}')
    path = os.path.join(path, _CHECKPOINT_FILE)
  if not os.path.exists(path) or os.path.isdir(path):
    raise ValueError(f'Path is not a valid checkpoint: {path}')
  return path


def _is_ts_spec(node) -> bool:
  return isinstance(node, dict) and 'driver' in node and 'kvstore' in node


def _decompress(raw: bytes, compressor) -> bytes:
  if compressor is None:
    return raw
  cid = compressor.get('id')
  if cid == 'gzip':
    return gzip.decompress(raw)
  if cid == 'zlib':
    return zlib.decompress(raw)
  raise NotImplementedError(f'zarr compressor {cid!r} is not supported')


def read_zarr_array(spec: dict, ckpt_dir: str) -> np.ndarray:
  """Reads the whole array a TensorStore zarr spec describes."""
  if spec.get('driver') != 'zarr':
    raise NotImplementedError(f"TensorStore driver {spec.get('driver')!r}")
  kv = spec['kvstore']
  rel = kv['path'] if isinstance(kv, dict) else str(kv)
  if isinstance(kv, dict) and kv.get('driver') not in (None, 'file', 'gfile'):
    raise NotImplementedError(
        f"kvstore driver {kv.get('driver')!r}: only local files are read")
  base = rel if os.path.isabs(rel) else os.path.join(ckpt_dir, rel)
  meta = spec['metadata']
  shape = tuple(meta['shape'])
  chunks = tuple(meta['chunks'])
  dtype = np.dtype(spec.get('dtype') or meta.get('dtype'))
  if meta.get('order', 'C') != 'C':
    raise NotImplementedError('only C-order zarr chunks are supported')
  sep = meta.get('dimension_separator', '.')
  fill = meta.get('fill_value', 0) or 0
  out = np.full(shape, fill, dtype=dtype)
  if not shape:  # scalar: a single chunk named '0'
    raw = _decompress(open(os.path.join(base, '0'), 'rb').read(),
                      meta.get('compressor'))
    return np.frombuffer(raw, dtype=dtype)[:1].reshape(())[()].copy()
  grid = [range((s + c - 1) // c) for s, c in zip(shape, chunks)]
  for idx in itertools.product(*grid):
    name = os.path.join(base, sep.join(str(i) for i in idx))
    if not os.path.exists(name):
      continue  # an absent chunk is all fill_value
    raw = _decompress(open(name, 'rb').read(), meta.get('compressor'))
    block = np.frombuffer(raw, dtype=dtype).reshape(chunks)
    sel = tuple(slice(i * c, min((i + 1) * c, s))
                for i, c, s in zip(idx, chunks, shape))
    out[sel] = block[tuple(slice(0, s.stop - s.start) for s in sel)]
  return out


def _restore(node: Any, ckpt_dir: str):
  if _is_ts_spec(node):
    return read_zarr_array(node, ckpt_dir)
  if isinstance(node, dict):
    return {k: _restore(v, ckpt_dir) for k, v in node.items()}
  return node


def _cast(tree, dtype):
  """t5x/checkpoints.py:220-235."""
  if isinstance(tree, dict):
    return {k: _cast(v, dtype) for k, v in tree.items()}
  if isinstance(tree, (int, str)) or not hasattr(tree, 'dtype'):
    return tree
  return tree if tree.dtype == dtype else tree.astype(dtype)


def load_t5x_checkpoint(path: str, step: Optional[int] = None,
                        restore_dtype=None) -> dict:
  """Returns `{'state': ..., 'target': ...}` with NumPy leaves."""
  path = find_checkpoint(path, step)
  with open(path, 'rb') as fp:
    contents = msgpack.unpackb(fp.read(), ext_hook=_ext_hook, raw=False,
                               strict_map_key=False)
  version = contents.get('version', 0)
  if version < 2:
    raise ValueError('Checkpoint versions earlier than 2 are not supported. '
                     f'Got version: {version}')
  state = _restore(contents['optimizer'], os.path.dirname(path))
  if restore_dtype is not None and 'target' in state:
    state['target'] = _cast(state['target'], np.dtype(restore_dtype))
  return state


def load_params(path: str, step: Optional[int] = None) -> dict:
  """The model parameters (`target`) of a checkpoint as float32 arrays, in the
  tree layout `EncoderDecoderModel.predict_batch` takes."""
  return load_t5x_checkpoint(path, step, restore_dtype=np.float32)['target']
