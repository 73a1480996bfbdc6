"""The host loop around `predict_batch`: `get_infer_fn` of t5x/utils.py:1543-1817.

Takes an enumerated dataset of `(index, example)` pairs, pads it to a multiple
of the batch size with copies of the first example under index -1
(:1649-1662), takes this host's shard and batches it (:1664-1667), runs
`infer_step` per batch with a per-batch split of the rng (:1684-1687), then
concatenates, drops the pads (:1526-1540), restores dataset order by index
(:1766-1767) and returns `[(index, inference)]`, plus the aux dict when
`infer_step` returns `(inferences, aux)` (:1769-1815).

One process drives one GPU here, so "partitioning" reduces to the data layout
(`shard_id`, `num_shards`) the optional partitioner reports; the
`infer_step` signature is inspected exactly as the reference does
(:1584-1603).  Datasets are anything sized and iterable (a list of pairs, or an
object with `as_numpy_iterator()` such as a tf.data.Dataset).
"""

import collections
import functools
import inspect
import itertools
from typing import Any, Callable, Mapping, Optional, Sequence

import numpy as np


def _to_numpy(x):
  if hasattr(x, 'detach'):  # torch tensor, possibly on the device
    x = x.detach()
    if x.is_floating_point() and x.element_size() == 2:
      x = x.float()
    return x.cpu().numpy()
  return np.asarray(x)


def tree_map(fn, tree, *rest):
  """Structure-preserving map over dicts / lists / tuples (jax.tree.map)."""
  if isinstance(tree, Mapping):
    return {k: tree_map(fn, v, *[r[k] for r in rest]) for k, v in tree.items()}
  if isinstance(tree, tuple):
    return tuple(tree_map(fn, v, *[r[i] for r in rest])
                 for i, v in enumerate(tree))
  if isinstance(tree, list):
    return [tree_map(fn, v, *[r[i] for r in rest]) for i, v in enumerate(tree)]
  return fn(tree, *rest)


def _remove_padding(all_inferences, all_indices):
  """t5x/utils.py:1526-1540."""
  keep = np.where(all_indices >= 0)
  return tree_map(lambda x: x[keep], all_inferences), all_indices[keep]


def split_rng(rng):
  """`step_rng, rng = jax.random.split(rng)` for the rng kinds this package
  accepts: an object with `split()` (returning two such objects) or a NumPy
  SeedSequence / int seed.  The reference's threefry stream is not
  reproduced (no vector of it is held by the reference's tests)."""
  if hasattr(rng, 'split'):
    return tuple(rng.split())
  seq = rng if isinstance(rng, np.random.SeedSequence) else (
      np.random.SeedSequence(int(rng)))
  step, nxt = seq.spawn(2)
  return step, nxt


def _iterate(ds):
  if hasattr(ds, 'as_numpy_iterator'):
    return ds.as_numpy_iterator()
  return iter(ds)


def _stack(examples):
  return tree_map(lambda *xs: np.stack([np.asarray(x) for x in xs]),
                  examples[0], *examples[1:])


def map_in_flight(begin, items, in_flight: int, max_unclaimed: int = 16):
  """begin(item) for every item of an iterable, with up to `in_flight` of the
  returned objects running at once, yielding their result() in the order of
  the items.  An object has poll(block=False) -> bool (has it ended; waits
  only when asked to) and result().  What has ended is collected at once —
  which frees whatever it holds for the next item — also when an older one is
  still running, so one slow item does not idle the others' places; at most
  `max_unclaimed` results wait for an older item that way."""
  in_flight = max(1, int(in_flight))
  todo = iter(items)
  pending = collections.deque()   # [object or None once collected, result]

  def collect():
    for entry in pending:
      if entry[0] is not None and entry[0].poll():
        entry[1] = entry[0].result()
        entry[0] = None

  def running():
    return [e[0] for e in pending if e[0] is not None]

  exhausted = False
  while True:
    collect()
    while pending and pending[0][0] is None:
      yield pending.popleft()[1]
    if exhausted and not pending:
      return
    active = running()
    if (not exhausted and len(active) < in_flight and
        len(pending) < in_flight + max_unclaimed):
      try:
        item = next(todo)
      except StopIteration:
        exhausted = True
        continue
      pending.append([begin(item), None])
      continue
    # nothing to start: wait for the oldest one running (the others keep
    # their chunks enqueued ahead and are looked at right after)
    active[0].poll(block=True)


def _defined_at(obj, name):
  """Position in type(obj)'s method resolution order of the class that defines
  `name` (0: the most derived class); None if no class does."""
  for depth, cls in enumerate(type(obj).__mro__):
    if name in vars(cls):
      return depth
  return None


def _begin_of(infer_step):
  """`begin_<name>` of the object whose bound method `infer_step` is (through
  functools.partial wrappers), with the wrappers' arguments bound again: the
  variant of the step that returns, without waiting, an object with poll() and
  result().  None when there is no such variant, and also when a subclass has
  overridden the step (or a method the variant stands for, listed in its
  `stands_for`) without overriding the variant: the override is then what the
  reference's `infer_step(params, batch, rng)` contract calls, and the
  inherited variant would bypass it."""
  fn, args, kwargs = infer_step, (), {}
  while isinstance(fn, functools.partial):
    args, kwargs = fn.args + args, {**fn.keywords, **kwargs}
    fn = fn.func
  owner, name = getattr(fn, '__self__', None), getattr(fn, '__name__', '')
  begin = getattr(owner, 'begin_' + name, None)
  if begin is None or not inspect.ismethod(fn) or not inspect.ismethod(begin):
    return None
  begin_depth = _defined_at(owner, 'begin_' + name)
  if begin_depth is None:
    return None
  for covered in getattr(begin, 'stands_for', (name,)):
    depth = _defined_at(owner, covered)
    if depth is None or depth < begin_depth:
      return None
  return functools.partial(begin, *args, **kwargs)


def get_infer_fn(infer_step: Callable, batch_size: int,
                 train_state_axes: Any = None, partitioner: Any = None,
                 keep_aux_as_numpy: bool = False,
                 decodes_in_flight: Optional[int] = None):
  """t5x/utils.py:1543-1817 -> infer_fn(ds, train_state, rng=None).

  `decodes_in_flight` (no counterpart in the reference): when `infer_step` is
  `predict_batch` / `predict_batch_with_aux` of a model that can start a
  prediction without waiting for it, up to that many batches decode on the
  device at once (each holds its own caches and cross K/V); each batch's
  result is unchanged.  None: what the model's batches_in_flight() says for
  the first batch; 1: one batch after the other, as the reference."""
  del train_state_axes  # one device: parameters are not partitioned
  params_of_step = inspect.signature(infer_step).parameters
  takes_rng = 'rng' in params_of_step
  takes_mutables = 'flax_mutables' in params_of_step

  if partitioner is not None:
    layout = partitioner.get_data_layout(batch_size)
    shard_id, num_shards = layout.shard_id, layout.num_shards
    if num_shards != 1:
      # In the reference the partitioned step returns the de-sharded global
      # batch on every host; with one process and one GPU there is one shard.
      raise NotImplementedError(
          f'get_infer_fn: {num_shards} data shards; this build drives one GPU '
          'from one process (one shard)')
  else:
    shard_id, num_shards = 0, 1
  per_shard_batch_size = batch_size // num_shards

  def infer_fn(ds, train_state, rng=None):
    try:
      original_ds_length = len(ds)
    except TypeError as e:
      raise TypeError('infer dataset length is unknown.') from e
    examples = list(_iterate(ds))
    remainder = original_ds_length % batch_size
    if remainder:
      # Pad with the first example under index -1 (:1649-1662).
      examples = examples + [(np.int64(-1), examples[0][1])] * (
          batch_size - remainder)
    shard = examples[shard_id::num_shards]
    n_batches = len(shard) // per_shard_batch_size  # drop_remainder=True

    batched_results, all_indices = [], []
    params = getattr(train_state, 'params', train_state)
    mutables = getattr(train_state, 'flax_mutables', None)
    begin = _begin_of(infer_step) if decodes_in_flight != 1 else None
    if takes_mutables or 'rng' not in params_of_step:
      begin = None
    n_in_flight = decodes_in_flight

    def batches():
      nonlocal rng
      for i in range(n_batches):
        chunk = shard[i * per_shard_batch_size:(i + 1) * per_shard_batch_size]
        index = np.asarray([c[0] for c in chunk], dtype=np.int64)
        infer_batch = _stack([c[1] for c in chunk])
        if rng is None:
          step_rng = None
        else:
          step_rng, rng = split_rng(rng)
        all_indices.append(index)
        yield infer_batch, step_rng

    todo = batches()
    if begin is not None and n_in_flight is None and n_batches:
      first = next(todo)
      ask = getattr(begin.func.__self__, 'batches_in_flight', None)
      n_in_flight = (ask(first[0], begin.keywords.get('num_decodes'))
                     if ask is not None else 1)
      todo = itertools.chain([first], todo)
    if begin is not None and (n_in_flight or 1) > 1:
      batched_results.extend(map_in_flight(
          lambda b: begin(params, b[0], b[1], in_flight=True), todo,
          n_in_flight))
    else:
      # Results stay on the device until everything is enqueued; the copies
      # below are what the reference's copy_to_host_async overlaps.
      for infer_batch, step_rng in todo:
        kwargs = {'flax_mutables': mutables} if takes_mutables else {}
        if takes_rng:
          batched_results.append(infer_step(params, infer_batch, step_rng,
                                            **kwargs))
        else:
          batched_results.append(infer_step(params, infer_batch, **kwargs))

    batched_results = [tree_map(_to_numpy, r) for r in batched_results]
    all_inferences = tree_map(lambda *xs: np.concatenate(xs),
                              batched_results[0], *batched_results[1:])
    indices = np.concatenate(all_indices)
    all_inferences, indices = _remove_padding(all_inferences, indices)
    # Undo the shard interleave: order by dataset index (:1766-1767).
    all_inferences = tree_map(lambda x: x[indices], all_inferences)
    indices = indices[indices]

    aux_values = None
    if (isinstance(all_inferences, tuple) and len(all_inferences) == 2 and
        isinstance(all_inferences[1], Mapping)):
      all_inferences, aux_values = all_inferences

    leaves, rebuild = _flatten(all_inferences)
    per_example = [rebuild([np.array(leaf[i]).tolist() for leaf in leaves])
                   for i in range(len(indices))]
    indices_and_outputs = list(zip(indices.tolist(), per_example))
    if len(indices_and_outputs) != original_ds_length:
      raise ValueError(
          'Size of indices_and_outputs does not match length of original '
          'dataset: %d versus %d' % (len(indices_and_outputs),
                                     original_ds_length))
    if aux_values is None:
      return indices_and_outputs
    if keep_aux_as_numpy:
      aux_values = tree_map(lambda x: list(np.array(x)), aux_values)
    else:
      aux_values = tree_map(lambda x: np.array(x).tolist(), aux_values)
    return indices_and_outputs, aux_values

  return infer_fn


def _flatten(tree):
  """Leaves of a pytree and a function rebuilding the same structure from a
  list of replacement leaves (jax.tree_util.tree_flatten / tree_unflatten)."""
  leaves = []

  def collect(node):
    if isinstance(node, Mapping):
      return {k: collect(node[k]) for k in sorted(node)}
    if isinstance(node, (tuple, list)):
      return type(node)(collect(v) for v in node)
    leaves.append(node)
    return len(leaves) - 1

  skeleton = collect(tree)

  def rebuild(new_leaves: Sequence[Any]):
    def fill(node):
      if isinstance(node, Mapping):
        return {k: fill(v) for k, v in node.items()}
      if isinstance(node, (tuple, list)):
        return type(node)(fill(v) for v in node)
      return new_leaves[node]
    return fill(skeleton)

  return leaves, rebuild
