#!/usr/bin/env python3
"""Decode-path benchmark: T5.1.1-base, beam_search with 4 beams, batch 32,
encoder length 512 (rows 128..512 valid), max decode length 128, bf16, on one
MI355X.  Synthetic random-init weights and seeded synthetic tokens.

A "step" is one iteration of the beam-search loop: one decoder forward for the
128 beam rows, log_softmax + top-2K over beam x vocab, beam bookkeeping, cache
reorder and the loop-condition check.  `value` = batch * steps / seconds
(decoded tokens per second: every batch item emits one token per step).  The
encoder output is synthetic and the cross-attention K/V projection, weight
packing and upload happen before the timed region.  An iteration costs more
the later it comes in a decode (self-attention streams the cache filled so
far), so the timed iterations are whole decodes plus, for a remainder or a
step count below the decode length, a window centred on the middle of a fresh
decode (`config.t_first` / `t_last`); decode starts are outside the clock.

Prints ONE JSON line.  `roofline` describes the dominant HBM-bound kernel of
the step, timed live with HIP events on the launch stream; `cpu_baseline` is the
NumPy oracle (a port of the reference algorithm, not the reference itself) on
this host's cores over a bounded sample of the same workload.
"""

import argparse
import functools
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, vendor peak

CONFIGS = {
    # name: (size, batch, decodes per item, enc_len, enc_min_len,
    #        max_decode_len, dtype, weight_dtype, loop)
    # loop: 'beam' or ('sample', temperature, topk)
    'small-fp32-greedy': ('small', 8, 1, 64, 64, 32, 'float32', None,
                          ('sample', 0.0, 0)),
    'base-beam4': ('base', 32, 4, 512, 128, 128, 'bfloat16', None, 'beam'),
    'xl-int8-beam4': ('xl', 16, 4, 512, 512, 128, 'bfloat16', 'int8', 'beam'),
    'large-sample': ('large', 64, 1, 512, 512, 256, 'bfloat16', None,
                     ('sample', 0.7, 40)),
    'xxl-greedy': ('xxl', 128, 1, 1024, 1024, 256, 'bfloat16', None,
                   ('sample', 0.0, 0)),
}
DEFAULT_CONFIG = 'base-beam4'


def parse_args():
  ap = argparse.ArgumentParser()
  ap.add_argument('--gpus', type=int, default=1)
  ap.add_argument('--steps', type=int, default=256)
  ap.add_argument('--warmup', type=int, default=128)
  ap.add_argument('--config', default=DEFAULT_CONFIG, choices=sorted(CONFIGS))
  ap.add_argument('--seed', type=int, default=0)
  ap.add_argument('--hw-queues', type=int, default=8,
                  help='hardware queues of this process (GPU_MAX_HW_QUEUES, '
                       'which the HIP runtime reads when it starts; its own '
                       'default is 4, of which one serves the default stream). '
                       'With 8, four decodes run side by side instead of '
                       'three: what `in_flight` measures; `value`, the single '
                       'batch on two lanes, is the same either way.  0: leave '
                       'the environment as it is')
  ap.add_argument('--no-cpu-baseline', action='store_true')
  ap.add_argument('--lanes', type=int, default=None,
                  help='batch slices stepped concurrently (default: library)')
  ap.add_argument('--stage', default='decode',
                  choices=['decode', 'encoder', 'dense', 'memory'],
                  help="'encoder': the once-per-batch stage before the decode "
                       'loop (encoder forward + cross K/V projection); a step '
                       "is one batch.  'dense': the decoder's dense layers on "
                       'their own, each kind replayed over the layers (a step '
                       'is one pass over every dense layer of the decoder): '
                       "weight streaming rate and matrix-core rate per kind.  "
                       "'memory': what serves a buffer that one kernel wrote "
                       'and the next reads (an XCD\'s own L2, the memory-side '
                       'cache, HBM), for plain streaming kernels and for the '
                       'logits between the vocabulary projection and the '
                       'selection kernel')
  ap.add_argument('--in-flight', type=int, default=None,
                  help='also measure this many whole decodes of different '
                       'batches running on the device at once (default for '
                       'the default config: as many as the device runs side '
                       'by side, 3 with 4 hardware queues; 0 = skip, the '
                       'default for the other configs)')
  ap.add_argument('--replay-roofline', action='store_true',
                  help='time the roofline kernel by back-to-back replay only '
                       '(no decodes enqueued without it); for runs under '
                       'hardware counters, which serialise every dispatch')
  ap.add_argument('--roofline-only', action='store_true',
                  help='only the dominant-kernel replay plus a plain copy of '
                       'known size (for counter runs under rocprofv3 --pmc)')
  ap.add_argument('--counter-copy', action='store_true',
                  help='end the run with a plain device copy of 256 MiB, 5 '
                       'times (for runs under rocprofv3 --pmc: what FETCH_SIZE '
                       '/ WRITE_SIZE read for a copy of known size scales the '
                       "kernels' readings)")
  ap.add_argument('--cpu-steps', type=int, default=6,
                  help='size of the CPU oracle sample: decode steps (batch '
                       'rows with --stage encoder)')
  return ap.parse_args()


class Workload:
  """Synthetic batch + model state for repeated full decodes."""

  def __init__(self, name, seed, lanes=None):
    import torch
    from t5x_amd import decoding, models, network
    self.torch, self.decoding = torch, decoding
    size, B, K, E, Emin, L, dtype, wdt, loop = CONFIGS[name]
    self.name, self.B, self.K, self.E, self.L = name, B, K, E, L
    self.loop_kind, self.seed = loop, seed
    self.cfg = network.t5_1_1_config(size, dtype=dtype, weight_dtype=wdt)
    dev = torch.device('cuda')
    self.params = network.init_params(self.cfg, seed, dev, with_encoder=False)
    self.module = network.Transformer(self.cfg, dev)
    if lanes:
      self.module.decode_lanes = lanes
    self.model = models.EncoderDecoderModel(self.module,
                                            decode_fn=decoding.beam_search)
    rs = np.random.Generator(np.random.PCG64(seed + 1))
    tok = rs.integers(2, 32128, size=(B, E)).astype(np.int32)
    lens = rs.integers(Emin, E + 1, size=(B,))
    tok[np.arange(E)[None, :] >= lens[:, None]] = 0
    self.enc_lens = lens
    self.enc_tokens = torch.as_tensor(tok, device=dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed + 2)
    self.encoded = torch.randn((B, E, self.cfg.emb_dim), generator=gen,
                               device=dev).to(network._TORCH_DTYPE[dtype])
    self.inputs = np.zeros((B, L), np.int32)
    self.tokens_to_logits = models.StepFunction(
        self.model, self.params, network.BeamShared(self.encoded, K),
        network.BeamShared(self.enc_tokens, K), L)
    self.weights = self.module.decoder_weights(self.params)
    self.loop = None
    self.decodes = 0
    self.bf16 = dtype == 'bfloat16'

  def new_decode(self):
    # Drop the finished decode first so that its cache buffers go back to the
    # allocator before the new ones are requested: no hipMalloc per decode.
    self.loop = None
    cache = self.module.init_cache(self.B, self.L)
    if self.loop_kind == 'beam':
      self.loop = self.decoding.BeamLoop(
          self.inputs, cache, self.tokens_to_logits, eos_id=1,
          num_decodes=self.K, alpha=0.6)
    else:
      _, temperature, topk = self.loop_kind
      self.decodes += 1
      self.loop = self.decoding.SampleLoop(
          self.inputs, cache, self.tokens_to_logits, 1,
          self.seed + self.decodes, self.K, temperature, topk,
          use_fused=True)
    if not self.loop.cond():
      raise RuntimeError('fresh decode terminated immediately')

  def prime(self):
    """Set-up, before the warm-up steps: a few iterations of a first decode
    (builds the decode context, captures its graphs, replays each once) and
    of a second (the first pass through the path that re-binds the kept
    context, about 40 ms of one-time work), so that no step count of the
    warm-up leaves either inside the timed region."""
    for _ in range(2):
      self.run_steps(9)
      self.loop = None
    self.torch.cuda.synchronize()

  def run_steps(self, n, timed=False):
    """Runs exactly n loop iterations, starting a new decode whenever the
    current one has produced its max_decode_len tokens.  The loop condition is
    evaluated on the device after every iteration; it is read back once per
    decode (with these random-init weights no decode ends early, which the
    read-back at the end of each decode verifies).

    timed: returns (seconds, windows).  The cost of an iteration grows with
    its position t in the decode (self-attention streams t + 1 cache columns),
    so the timed iterations are whole decodes (t = 0 .. L-1) and, for what is
    left over (or all of it when n < L), a window centred on t = (L-1)/2 of a
    fresh decode, which is advanced to the window's start untimed.  Decode
    starts (cache clear, state initialisation, cross K/V projection: once per
    batch, not part of the step loop) and the end-of-decode read-back are
    outside the clock; every timed segment has a device synchronisation on
    both sides."""
    sync = self.torch.cuda.synchronize
    if timed:
      self.loop = None
    done, seconds, windows = 0, 0.0, []
    while done < n:
      if self.loop is None or self.loop.step >= self.L:
        if self.loop is not None:
          self.check_full_decode()
        self.new_decode()
      take = min(n - done, self.L - self.loop.step)
      if timed and self.loop.step == 0 and take < self.L:
        self.loop.advance((self.L - take) // 2)
      first = self.loop.step
      if timed:
        sync()
        t0 = time.perf_counter()
      self.loop.advance(take)
      if timed:
        sync()
        seconds += time.perf_counter() - t0
        windows.append((first, first + take - 1))
        # A loop flag that had closed would turn every kernel of the window
        # into an early return and the window would read fast: the device's
        # own step count must have advanced by what was timed.
        if self.steps_on_device() != first + take:
          raise RuntimeError(
              f'timed window {first}..{first + take - 1}: the device is at '
              f'step {self.steps_on_device()}, not {first + take}')
      done += take
    if timed and self.loop.step >= self.L:
      self.check_full_decode()
    return seconds, windows

  def steps_on_device(self):
    """Loop iterations the device has completed in the current decode."""
    fused = getattr(self.loop, 'fused', None)
    if self.loop_kind == 'beam':
      if fused is not None:
        fused.synchronize()   # brings the lanes' counter into loop.cur
      return int(self.loop.cur.cur_index.item())
    return int(fused.step_count.item())

  def check_full_decode(self):
    if self.loop.cond():
      raise RuntimeError('decode did not stop at max_decode_len')
    count = self.steps_on_device()
    if count != self.L:
      raise RuntimeError(f'decode stopped early at step {count}; the step '
                         'count of this run would be wrong')

  # -- algorithmic traffic (bytes) of one launch, by kernel ---------------------
  def cross_attention_bytes(self):
    """Algorithmic bytes of one cross-attention launch: the valid K and V
    rows once per batch item (shared by its beams, padded keys skipped), the
    queries in and the attention output out."""
    s = self.encoded.element_size()
    hd = self.cfg.num_heads * self.cfg.head_dim
    R = self.B * self.K
    return int(self.enc_lens.sum()) * hd * 2 * s + 2 * R * hd * s

  def fused_query_bytes(self):
    """What the launch moves on top of that when the pre-attention layer norm
    and the query projection ride inside it: residual-stream rows and the
    norm scale in and the query kernel once, instead of the queries in.  It
    belongs to the dense layers' account, not to the attention's."""
    s = self.encoded.element_size()
    hd = self.cfg.num_heads * self.cfg.head_dim
    d = self.cfg.emb_dim
    R = self.B * self.K
    return R * d * s + d * s + d * hd * s - R * hd * s

  def step_bytes(self):
    """Algorithmic bytes of one loop iteration, averaged over the positions
    of a decode: every decoder weight once, the valid self-attention prefix
    and the valid cross K/V once per batch item per layer, the cache rows
    the beam reorder has to move (none here: beams inherit their parents'
    slots; the reference's gather is not counted), activations."""
    c = self.cfg
    s = self.encoded.element_size()
    wbytes = 1 if c.weight_dtype == 'int8' else s
    d, F, V = c.emb_dim, c.mlp_dim, c.vocab_size
    hd = c.num_heads * c.head_dim
    R, nl = self.B * self.K, c.num_decoder_layers
    weights = nl * (d * 3 * hd + hd * d + d * hd + hd * d + d * 2 * F +
                    F * d) * wbytes + d * V * wbytes
    self_kv = nl * float(np.mean([self.self_attention_bytes(t)
                                  for t in range(self.L)]))
    cross = nl * self.cross_attention_bytes()
    return int(weights + self_kv + cross)

  def self_attention_bytes(self, t):
    s = 2
    hd = self.cfg.num_heads * self.cfg.head_dim
    R = self.B * self.K
    return R * hd * (t + 1) * 2 * s + R * hd * 2 * s + 2 * R * hd * s


def time_kernel(torch, fn, launches, replays=5):
  """Average duration of one kernel launch of `fn`: `launches` launches are
  captured into a HIP graph on a side stream (so the host launch rate does not
  enter), the graph is replayed `replays` times, and HIP events recorded on
  that same stream bracket the replays."""
  import ctypes
  from t5x_amd import _lib
  st = torch.cuda.Stream()
  st.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(st):
    fn()
    st.synchronize()
    _lib.call('t5d_graph_begin', st.cuda_stream)
    try:
      for _ in range(launches):
        fn()
    finally:
      graph = ctypes.c_void_p()
      _lib.call('t5d_graph_end', st.cuda_stream, ctypes.byref(graph))
    _lib.call('t5d_graph_launch', graph, st.cuda_stream)
    st.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record(st)
    for _ in range(replays):
      _lib.call('t5d_graph_launch', graph, st.cuda_stream)
    end.record(st)
    end.synchronize()
  _lib.call('t5d_graph_destroy', graph)
  return start.elapsed_time(end) * 1e-3 / (launches * replays)


PROFILE_NOTE = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                            'profiles',
                            'cross_attn_mfma_kernel_base-beam4_pmc.txt')


STEP_TRAFFIC_NOTE = os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                 'profiles',
                                 'decode_step_base-beam4_hbm_traffic_pmc.txt')


def _noted(path, key):
  if not os.path.exists(path):
    return None
  with open(path) as f:
    for line in f:
      if line.startswith(key + ':'):
        return int(float(line.split(':', 1)[1].split()[0]))
  return None


def measured_traffic(name):
  """HBM bytes per launch of the dominant kernel from the committed counter
  summary (FETCH_SIZE + WRITE_SIZE, calibrated against a plain copy), or None
  when no summary exists for this workload."""
  if name != 'base-beam4':
    return None
  return _noted(PROFILE_NOTE, 'traffic_bytes_per_launch')


def device_level(w, ms_per_step, in_flight):
  """Bytes per loop iteration over the wall-clock time of an iteration, for
  the modes the product runs in (batch lanes side by side; several batches in
  flight): the device-level counterpart of the per-launch roofline figure,
  which is measured on a single chain of kernels.  `algorithmic`: the bytes an
  iteration has to move (Workload.step_bytes); `traffic`: what the memory
  counters read for all kernels of an iteration (FETCH_SIZE + WRITE_SIZE summed
  over a kernel trace of the loop, from the committed summary; the counters
  serialise dispatches, which changes when bytes move, not how many)."""
  alg = w.step_bytes()
  traffic = (_noted(STEP_TRAFFIC_NOTE, 'step_traffic_bytes')
             if w.name == 'base-beam4' else None)

  def rates(ms):
    out = {'ms_per_step': ms,
           'algorithmic_gbps': round(alg / ms / 1e6, 1),
           'algorithmic_frac': round(alg / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    if traffic:
      out['traffic_gbps'] = round(traffic / ms / 1e6, 1)
      out['traffic_frac'] = round(traffic / ms / 1e6 / HBM_PEAK_GBPS, 4)
    return out

  out = {'algorithmic_bytes_per_step': alg, 'traffic_bytes_per_step': traffic,
         'one_batch': rates(ms_per_step)}
  if in_flight and in_flight.get('value'):
    out['batches_in_flight'] = rates(in_flight['ms_per_step'])
  return out


def in_loop_kernel_times(w, families, repeats=3):
  """Device time per launch of kernel families where they run: inside the
  decode loop, between the step's other kernels, with the caches as those
  leave them.  Measured by difference: one whole decode is replayed from a
  graph of the full iteration and from graphs of the iteration enqueued
  without one family's launches (t5d_model_step::leave_out), each bracketed
  by HIP events on the stream the graphs are launched on; what leaving the
  family out saves, divided by its launches, is its average duration in the
  loop.  (Events around single launches inside the loop were tried first:
  a launch that carries events runs 1-2 us slower than the same launch
  without, by the profiler's own trace.)  Returns {mask: (seconds, launches)}."""
  from t5x_amd import _lib
  torch = w.torch
  nl = w.cfg.num_decoder_layers

  def one_decode(mask):
    w.loop = None
    w.new_decode()               # re-binds the kept context: state restarts
    fused = w.loop.fused
    graph = fused.iteration_graph(mask)
    try:
      start = torch.cuda.Event(enable_timing=True)
      end = torch.cuda.Event(enable_timing=True)
      fused.launch_graph(graph, 1)   # first replay of a new graph: untimed
      fused.stream.synchronize()
      start.record(fused.stream)
      fused.launch_graph(graph, w.L - 1)
      end.record(fused.stream)
      end.synchronize()
      w.loop.step = w.L
      w.check_full_decode()
    finally:
      fused.stream.synchronize()
      _lib.call('t5d_graph_destroy', graph)
      w.loop = None
    return start.elapsed_time(end) * 1e-3

  masks = [0] + list(families)
  lanes, w.module.decode_lanes = w.module.decode_lanes, 1  # one chain of kernels
  try:
    best = {m: min(one_decode(m) for _ in range(repeats)) for m in masks}
  finally:
    w.module.decode_lanes = lanes
    w.loop = None
  launches = nl * (w.L - 1)
  return {m: ((best[0] - best[m]) / launches, launches) for m in families}


def roofline_cross_attention(w, reps_per_layer=4, in_loop=True):
  """The step's largest single stream of HBM bytes per launch: the
  cross-attention kernel over the encoder K/V (with the pre-attention layer
  norm and the query projection fused in where the model width allows), one
  launch per layer per step, same shape every step.  Replayed here back to
  back, walking the layers so no launch finds its K/V in a cache, and timed
  with HIP events on the launch stream."""
  from t5x_amd import ops
  torch = w.torch
  cross = w.module._cross[1]
  R = w.B * w.K
  cfg = w.cfg
  hd = cfg.num_heads * cfg.head_dim
  act = w.encoded.dtype
  x = torch.randn((R, cfg.emb_dim), device='cuda').to(act)
  q = torch.randn((R, hd), device='cuda').to(act)
  out = torch.empty((R, hd), dtype=act, device='cuda')
  layers = w.weights.layers
  nl = len(cross['k'])
  fused = (w.weights.layers[0]['cross_q'].w_dtype == 1 and cross['E'] <= 512
           and cfg.emb_dim <= 768)  # as t5d_decoder_step chooses
  state = {'i': 0}

  def launch():
    i = state['i'] = (state['i'] + 1) % nl  # walk the layers: no cache reuse
    if fused:
      ops.cross_attention_step_norm_q(x, layers[i]['ln_cross'],
                                      layers[i]['cross_q'], cross['k'][i],
                                      cross['v'][i], cross['enc_len'], w.K, out,
                                      units=cross.get('units'))
    else:
      ops.cross_attention_step(q, cross['k'][i], cross['v'][i],
                               cross['enc_len'], w.K, out,
                               units=cross.get('units'))

  reps = max(1, min(reps_per_layer, 96 // nl))
  replay_sec = time_kernel(torch, launch, reps * nl)
  nbytes = w.cross_attention_bytes()
  if fused:
    name = 'cross_attn_mfma_kernel<4,4,%d>' % ((cfg.emb_dim // 64 + 3) // 4)
  elif w.bf16:
    name = 'cross_attn_mfma_kernel (query projected separately)'
  else:
    name = 'cross_attn_f32_kernel (float32 on the vector ALUs)'
  out = {'kernel': name, 'bound': 'hbm', 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
         'traffic': measured_traffic(w.name), 'bytes_per_launch': nbytes,
         # moved by the same launch for the dense layers' account (layer norm
         # + query projection fused in); not part of `achieved`
         'fused_query_bytes': w.fused_query_bytes() if fused else 0}
  sec, where = replay_sec, 'back-to-back replay over the layers'
  if in_loop and w.bf16:
    # The figure that counts is the kernel's duration inside the decode loop
    # (what a kernel trace of the loop shows); the back-to-back replay, which
    # finds the instruction cache and the translation caches warm, is kept
    # next to it.
    from t5x_amd import _lib
    times = in_loop_kernel_times(w, (_lib.LEAVE_OUT_CROSS_ATTENTION,
                                     _lib.LEAVE_OUT_SELF_ATTENTION))
    sec, n = times[_lib.LEAVE_OUT_CROSS_ATTENTION]
    where = (f'inside the decode loop (the whole batch as one chain of '
             f'kernels), by difference: {n} launches of one whole decode '
             'left out')
    out['replay_launch_us'] = round(replay_sec * 1e6, 2)
    ssec, sn = times[_lib.LEAVE_OUT_SELF_ATTENTION]
    sbytes = float(np.mean([w.self_attention_bytes(t)
                            for t in range(1, w.L)]))
    out['self_attention'] = {
        'kernel': 'self_attn_tail_kernel', 'avg_launch_us': round(ssec * 1e6, 2),
        'launches': sn, 'mean_bytes_per_launch': int(sbytes),
        'achieved': round(sbytes / ssec / 1e9, 1),
        'frac': round(sbytes / ssec / 1e9 / HBM_PEAK_GBPS, 4)}
  achieved = nbytes / sec / 1e9
  out.update({'achieved': round(achieved, 1),
              'frac': round(achieved / HBM_PEAK_GBPS, 4),
              'avg_launch_us': round(sec * 1e6, 2), 'measured': where})
  return out


def in_flight_throughput(w, n, groups=3):
  """Whole decodes of n different batches (same shape, same weights) running
  on the device at once, each on its own streams, driven by one host thread
  through the loops' start / poll protocol (chunks of 8 iterations enqueued
  ahead, the loop flag read back without waiting): the throughput of
  EncoderDecoderModel.predict_batches.  Like the single-decode figure, decode
  starts are outside the clock; everything the loops do until the last one has
  ended, read-backs and the iterations enqueued past the end included, is
  inside."""
  import torch
  from t5x_amd import decoding, models, network
  dev = w.encoded.device
  fns = []
  for i in range(n):
    rs = np.random.Generator(np.random.PCG64(w.seed + 101 + i))
    tok = rs.integers(2, 32128, size=(w.B, w.E)).astype(np.int32)
    lens = rs.integers(w.enc_lens.min(), w.E + 1, size=(w.B,))
    tok[np.arange(w.E)[None, :] >= lens[:, None]] = 0
    gen = torch.Generator(device=dev)
    gen.manual_seed(w.seed + 201 + i)
    encoded = torch.randn(tuple(w.encoded.shape), generator=gen,
                          device=dev).to(w.encoded.dtype)
    fns.append(models.StepFunction(
        w.model, w.params, network.BeamShared(encoded, w.K),
        network.BeamShared(torch.as_tensor(tok, device=dev), w.K), w.L,
        in_flight=True))

  def group():
    loops = []
    for i, fn in enumerate(fns):
      cache = w.module.init_cache(w.B, w.L)
      if w.loop_kind == 'beam':
        loops.append(decoding.BeamLoop(w.inputs, cache, fn, eos_id=1,
                                       num_decodes=w.K, alpha=0.6))
      else:
        _, temperature, topk = w.loop_kind
        w.decodes += 1
        loops.append(decoding.SampleLoop(
            w.inputs, cache, fn, 1, w.seed + w.decodes, w.K, temperature,
            topk, use_fused=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    decoding.run_in_flight(loops)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for loop in loops:
      loop.finish()
      count = int((loop.cur.cur_index if w.loop_kind == 'beam' else
                   loop.fused.step_count).item())
      if count != w.L:
        raise RuntimeError(f'decode in flight stopped at step {count}')
    return dt

  w.loop = None
  for _ in range(2):   # builds the n contexts; first pass of re-binding them
    group()
  seconds = sum(group() for _ in range(groups))
  steps = groups * n * w.L
  return {'decodes': n, 'value': round(w.B * steps / seconds, 1),
          'unit': 'tokens/s', 'steps': steps,
          'ms_per_step': round(seconds / steps * 1e3, 4),
          'what': (f'{n} batches of the same shape decoding at once '
                   '(separate streams, one host thread), whole decodes')}


def copy_calibration(torch, nbytes=256 << 20, reps=5):
  """A plain device copy of known size, so FETCH_SIZE / WRITE_SIZE readings can
  be scaled: it reads nbytes and writes nbytes."""
  src = torch.empty(nbytes, dtype=torch.uint8, device='cuda')
  src.zero_()
  dst = torch.empty_like(src)
  for _ in range(reps):
    dst.copy_(src)
  torch.cuda.synchronize()
  return nbytes


def cpu_baseline(name, steps, seed):
  """NumPy oracle on this host: `steps` beam-search iterations at the same
  shape (decoder only, cross K/V hoisted as in the GPU path)."""
  from oracle import decoding as odec
  from oracle import t5 as ot5
  size, B, K, E, Emin, L, dtype, wdt, loop = CONFIGS[name]
  if size == 'small':
    steps = max(steps, L - 2)  # a few steps of this one are over in a blink
  from t5x_amd import network
  kw = dict(network.T5_1_1[size])
  kw['num_encoder_layers'] = 0
  cfg = ot5.T5Config(dtype=dtype, **kw)
  params = ot5.init_params(cfg, seed, with_encoder=False)
  rs = np.random.Generator(np.random.PCG64(seed + 1))
  tok = rs.integers(2, 32128, size=(B, E)).astype(np.int32)
  lens = rs.integers(Emin, E + 1, size=(B,))
  tok[np.arange(E)[None, :] >= lens[:, None]] = 0
  encoded = ot5.bf16_round(
      rs.standard_normal((B, E, cfg.emb_dim), dtype=np.float32))
  cross_kv = ot5.project_cross_kv(params, cfg, encoded)
  cross_kv = [(np.repeat(k, K, 0), np.repeat(v, K, 0)) for k, v in cross_kv]
  enc_tok_rows = np.repeat(tok, K, axis=0)
  calls = {'n': 0, 't0': None}

  def tokens_to_logits(state):
    if calls['t0'] is None:
      calls['t0'] = time.perf_counter()
    calls['n'] += 1
    t = state.cur_token
    logits, cache = ot5.decode(params, cfg, None, enc_tok_rows, t, t,
                               decode=True, cache=state.cache,
                               max_decode_length=L, cross_kv=cross_kv)
    return logits[:, 0], cache

  inputs = np.zeros((B, L), np.int32)
  if loop == 'beam':
    odec.beam_search(inputs, ot5.init_cache(cfg, B, L), tokens_to_logits, 1,
                     num_decodes=K, alpha=0.6, max_decode_step=steps)
    what = 'beam-search'
  else:
    odec.temperature_sample(inputs, ot5.init_cache(cfg, B, L), tokens_to_logits,
                            1, decode_rng=seed, num_decodes=K,
                            temperature=loop[1], topk=loop[2],
                            max_decode_steps=steps)
    what = 'temperature_sample'
  sec = time.perf_counter() - calls['t0']
  return {'value': round(B * calls['n'] / sec, 2), 'unit': 'tokens/s',
          'cores': host_threads(), 'kind': 'port',
          'sample': f'{calls["n"]} {what} steps of {name} (NumPy oracle, '
                    f'decoder only, {sec:.1f} s)'}


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak, vendor figure


class EncoderStage:
  """What runs once per batch before the decode loop: the encoder forward over
  the [B, E] tokens and the projection of its output to every decoder layer's
  cross-attention K/V.  Same synthetic batch as the decode workload."""

  def __init__(self, name, seed):
    import torch
    from t5x_amd import network
    self.torch = torch
    size, B, K, E, Emin, L, dtype, wdt, _ = CONFIGS[name]
    if dtype != 'bfloat16':
      raise SystemExit('bench.py --stage encoder measures the bfloat16 '
                       f'encoder (matrix-core kernels); {name} is {dtype}')
    self.size, self.B, self.K, self.E = size, B, K, E
    self.cfg = network.t5_1_1_config(size, dtype=dtype, weight_dtype=wdt)
    dev = torch.device('cuda')
    self.params = network.init_params(self.cfg, seed, dev, with_encoder=True)
    self.module = network.Transformer(self.cfg, dev)
    rs = np.random.Generator(np.random.PCG64(seed + 1))
    tok = rs.integers(2, 32128, size=(B, E)).astype(np.int32)
    lens = rs.integers(Emin, E + 1, size=(B,))
    tok[np.arange(E)[None, :] >= lens[:, None]] = 0
    self.tok_host, self.lens = tok, lens
    self.tokens = torch.as_tensor(tok, device=dev)
    self.weights = self.module.decoder_weights(self.params)

  def run_steps(self, n):
    for _ in range(n):
      encoded = self.module.apply({'params': self.params}, self.tokens,
                                  enable_dropout=False,
                                  method=self.module.encode)
      # a fresh encoder output every pass: nothing is served from a cache
      self.module._cross_kv(self.weights, encoded, self.tokens, self.K)

  def flops(self):
    """Dense-equivalent multiply-adds x 2 of one pass (padding included)."""
    c = self.cfg
    M, d, F = self.B * self.E, c.emb_dim, c.mlp_dim
    hd = c.num_heads * c.head_dim
    enc = c.num_encoder_layers * (2 * M * d * (3 * hd) + 2 * M * hd * d +
                                  2 * M * d * 2 * F + 2 * M * F * d +
                                  4 * self.B * c.num_heads * self.E * self.E *
                                  c.head_dim)
    cross = c.num_decoder_layers * 2 * (2 * M * d * hd)
    return enc + cross

  def roofline(self):
    """The stage's dominant kernel: rows_gemm_direct_kernel on the gated MLP input
    projection ([B*E, d] x [d, 2F], GELU gate in the epilogue), one launch per
    encoder layer; replayed over the layers' kernels and timed with HIP events
    on the launch stream."""
    from t5x_amd import ops
    torch, c = self.torch, self.cfg
    layers = self.module._enc_weights[('hip', id(self.params))][1].layers
    M = self.B * self.E
    y = torch.randn((M, c.emb_dim), device='cuda').to(torch.bfloat16)
    out = torch.empty((M, c.mlp_dim), dtype=torch.bfloat16, device='cuda')
    state = {'i': 0}

    def launch():
      i = state['i'] = (state['i'] + 1) % len(layers)
      ops.gemm_rows(y, layers[i]['wi'], out=out)

    sec = time_kernel(torch, launch, 2 * len(layers))
    flops = 2.0 * M * c.emb_dim * 2 * c.mlp_dim
    achieved = flops / sec / 1e12
    return {'kernel': 'rows_gemm_direct_kernel (gated MLP input projection)',
            'bound': 'mfma', 'achieved': round(achieved, 1),
            'peak': MFMA_BF16_PEAK_TFLOPS, 'unit': 'TFLOP/s',
            'frac': round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
            'traffic': None, 'flops_per_launch': flops,
            'avg_launch_us': round(sec * 1e6, 2)}

  def cpu_baseline(self, rows, seed):
    """NumPy oracle on this host: encoder forward + cross K/V projection of the
    first `rows` batch items."""
    from oracle import t5 as ot5
    from t5x_amd import network
    cfg = ot5.T5Config(dtype='bfloat16', **network.T5_1_1[self.size])
    params = ot5.init_params(cfg, seed, with_encoder=True)
    tok = self.tok_host[:rows]
    t0 = time.perf_counter()
    encoded = ot5.encode(params, cfg, tok)
    ot5.project_cross_kv(params, cfg, encoded)
    sec = time.perf_counter() - t0
    return {'value': round(rows * self.E / sec, 1), 'unit': 'tokens/s',
            'cores': host_threads(), 'kind': 'port',
            'sample': f'{rows} of the {self.B} batch rows, one pass'}


def main_dense(args):
  """The dense layers of the configuration's decoder at its decode rows: every
  kind (q/k/v with its layer norm, the two attention outputs, the gated MLP
  input with its norm, the MLP output, the vocabulary projection with the
  final norm) replayed back to back over the layers' weights, so no launch
  finds its weights cached; time per launch from HIP events on the launch
  stream.  `value`: passes over all dense layers of the decoder per second."""
  import torch
  from t5x_amd import network, ops
  size, B, K, E, Emin, L, dtype, wdt, loop = CONFIGS[args.config]
  if dtype != 'bfloat16':
    raise SystemExit('bench.py --stage dense measures the matrix-core kernels '
                     f'(bfloat16 activations); {args.config} is {dtype}')
  cfg = network.t5_1_1_config(size, dtype=dtype, weight_dtype=wdt)
  dev = torch.device('cuda')
  params = network.init_params(cfg, args.seed, dev, with_encoder=False)
  module = network.Transformer(cfg, dev)
  w = module.decoder_weights(params)
  R, d, F, V = B * K, cfg.emb_dim, cfg.mlp_dim, cfg.vocab_size
  hd = cfg.num_heads * cfg.head_dim
  act = torch.bfloat16
  wb = 1 if wdt == 'int8' else 2
  rnd = lambda *s: torch.randn(s, device=dev).to(act)
  x, ao, h = rnd(R, d), rnd(R, hd), rnd(R, F)
  norm_rides = d <= 1024 or (wdt == 'int8' and d <= 2048)
  nl = len(w.layers)
  state = {'i': 0}

  def layer():
    state['i'] = (state['i'] + 1) % nl
    return w.layers[state['i']]

  xn = ops.rmsnorm(x, w.layers[0]['ln_self'])
  own_norm = []

  def normed(name, ln):
    # The layer norm rides in the projection's kernel where the step does so;
    # elsewhere it is a launch of its own, timed as its own row below.
    rides = norm_rides and (d <= 1024 or w.layers[0][name].N <= 2048)
    if not rides:
      own_norm.append(name)
    def run():
      l = layer()
      if rides:
        ops.gemm(x, l[name], norm_scale=l[ln])
      else:
        ops.gemm(xn, l[name])
    return run

  with_norm = lambda name, key: name + (
      '' if key in own_norm else ' with its layer norm')
  qkv_fn, cq_fn, wi_fn = (normed('qkv', 'ln_self'),
                          normed('cross_q', 'ln_cross'), normed('wi', 'ln_mlp'))
  kinds = [
      (with_norm('q, k, v', 'qkv'), qkv_fn, d, 3 * hd, 1),
      ('attention output + residual',
       lambda: ops.gemm(ao, layer()['self_out'], residual=x), hd, d, 2),
      (with_norm('cross-attention query', 'cross_q'), cq_fn, d, hd, 1),
      (with_norm('gated MLP input', 'wi'), wi_fn, d, 2 * F, 1),
      ('MLP output + residual',
       lambda: ops.gemm(h, layer()['wo'], residual=x), F, d, 1),
  ]
  rows, total = [], 0.0
  for name, fn, k, n, per_layer in kinds:
    sec = time_kernel(torch, fn, 2 * nl)
    nbytes = k * n * wb + R * (k + n) * 2
    rows.append({'layer': name, 'K': k, 'N': n, 'launches_per_step':
                 per_layer * nl, 'us': round(sec * 1e6, 2),
                 'weight_gbps': round(k * n * wb / sec / 1e9, 1),
                 'tflops': round(2.0 * R * k * n / sec / 1e12, 1),
                 'bytes': nbytes})
    total += sec * per_layer * nl
  if norm_rides and d <= 1024:
    vocab = lambda: ops.gemm(x, w.logits, norm_scale=w.ln_final,
                             out_dtype=torch.float32)
  else:
    own_norm.append('logits')
    vocab = lambda: ops.gemm(xn, w.logits, out_dtype=torch.float32)
  if own_norm:
    sec = time_kernel(torch, lambda: ops.rmsnorm(x, layer()['ln_mlp']), 2 * nl)
    n_norms = nl * sum(k in own_norm for k in ('qkv', 'cross_q', 'wi')) + (
        'logits' in own_norm)
    rows.append({'layer': 'layer norm as a launch of its own', 'K': d, 'N': d,
                 'launches_per_step': n_norms, 'us': round(sec * 1e6, 2),
                 'weight_gbps': 0.0, 'tflops': 0.0, 'bytes': 2 * R * d * 2})
    total += sec * n_norms
  sec = time_kernel(torch, vocab, 8)
  rows.append({'layer': with_norm('vocabulary projection', 'logits'),
               'K': d, 'N': V,
               'launches_per_step': 1, 'us': round(sec * 1e6, 2),
               'weight_gbps': round(d * V * wb / sec / 1e9, 1),
               'tflops': round(2.0 * R * d * V / sec / 1e12, 1),
               'bytes': d * V * wb + R * d * 2 + R * V * 4})
  total += sec
  best = max(rows, key=lambda r: r['weight_gbps'])
  weights = sum(r['K'] * r['N'] * wb * r['launches_per_step'] for r in rows
                if r['weight_gbps'])
  out = {
      'metric': f'passes over the decoder\'s dense layers per second, '
                f'{args.config} at {R} rows on 1 GPU',
      'value': round(1.0 / total, 1), 'unit': 'passes/s', 'n_gpus': 1,
      'steps': 1, 'warmup': 0, 'ms_per_step': round(total * 1e3, 4),
      'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
      'dtype': 'bf16' if wdt is None else f'bf16 act / {wdt} weights',
      'data': 'synthetic',
      'config': {'workload': f'T5.1.1-{size} decoder dense layers at {R} rows',
                 'name': args.config, 'stage': 'dense', 'layers': rows,
                 'weight_bytes_per_pass': weights,
                 'weights_gbps_whole_pass': round(weights / total / 1e9, 1)},
      'roofline': {'kernel': best['layer'], 'bound': 'hbm',
                   'achieved': best['weight_gbps'], 'peak': HBM_PEAK_GBPS,
                   'unit': 'GB/s',
                   'frac': round(best['weight_gbps'] / HBM_PEAK_GBPS, 4),
                   'traffic': None, 'bytes_per_launch': best['bytes'],
                   'avg_launch_us': best['us']},
  }
  if args.counter_copy:
    out['counter_copy_bytes'] = copy_calibration(torch)
  print(json.dumps(out))


def main_memory(args):
  """Who serves data that one kernel wrote and the next kernel reads.  Every
  case is `reps` rounds of (writer, [evictor,] reader) with HIP events around
  the reader.
  Plain kernels of known size (t5d_measure_fill / t5d_measure_read): the
  reader takes each piece on the XCD that wrote it, on another XCD, or after
  1.5 GB of other data has gone through the caches.  Then the pair this
  question is about: the float32 logits written by the vocabulary projection
  and read back by the selection kernel."""
  import torch
  from t5x_amd import _lib, network, ops
  size, B, K, E, Emin, L, dtype, wdt, loop = CONFIGS[args.config]
  dev = torch.device('cuda')
  reps, blocks = 20, 1024
  sink = torch.zeros(4, dtype=torch.int32, device=dev)
  big_a = torch.zeros((768 << 20,), dtype=torch.uint8, device=dev)
  big_b = torch.zeros_like(big_a)
  evict = lambda: big_b.copy_(big_a)   # 768 MB read + 768 MB written

  def reader_us(write, read, evicted):
    """Median duration of `read` between two events on its stream.  A busy
    kernel in front of every round lets the host enqueue the whole round
    before the device reaches it, so no launch latency falls between the
    events; what two events cost with nothing between them is taken off."""
    def rounds(with_read):
      ts = []
      for _ in range(reps + 4):
        torch.cuda._sleep(400000)
        write()
        if evicted:
          evict()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        if with_read:
          read()
        e1.record()
        ts.append((e0, e1))
      torch.cuda.synchronize()
      return float(np.median([a.elapsed_time(b) for a, b in ts[4:]])) * 1e3
    return rounds(True) - rounds(False)

  s = _lib.stream_handle
  plain = []
  for mb in (16.45, 65.8):
    nbytes = int(mb * 1e6) // 16 * 16
    buf = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    fill = lambda: _lib.call('t5d_measure_fill', s(), buf.data_ptr(), nbytes,
                             1, blocks)
    rd = lambda shift, tag: (lambda: _lib.call(
        't5d_measure_read', s(), buf.data_ptr(), nbytes, shift, blocks,
        sink.data_ptr(), tag))
    row = {'bytes': nbytes}
    for case, (name, shift, evicted) in enumerate((
        ('same_xcd_us', 0, False), ('other_xcd_us', 3, False),
        ('evicted_us', 3, True))):
      # measure_read_kernel<tag> in a kernel trace: tag = 3 * size + case
      us = reader_us(fill, rd(shift, 3 * len(plain) + case), evicted)
      row[name] = round(us, 2)
      row[name.replace('_us', '_gbps')] = round(nbytes / us / 1e3, 1)
    plain.append(row)

  cfg = network.t5_1_1_config(size, dtype=dtype, weight_dtype=wdt)
  params = network.init_params(cfg, args.seed, dev, with_encoder=False)
  module = network.Transformer(cfg, dev)
  w = module.decoder_weights(params)
  R, d, V = B * K, cfg.emb_dim, cfg.vocab_size
  x = torch.randn((R, d), device=dev).to(torch.bfloat16)
  logits = torch.empty((R, V), dtype=torch.float32, device=dev)
  live = torch.zeros((B, K), dtype=torch.float32, device=dev)
  k2 = 2 * K
  bufs = (torch.empty((B, k2), dtype=torch.float32, device=dev),
          torch.empty((B, k2), dtype=torch.int32, device=dev),
          torch.empty((R,), dtype=torch.float32, device=dev),
          torch.empty((R,), dtype=torch.float32, device=dev),
          torch.empty((2 * R * k2,), dtype=torch.int32, device=dev))
  project = lambda: ops.gemm(x, w.logits, norm_scale=w.ln_final,
                             out_dtype=torch.float32, out=logits)
  select = lambda: ops.beam_topk(logits, live, k2, bufs)
  fresh = reader_us(project, select, False)
  stale = reader_us(project, select, True)
  out = {
      'metric': 'read-back of data the previous kernel wrote, by what serves '
                'it, on 1 GPU',
      'value': plain[0]['other_xcd_gbps'], 'unit': 'GB/s', 'n_gpus': 1,
      'steps': reps, 'warmup': 1, 'ms_per_step': plain[0]['other_xcd_us'] / 1e3,
      'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
      'dtype': 'u8', 'data': 'synthetic',
      'config': {'workload': 'plain 16-byte streaming reads of a buffer a '
                             'plain kernel just wrote; logits [%d, %d] float32 '
                             'between projection and selection' % (R, V),
                 'stage': 'memory', 'plain': plain,
                 'logits_bytes': R * V * 4,
                 'selection_after_projection_us': round(fresh, 2),
                 'selection_after_eviction_us': round(stale, 2)},
      'roofline': {'kernel': 'measure_read_kernel (evicted: from HBM)',
                   'bound': 'hbm', 'achieved': plain[1]['evicted_gbps'],
                   'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                   'frac': round(plain[1]['evicted_gbps'] / HBM_PEAK_GBPS, 4),
                   'traffic': None, 'bytes_per_launch': plain[1]['bytes'],
                   'avg_launch_us': plain[1]['evicted_us']},
  }
  print(json.dumps(out))


def host_threads():
  try:
    from threadpoolctl import threadpool_info
    return int(max([p.get('num_threads', 1) for p in threadpool_info()] or [1]))
  except Exception:  # pylint: disable=broad-except
    return os.cpu_count() or 1


def main_encoder(args):
  import torch
  w = EncoderStage(args.config, args.seed)
  w.run_steps(max(1, args.warmup))
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  w.run_steps(args.steps)
  torch.cuda.synchronize()
  elapsed = time.perf_counter() - t0
  size = CONFIGS[args.config][0]
  out = {
      'metric': f'encoder tokens/sec, T5.1.1-{size} encoder forward + cross '
                'K/V projection on 1 GPU',
      'value': round(w.B * w.E * args.steps / elapsed, 1),
      'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps,
      'warmup': max(1, args.warmup),
      'ms_per_step': round(elapsed / args.steps * 1e3, 4),
      'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
      'dtype': 'bf16', 'data': 'synthetic',
      'config': {'workload': f'T5.1.1-{size} encoder forward over batch {w.B} x '
                             f'{w.E} tokens ({int(w.lens.min())}..'
                             f'{int(w.lens.max())} valid) + cross K/V '
                             f'projection for {w.cfg.num_decoder_layers} '
                             'decoder layers',
                 'name': args.config, 'stage': 'encoder',
                 'tflops_whole_stage': round(
                     w.flops() * args.steps / elapsed / 1e12, 1)},
      'roofline': w.roofline(),
  }
  if not args.no_cpu_baseline:
    out['cpu_baseline'] = w.cpu_baseline(args.cpu_steps, args.seed)
  print(json.dumps(out))


def main():
  args = parse_args()
  if args.gpus != 1:
    print('bench.py: this build measures ONE GPU; --gpus must be 1 '
          f'(got {args.gpus}). The decode path shards over batch with no '
          'exchange: each GPU would run this program on its share of the '
          'batch.', file=sys.stderr)
    sys.exit(2)
  if args.hw_queues > 0:  # before anything touches the GPU
    os.environ['GPU_MAX_HW_QUEUES'] = str(args.hw_queues)
  import torch
  if not torch.cuda.is_available():
    print('bench.py: no GPU visible', file=sys.stderr)
    sys.exit(3)
  if args.stage == 'encoder':
    return main_encoder(args)
  if args.stage == 'dense':
    return main_dense(args)
  if args.stage == 'memory':
    return main_memory(args)
  w = Workload(args.config, args.seed, args.lanes)
  if args.roofline_only:
    w.new_decode()  # builds the cross-attention K/V
    r = roofline_cross_attention(w, reps_per_layer=1, in_loop=False)
    r['copy_bytes'] = copy_calibration(torch)
    print(json.dumps(r))
    return
  w.prime()
  w.run_steps(args.warmup)
  torch.cuda.synchronize()
  elapsed, windows = w.run_steps(args.steps, timed=True)

  size, B, K, E, Emin, L, dtype, wdt, loop = CONFIGS[args.config]
  if loop == 'beam':
    what = f'beam_search decode loop: batch {B} x {K} beams'
  elif loop[1] > 0:
    what = (f'temperature_sample decode loop (temperature {loop[1]}, top-k '
            f'{loop[2]}): batch {B}')
  else:
    what = f'temperature_sample decode loop (greedy): batch {B}'
  out = {
      'metric': ('decoded tokens/sec, T5.1.1-base beam=4 on 1 GPU'
                 if args.config == DEFAULT_CONFIG else
                 f'decoded tokens/sec, {args.config} on 1 GPU'),
      'value': round(B * args.steps / elapsed, 1),
      'unit': 'tokens/s',
      'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
      'ms_per_step': round(elapsed / args.steps * 1e3, 4),
      'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
      'dtype': ({'bfloat16': 'bf16', 'float32': 'f32'}[dtype] if wdt is None
                else f'bf16 act / {wdt} weights'),
      'data': 'synthetic',
      'config': {'workload': f'T5.1.1-{size} {what}, encoder {E} ({Emin}..{E} '
                             f'valid), max decode length {L}',
                 'name': args.config, 'beam_rows': B * K,
                 # batch slices stepped side by side on separate streams
                 'batch_lanes': getattr(getattr(w.loop, 'fused', None),
                                        'n_lanes', 1),
                 # decode streams the device was found (or told) to run side
                 # by side: decides the lanes above and the batches in flight
                 'streams_side_by_side': w.module.streams_side_by_side(),
                 'gpu_max_hw_queues': os.environ.get('GPU_MAX_HW_QUEUES'),
                 # positions t of the decode the timed iterations covered:
                 # whole decodes, then a window centred on (L-1)/2
                 't_first': windows[-1][0], 't_last': windows[-1][1],
                 'timed_windows': [list(x) for x in windows],
                 'rows_x_steps_per_s': round(B * K * args.steps / elapsed, 1)},
      'roofline': roofline_cross_attention(
          w, in_loop=not args.replay_roofline),
  }
  # (the oracle's float32 copy of the XXL weights alone is 45 GB and minutes
  # of initialisation: no CPU figure for that shape)
  n_in_flight = args.in_flight
  if n_in_flight is None:
    n_in_flight = (w.module.streams_side_by_side()
                   if args.config == DEFAULT_CONFIG else 0)
  if n_in_flight > 1:
    # an extra figure: whatever goes wrong in it must not cost the line
    try:
      out['in_flight'] = in_flight_throughput(w, n_in_flight)
    except Exception as e:  # pylint: disable=broad-except
      out['in_flight'] = {'decodes': n_in_flight, 'value': None,
                          'error': f'{type(e).__name__}: {e}'}
  if args.counter_copy:
    out['counter_copy_bytes'] = copy_calibration(torch)
  out['roofline']['device_level'] = device_level(
      w, out['ms_per_step'], out.get('in_flight'))
  if not args.no_cpu_baseline and size != 'xxl':
    out['cpu_baseline'] = cpu_baseline(args.config, args.cpu_steps, args.seed)
  print(json.dumps(out))


if __name__ == '__main__':
  main()
