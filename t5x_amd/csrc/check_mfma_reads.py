#!/usr/bin/env python3
"""Build-time check of the compiled kernels: no result of a matrix instruction
is read too early.

On gfx950 a v_mfma result must not be read by a non-matrix instruction before
enough issue slots have passed; nothing in the hardware holds the reader back,
the compiler pads with s_nop.  Its count follows the fall-through side of a
branch only: with a uniform branch between a v_mfma and the first read of its
accumulator, one kernel of this library read the accumulator 4 slots after the
v_mfma on the taken side and got the previous tile's value (wrong attention
scores, no error).  This script walks the assembly that `make check` writes
for every source (hipcc -S of the same flags), follows taken branches as well,
and fails when any path from a v_mfma / v_smfmac to a reader of its
destination is shorter than NEED slots (9: what the compiler itself pads
straight-line code to for the 16x16x32 instructions used here).

A second check, for the kernels that fill LDS with global_load_lds behind
hand-placed barriers: a barrier orders instructions that have been issued,
not LDS reads that have completed, and the compiler may sink a k-tile's last
operand reads below the next barrier; a faster wavefront could then refill
the stage while those reads were still queued (seen as a wrong 16-row slice
in one launch in ten of the many-row dense kernel).  So in such a kernel
every s_barrier must come after an s_waitcnt that includes
lgkmcnt(0) — checked as: walking backwards from a barrier, over branches too,
no LDS instruction is met before such a wait.

usage: check_mfma_reads.py file.s [...]
"""
import collections
import re
import sys

NEED = 9
WINDOW = 16   # slots to follow a result for


def _regs(token):
  m = re.match(r'([av])\[(\d+):(\d+)\]', token)
  if m:
    return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
  m = re.match(r'([av])(\d+)$', token)
  if m:
    return {(m.group(1), int(m.group(2)))}
  return set()


def parse(text):
  """-> (instructions [(kernel, text)], labels {(kernel, label): index})."""
  kernel, ins, labels = None, [], {}
  for line in text.split('\n'):
    t = line.strip()
    if re.match(r'^_Z\w+:', t):
      kernel = t.split(':')[0]
      continue
    if not t or t.startswith(';'):
      continue
    m = re.match(r'^(\.LBB\w+):', t)
    if m:
      labels[(kernel, m.group(1))] = len(ins)
      continue
    if t.startswith('.') or kernel is None:
      continue
    ins.append((kernel, t.split(';')[0].strip()))
  return ins, labels


def _is_matrix(text):
  return text.startswith('v_mfma') or text.startswith('v_smfmac')


def short_reads(text, need=NEED):
  """-> ([(kernel, matrix instruction, slots, reader)], {slots: count})."""
  ins, labels = parse(text)
  found, hist = [], collections.Counter()
  for i, (kernel, t) in enumerate(ins):
    if not _is_matrix(t):
      continue
    dst = _regs(t.split(None, 1)[1].split(',')[0].strip())
    best = {}
    stack = [(i + 1, 0)]
    while stack:
      j, n = stack.pop()
      while j < len(ins) and ins[j][0] == kernel and n <= WINDOW:
        if best.get(j, 1 << 30) <= n:
          break
        best[j] = n
        t2 = ins[j][1]
        n += 1
        m = re.match(r's_nop (\d+)', t2)
        if m:
          n += int(m.group(1))
        parts = t2.split(None, 1)
        ops = [o.strip() for o in parts[1].split(',')] if len(parts) > 1 else []
        stores = t2.startswith(('global_store', 'ds_write', 'buffer_store',
                                'flat_store', 'scratch_store'))
        read = set()
        for o in (ops if stores else ops[1:]):
          read |= _regs(o)
        if read & dst:
          if not _is_matrix(t2):   # matrix -> matrix is interlocked
            hist[n] += 1
            if n < need:
              found.append((kernel, t, n, t2))
          break
        if ops and not stores and _regs(ops[0]) & dst:
          break                    # overwritten before any read
        if t2.startswith('s_endpgm'):
          break
        mb = re.match(r's_(c?)branch\w*\s+(\.LBB\w+)', t2)
        if mb:
          target = labels.get((kernel, mb.group(2)))
          if target is not None:
            stack.append((target, n))
          if not mb.group(1):
            break                  # unconditional: no fall-through
        j += 1
  return found, hist


def unguarded_barriers(text, depth=96):
  """-> [(kernel, index of the barrier among the kernel's barriers)] for
  kernels that use global_load_lds: barriers that an LDS read can reach
  without a wait for lgkmcnt(0) in between, on any path (walking backwards
  from the barrier, over branches too, until such a wait ends the path)."""
  ins, labels = parse(text)
  uses_dma = {k for k, t in ins if t.startswith('global_load_lds')}
  if not uses_dma:
    return []
  preds = collections.defaultdict(list)
  for i, (kernel, t) in enumerate(ins):
    m = re.match(r's_(c?)branch\w*\s+(\.LBB\w+)', t)
    if m:
      target = labels.get((kernel, m.group(2)))
      if target is not None:
        preds[target].append(i)
    falls_through = not (m and not m.group(1)) and not t.startswith('s_endpgm')
    if falls_through and i + 1 < len(ins) and ins[i + 1][0] == kernel:
      preds[i + 1].append(i)
  found, count = [], collections.Counter()
  for i, (kernel, t) in enumerate(ins):
    if kernel not in uses_dma or not t.startswith('s_barrier'):
      continue
    count[kernel] += 1
    seen, stack, bad = set(), [(p, 0) for p in preds[i]], False
    while stack and not bad:
      j, d = stack.pop()
      if j in seen or d > depth:
        continue
      seen.add(j)
      tj = ins[j][1]
      if tj.startswith('s_waitcnt') and 'lgkmcnt(0)' in tj:
        continue                   # this path is guarded
      if tj.startswith('ds_'):
        bad = True
        break
      stack.extend((p, d + 1) for p in preds[j])
    if bad:
      found.append((kernel, count[kernel]))
  return found


def main(paths):
  bad = barriers = 0
  total = collections.Counter()
  for path in paths:
    with open(path) as f:
      text = f.read()
    found, hist = short_reads(text)
    for kernel, nth in unguarded_barriers(text):
      barriers += 1
      print(f'{path}: {kernel}: barrier {nth} of a kernel that loads into LDS '
            'is reached by an LDS instruction with no wait for lgkmcnt(0) '
            'in between')
    total.update(hist)
    for kernel, t, n, t2 in found:
      bad += 1
      print(f'{path}: {kernel}: "{t}" is read {n} slots later by "{t2}" '
            f'(need {NEED})')
  print(f'check_mfma_reads: {sum(total.values())} reads of matrix results in '
        f'{len(paths)} files, shortest {min(total) if total else "-"} slots, '
        f'{bad} too early; {barriers} unguarded barriers')
  return 1 if bad or barriers else 0


if __name__ == '__main__':
  sys.exit(main(sys.argv[1:]))
