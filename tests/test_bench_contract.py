"""bench.py's command-line contract: one GPU only, one JSON line per run with
the agreed keys.  The GPU cases run the two short stages whose commands the
profile summaries quote (the default decode run is timed by the driver)."""

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KEYS = {'metric', 'value', 'unit', 'n_gpus', 'steps', 'warmup', 'ms_per_step',
        'higher_is_better', 'scaling', 'vs_baseline', 'dtype', 'data', 'config',
        'roofline'}


def run_bench(*flags, timeout=300):
  return subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), *flags],
                        cwd=ROOT, capture_output=True, text=True,
                        timeout=timeout)


def test_more_than_one_gpu_is_refused_with_a_message():
  r = run_bench('--gpus', '2', timeout=60)
  assert r.returncode == 2
  assert 'ONE GPU' in r.stderr and r.stdout.strip() == ''


@pytest.mark.gpu
@pytest.mark.parametrize('flags', [
    ('--stage', 'dense'),
    ('--stage', 'memory'),
])
def test_short_stages_print_one_json_line(flags):
  r = run_bench(*flags)
  assert r.returncode == 0, r.stderr[-2000:]
  lines = [l for l in r.stdout.splitlines() if l.strip()]
  assert len(lines) == 1
  out = json.loads(lines[0])
  assert KEYS <= set(out), KEYS - set(out)
  assert out['n_gpus'] == 1 and out['value'] > 0
  assert 'workload' in out['config'] and 'model' not in out['config']
  roof = out['roofline']
  assert roof['bound'] in ('hbm', 'mfma') and 0 < roof['frac'] <= 1.0
  assert abs(roof['frac'] - roof['achieved'] / roof['peak']) < 1e-3
