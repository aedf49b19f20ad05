"""bench.py prints one JSON line with the agreed fields (run on the small GPT-2 chunk set)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_json_line():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--workload', 'c2', '--steps', '3',
                           '--warmup', '1', '--cpu-sample', str(1 << 20), '--landing-steps', '2'],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=280)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.startswith('{')]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ('metric', 'value', 'unit', 'n_gpus', 'steps', 'warmup', 'ms_per_step', 'higher_is_better', 'scaling',
                'vs_baseline', 'dtype', 'data', 'config', 'roofline', 'cpu_baseline'):
        assert key in out, key
    assert out['n_gpus'] == 1 and out['steps'] == 3 and out['warmup'] == 1 and out['vs_baseline'] is None
    assert out['config']['workload'].startswith('c2') and out['config']['valid_elements'] == 124_439_808
    assert abs(out['value'] - out['config']['valid_elements'] / (out['ms_per_step'] * 1e-3)) <= 1e-6 * out['value']
    r = out['roofline']
    assert r['bound'] == 'hbm' and r['peak'] == 8000.0 and r['unit'] == 'GB/s'
    assert abs(r['frac'] - r['achieved'] / r['peak']) < 1e-12 and 0 < r['frac'] < 1
    assert abs(r['achieved'] - r['bytes_per_launch'] / (r['ms_per_launch'] * 1e-3) / 1e9) <= 1e-6 * r['achieved']
    assert r['bytes_per_launch'] == 28 * out['config']['valid_elements']
    c = out['cpu_baseline']
    assert c['kind'] == 'port' and c['cores'] >= 1 and c['value'] > 0 and c['unit'] == 'elements/s'
    assert out['fused_landing']['ms_per_step'] > 0
    # the training flow: one landing launch per chunk, last chunk first, and still a step decided on the device
    per_chunk = out['fused_landing']['per_chunk_landing']
    assert per_chunk['launches'] == 2 and per_chunk['ms_per_step'] > 0
    per_tensor = out['fused_landing']['per_tensor_landing']
    assert per_tensor['ms_on_device'] > 0 and 0 < per_tensor['frac_of_hbm_peak'] < 1
    # configuration 3's timed part rides the c2 line: the step that finds an overflow
    skip = out['skip_step']
    assert skip['bytes_per_step'] == 2 * 124_439_808 + 6 * 134_217_728 and 0 < skip['frac'] < 1
    assert skip['loss_scale_after'] == 64.0 / 2**6    # 3 warm-up + 3 timed skipped steps, each halves the scale


def test_velocity_line():
    """The reference's flat-parameter micro-benchmark (profile/profile_optimizer.py:34-60) as a bench workload:
    10**9 fp32 elements, result checked against the closed form inside the run."""
    proc = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--workload', 'velocity', '--steps', '3',
                           '--warmup', '1'], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=280)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads([l for l in proc.stdout.splitlines() if l.startswith('{')][0])
    assert out['metric'] == 'adam_velocity' and out['config']['valid_elements'] == 10**9
    assert abs(out['vs_baseline'] - out['value'] / 50.0) < 1e-9
    assert abs(out['value'] - 1.0 / (out['ms_per_step'] * 1e-3)) <= 1e-6 * out['value']
    assert out['roofline']['bytes_per_launch'] == 28 * 10**9 and 0 < out['roofline']['frac'] < 1


def test_config1_line():
    """Configuration 1 (flat fp32 Adam, 16 Mi elements): the line's own figure is the step behind a copy that
    empties the memory-side cache, and it accounts for the step in microseconds: update launch, the floor any
    launch between two synchronisations costs, the host's own call."""
    proc = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--workload', 'c1', '--steps', '5',
                           '--warmup', '2', '--cpu-sample', '0'], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                          timeout=280)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads([l for l in proc.stdout.splitlines() if l.startswith('{')][0])
    assert out['config']['valid_elements'] == 1 << 24 and out['roofline']['bytes_per_launch'] == 28 << 24
    assert out['ms_per_step'] == out['step_cold_cache']['ms_per_step'] > 0
    acc = out['step_accounting_us']
    assert acc['steady_path_taken'] is True
    assert 0 < out['launch_sync_floor_us'] < 200 and 0 < out['host_us_in_step'] < 200
    assert abs(acc['step'] - acc['update_launch'] - acc['launch_sync_floor'] - acc['unaccounted']) < 1e-6
    assert out['step_state_in_cache']['ms_per_step'] > 0 and out['steps_back_to_back']['ms_per_step'] > 0
