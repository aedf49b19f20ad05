"""The HIP path against the committed golden vectors (tests/golden/step_cases.npz: outputs of
torch's CPU ops on small seeded inputs), through HybridAdam / the stats launch / the writeback."""
import math
import os

import numpy as np
import pytest
import torch

import elixir_amd as ea
from elixir_amd import _abi
from elixir_amd.chunk import l2_norm_from_sumsq, run_grad_stats

from helpers import from_bits, to_np, ulp_distance

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'step_cases.npz')
TORCH = {'f32': torch.float32, 'f16': torch.float16, 'bf16': torch.bfloat16}
CODE = {'f32': _abi.ELX_F32, 'f16': _abi.ELX_F16, 'bf16': _abi.ELX_BF16}
DEV = 'cuda'


@pytest.fixture(scope='module')
def golden():
    return np.load(GOLDEN)


def _to_dev(arr, dt):
    if dt == 'f32':
        return torch.from_numpy(arr.copy()).to(DEV)
    return from_bits(arr, TORCH[dt], DEV)


def _stats(t, n):
    row = np.zeros(1, dtype=_abi.CHUNK_DTYPE)
    row['grad'] = t.data_ptr()
    row['n_alloc'] = t.numel()
    row['n_valid'] = n
    rec = run_grad_stats(row, CODE[{torch.float32: 'f32', torch.float16: 'f16', torch.bfloat16: 'bf16'}[t.dtype]], t.device)
    return bool(rec['overflow'][0]), float(rec['sumsq'][0])


def test_adam_cases(golden):
    """exp_avg / exp_avg_sq: identical bits to torch's CPU Adam.  Master weights: within 1e-6 of the
    step size (torch's CPU sqrt is not correctly rounded for a fraction of a percent of inputs).
    Low-precision copy of the master: within 1 ulp.  Squared gradient norm: 1e-6 relative."""
    for entry in golden['case_names']:
        name, dt = str(entry).split(':')
        n, adamw, wd, b1, b2, div_scale, steps = golden[f'{name}/meta']
        p = torch.nn.Parameter(torch.from_numpy(golden[f'{name}/p_init'].copy()).to(DEV))
        p.grad_dtype = None
        opt = ea.HybridAdam([p], lr=1e-3, betas=(float(b1), float(b2)), eps=1e-8, weight_decay=float(wd),
                            adamw_mode=bool(adamw))
        st = opt.state[p]
        st['step'] = 0
        st['exp_avg'] = torch.from_numpy(golden[f'{name}/m_init'].copy()).to(DEV)
        st['exp_avg_sq'] = torch.from_numpy(golden[f'{name}/v_init'].copy()).to(DEV)
        for s in range(int(steps)):
            g = _to_dev(golden[f'{name}/g{s}'], dt)
            flag, sumsq = _stats(g, g.numel())
            assert flag is False
            assert math.isclose(l2_norm_from_sumsq(sumsq), float(golden[f'{name}/l2_{s}']), rel_tol=1e-6), name
            p.grad = g
            opt.step(div_scale=float(div_scale))
            assert np.array_equal(to_np(st['exp_avg']).view(np.uint32), golden[f'{name}/m_out{s}'].view(np.uint32)), name
            assert np.array_equal(to_np(st['exp_avg_sq']).view(np.uint32), golden[f'{name}/v_out{s}'].view(np.uint32)), name
            got, want = to_np(p.data), golden[f'{name}/p_out{s}']
            assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-6 * np.abs(want) + 1e-6 * 1e-3), f'{name} step {s}'
            # carry torch's master forward so every step is a single-step comparison
            p.data.copy_(torch.from_numpy(want.copy()))


def test_overflow_flags(golden):
    for dt in ('f16', 'bf16', 'f32'):
        for label in ('clean', 'pinf_first', 'ninf_last', 'nan_mid', 'largest_finite'):
            g = _to_dev(golden[f'overflow/{dt}/{label}/g'], dt)
            assert _stats(g, g.numel())[0] == bool(golden[f'overflow/{dt}/{label}/flag']), (dt, label)


def test_casts(golden):
    x = golden['cast/x']
    for dt in ('f16', 'bf16'):
        sr = ea.greedy_search([('w', x.size)], x.size, TORCH[dt])
        module = ea.ElixirModule({'w': (x.size, )}, sr, dtype=TORCH[dt])
        pc = module.param_chunks[0]
        pc.paired_chunk.shard.copy_(torch.from_numpy(x.copy()))
        pc.optim_update()
        assert np.array_equal(to_np(pc.shard), golden[f'cast/{dt}'])


def test_scaler_trajectories(golden):
    for label in ('clean_growth', 'one_overflow', 'burst', 'alternating'):
        sc = ea.DynamicGradScaler(initial_scale=1024.0, growth_factor=2, backoff_factor=0.5, growth_interval=3,
                                  hysteresis=1)
        got = []
        for f in golden[f'scaler/{label}/found']:
            sc.update(bool(f))
            got.append(sc.scale_value)
        assert got == list(golden[f'scaler/{label}/scale'])


def test_landing_vectors(golden):
    """The landing launch against the committed torch-CPU vectors: shard bits, flag, squared norm."""
    from elixir_amd.chunk import DeviceTable
    n_checked = 0
    for key in golden.files:
        parts = key.split('/')
        if parts[0] != 'land' or len(parts) != 5:
            continue
        _, sd, label, pg, dd = parts
        src = _to_dev(golden[f'land/{sd}/{label}/x'], sd)
        want = golden[key]
        dst = torch.zeros(src.numel(), dtype=TORCH[dd], device=DEV)
        row = np.zeros(1, dtype=_abi.CHUNK_DTYPE)
        row['grad'], row['lowp_out'], row['n_alloc'], row['n_valid'] = src.data_ptr(), dst.data_ptr(), src.numel(), src.numel()
        bpr = _abi.check_land_rows(row, None, CODE[sd], CODE[dd])
        rec = _abi.STATS_DTYPE.itemsize
        ws = torch.empty((_abi.land_workspace_records(1, bpr) + 1) * rec, dtype=torch.uint8, device=DEV)
        table = DeviceTable(row, dst.device)
        _abi.land_grads_mt(table.ptr, 1, CODE[sd], CODE[dd], float(np.float32(1.0 / int(pg[2:]))), bpr,
                           ws.data_ptr(), ws.data_ptr() + ws.numel() - rec, True, torch.cuda.current_stream().cuda_stream)
        stats = ws[-rec:].cpu().numpy().view(_abi.STATS_DTYPE)
        got = to_np(dst)
        if dd == 'f32':
            nan = np.isnan(want)
            assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan]), key
        else:
            nan = np.isnan(to_np(_to_dev(want, dd).float()))
            assert np.array_equal(got[~nan], want[~nan]), key
        assert bool(stats['overflow'][0]) == bool(golden[key + '/flag']), key
        if key + '/l2' in golden.files:
            l2 = float(np.float32(np.sqrt(stats['sumsq'][0])))**2
            assert abs(l2 - float(golden[key + '/l2'])) <= 2e-6 * float(golden[key + '/l2']), key
        n_checked += 1
    assert n_checked == 20
