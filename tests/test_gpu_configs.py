"""The two benchmark configurations that are not chunk-set throughput runs, at their full sizes:

  * configuration 1: plain fp32 Adam on one flat buffer of 16,777,216 elements (p ~ N(0, 0.02),
    g ~ N(0, 1e-2), m = v = 0, step 1, lr 1e-3, betas (0.9, 0.999), eps 1e-8, no weight decay, no
    loss scale) -- the case torch.optim.Adam runs on the CPU.  Every element is compared with the
    C oracle (identical bits) and with torch's CPU Adam (1e-6 relative);
  * configuration 3: the GPT-2-small chunk set (2 chunks of 64 Mi, fp16, loss scale 64) with about
    one gradient element per million replaced by +inf / -inf / NaN at seeded positions: the step
    must be skipped with master / exp_avg / exp_avg_sq untouched bit for bit, the low-precision
    shards restored, the loss scale halved (hysteresis 1) or held once and then halved
    (hysteresis 2), and a clean step at the new scale must then pass the numeric checks.
"""
import numpy as np
import pytest
import torch

import elixir_amd as ea
from elixir_amd import workloads
from oracle import oracle as O

from helpers import assert_close_f32, to_np, ulp_distance

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def test_config1_flat_fp32_adam_16mi(oracle):
    n = 1 << 24
    gen = torch.Generator(device='cpu')
    gen.manual_seed(1234 + 1)
    p0 = torch.randn(n, generator=gen) * 0.02
    p = torch.nn.Parameter(p0.clone().to(DEV))
    opt = ea.HybridAdam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    tp = torch.nn.Parameter(p0.clone())
    topt = torch.optim.Adam([tp], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    dp = torch.nn.Parameter(p0.clone().to(DEV))                       # torch's own Adam on the device
    dopt = torch.optim.Adam([dp], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, foreach=False)
    pn, mn, vn = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in (1, 2):
        g = torch.randn(n, generator=gen) * 1e-2
        p.grad = g.to(DEV)
        opt.step()                      # div_scale = -1: no unscale
        tp.grad = g.clone()
        topt.step()
        dp.grad = g.to(DEV)
        dopt.step()
        oracle.adam(g.numpy().copy(), O.F32, pn, mn, vn, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8,
                    weight_decay=0.0, step=step, adamw_mode=True)
        st = opt.state[p]
        assert st['step'] == step
        got = dict(p=to_np(p.data), m=to_np(st['exp_avg']), v=to_np(st['exp_avg_sq']))
        for name, want in (('p', pn), ('m', mn), ('v', vn)):
            assert np.array_equal(got[name].view(np.uint32), want.view(np.uint32)), f'step {step} {name} vs oracle'
        tst = topt.state[tp]
        gmax = float(g.abs().max())
        # exp_avg / exp_avg_sq: the same fused forms as torch's CPU kernels -> identical bits
        assert np.array_equal(got['m'].view(np.uint32), tst['exp_avg'].numpy().view(np.uint32))
        assert np.array_equal(got['v'].view(np.uint32), tst['exp_avg_sq'].numpy().view(np.uint32))
        # p: 1e-6 relative, with the step size lr as the scale of the cancelling operands
        assert_close_f32(got['p'], tp.data.numpy(), f'step {step} p vs torch', rtol=1e-6, atol=1e-6 * 1e-3)
        assert_close_f32(got['m'], tst['exp_avg'].numpy(), f'step {step} m', rtol=1e-6, atol=1e-6 * gmax)
        # and torch's Adam on the device (its kernels contract differently): the same 1e-6 bar
        dst = dopt.state[dp]
        assert_close_f32(got['p'], to_np(dp.data), f'step {step} p vs torch on the device', rtol=1e-6, atol=1e-6 * 1e-3)
        assert_close_f32(got['m'], to_np(dst['exp_avg']), f'step {step} m vs torch on the device', rtol=1e-6,
                         atol=1e-6 * gmax)
        assert_close_f32(got['v'], to_np(dst['exp_avg_sq']), f'step {step} v vs torch on the device', rtol=1e-6,
                         atol=1e-6 * gmax * gmax)


def _poison_per_million(built, seed):
    """ceil(N/1e6) gradient positions over the valid elements of all chunks, drawn with a seeded
    permutation, cycling +inf / -inf / NaN.  Returns the number of poisoned elements per chunk."""
    chunks = built.module.param_chunks
    sizes = [pc.n_valid for pc in chunks]
    total = sum(sizes)
    count = -(-total // 1_000_000)
    gen = torch.Generator(device='cpu')
    gen.manual_seed(seed)
    pos = torch.randperm(total, generator=gen)[:count].tolist()
    vals = [float('inf'), float('-inf'), float('nan')]
    per_chunk = [0] * len(chunks)
    for k, j in enumerate(pos):
        ci = 0
        while j >= sizes[ci]:
            j -= sizes[ci]
            ci += 1
        chunks[ci].shard[j] = vals[k % 3]
        per_chunk[ci] += 1
    return per_chunk


def _snapshot(built):
    out = []
    for pc in built.module.param_chunks:
        oc = pc.paired_chunk
        m, v = built.optimizer._binding.moments(oc)
        out.append((oc.shard.clone(), m.clone(), v.clone()))
    return out


def _assert_untouched(built, snap, dtype):
    for pc, (p0, m0, v0) in zip(built.module.param_chunks, snap):
        oc = pc.paired_chunk
        m, v = built.optimizer._binding.moments(oc)
        # bit for bit (torch.equal on the integer views, so that -0.0 / NaN patterns count too)
        assert torch.equal(oc.shard.view(torch.int32), p0.view(torch.int32))
        assert torch.equal(m.view(torch.int32), m0.view(torch.int32))
        assert torch.equal(v.view(torch.int32), v0.view(torch.int32))
        assert torch.equal(pc.shard.view(torch.int16), p0.to(dtype).view(torch.int16))


def _clean_step_matches_oracle(built, oracle, expect_scale, expect_step, width=8192):
    """A clean step, checked on seeded windows of every chunk against the C oracle."""
    opt, module = built.optimizer, built.module
    rng = np.random.default_rng(5)
    wins = []
    for ci, pc in enumerate(module.param_chunks):
        oc = pc.paired_chunk
        m, v = opt._binding.moments(oc)
        for b in sorted({0, max(0, pc.n_valid - width), *rng.integers(0, pc.n_valid - width, 4).tolist()}):
            e = b + width
            wins.append((ci, b, e, to_np(pc.shard[b:e]), to_np(oc.shard[b:e]), to_np(m[b:e]), to_np(v[b:e])))
    opt.step()
    info = opt.last_step_info
    assert info['found_inf'] is False and info['combined_scale'] == expect_scale
    assert all(st['step'] == expect_step for st in opt.state.values())
    for ci, b, e, g, p, m_, v_ in wins:
        pc = module.param_chunks[ci]
        oc = pc.paired_chunk
        m, v = opt._binding.moments(oc)
        # one weight-decay-free group with a single step count: the window is one flat Adam call
        # wherever it lies inside tensors; c2 has no padding before n_valid
        oracle.adam(g, O.F16, p, m_, v_, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0,
                    step=expect_step, adamw_mode=True, div_scale=float(expect_scale))
        assert np.array_equal(to_np(oc.shard[b:e]).view(np.uint32), p.view(np.uint32)), (ci, b)
        assert np.array_equal(to_np(m[b:e]).view(np.uint32), m_.view(np.uint32)), (ci, b)
        assert np.array_equal(to_np(v[b:e]).view(np.uint32), v_.view(np.uint32)), (ci, b)
        assert ulp_distance(to_np(pc.shard[b:e]), oracle.writeback(p, O.F16)) == 0
    for pc in module.param_chunks:
        assert torch.equal(pc.shard, pc.paired_chunk.shard.to(torch.float16))


@pytest.mark.parametrize('hysteresis', [1, 2])
def test_config3_overflow_on_gpt2_layout(oracle, hysteresis):
    spec = workloads.WORKLOADS['c2']
    assert spec.hysteresis == 1
    built = workloads.build('c2', seed=1234 + 3, hysteresis=hysteresis)
    opt, module, dtype = built.optimizer, built.module, spec.dtype
    assert len(module.param_chunks) == 2 and built.n_valid == 124_439_808
    scaler = O.DynamicGradScalerOracle(initial_scale=64.0, min_scale=1, max_scale=2**24, hysteresis=hysteresis)

    # ---- the poisoned step ----------------------------------------------------------------------
    built.land_gradients()
    per_chunk = _poison_per_million(built, seed=3)
    assert sum(per_chunk) == 125
    snap = _snapshot(built)
    opt.step()
    scaler.update(True)
    assert opt.last_step_info['found_inf'] is True
    assert [bool(f) for f in opt.last_step_info['chunk_overflow']] == [c > 0 for c in per_chunk]
    assert opt.loss_scale == scaler.scale == (32.0 if hysteresis == 1 else 64.0)
    assert all(st.get('step', 0) == 0 for st in opt.state.values())
    _assert_untouched(built, snap, dtype)

    if hysteresis == 2:    # the second overflow in a row backs off
        built.land_gradients()
        _poison_per_million(built, seed=4)
        opt.step()
        scaler.update(True)
        assert opt.last_step_info['found_inf'] is True
        assert opt.loss_scale == scaler.scale == 32.0
        _assert_untouched(built, snap, dtype)

    # ---- the clean follow-up at scale 32: the same gradients, scaled by 32 instead of 64 ---------
    for g in built.grads:
        g.mul_(0.5)
    built.land_gradients()
    _clean_step_matches_oracle(built, oracle, expect_scale=32.0, expect_step=1)
    scaler.update(False)
    assert opt.loss_scale == scaler.scale == 32.0
