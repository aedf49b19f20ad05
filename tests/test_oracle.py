"""Pins the CPU oracle (the checker of the GPU parity tests) without a GPU.

The reference's Adam arithmetic and loss scaler live in a dependency that is not available
offline, so the oracle is pinned against what is: the committed golden vectors (outputs of
torch's CPU ops, tests/golden/make_golden.py), live torch CPU ops on larger random inputs,
float64 closed forms, brute force and special cases chosen so that a dropped term, a wrong sign
or a swapped operand fails at least one of them.
"""
import math
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle.torch_ref import TorchCpuStep

from helpers import seeds

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'step_cases.npz')
CODE = {'f32': O.F32, 'f16': O.F16, 'bf16': O.BF16}
TORCH = {'f32': torch.float32, 'f16': torch.float16, 'bf16': torch.bfloat16}


@pytest.fixture(scope='module')
def golden():
    return np.load(GOLDEN)


def ordered(bits):
    b = bits.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)


def bits_of(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


# ------------------------------------------------------------------------------------------------
# golden vectors
# ------------------------------------------------------------------------------------------------


def test_golden_adam_cases(oracle, golden):
    """m and v must reproduce torch's CPU Adam bit for bit; p within 1e-6 of the step size (torch's
    CPU sqrt is not correctly rounded for a fraction of a percent of inputs, the oracle's is);
    the low-precision copy within 1 ulp; the squared norm within 1e-6."""
    for entry in golden['case_names']:
        name, dt = str(entry).split(':')
        n, adamw, wd, b1, b2, div_scale, steps = golden[f'{name}/meta']
        p, m, v = (golden[f'{name}/{k}_init'].copy() for k in 'pmv')
        for s in range(int(steps)):
            g = golden[f'{name}/g{s}']
            oracle.adam(g, CODE[dt], p, m, v, lr=1e-3, beta1=b1, beta2=b2, eps=1e-8, weight_decay=wd, step=s + 1,
                        adamw_mode=bool(adamw), div_scale=float(div_scale))
            assert np.array_equal(m.view(np.uint32), golden[f'{name}/m_out{s}'].view(np.uint32)), f'{name} m step {s}'
            assert np.array_equal(v.view(np.uint32), golden[f'{name}/v_out{s}'].view(np.uint32)), f'{name} v step {s}'
            want_p = golden[f'{name}/p_out{s}']
            assert np.all(np.abs(p.astype(np.float64) - want_p) <= 1e-6 * np.abs(want_p) + 1e-6 * 1e-3), f'{name} p step {s}'
            assert (p.view(np.uint32) != want_p.view(np.uint32)).mean() < 0.01
            if dt != 'f32':
                lowp = oracle.writeback(p, CODE[dt])
                assert np.max(np.abs(ordered(lowp) - ordered(golden[f'{name}/lowp{s}']))) <= 1
            l2 = oracle.l2norm_sq_ref(g, CODE[dt])
            assert math.isclose(l2, float(golden[f'{name}/l2_{s}']), rel_tol=1e-6)
            # continue from torch's state so that every step is an independent single-step check
            p = want_p.copy()


def test_golden_overflow_flags(oracle, golden):
    for dt in ('f16', 'bf16', 'f32'):
        for label in ('clean', 'pinf_first', 'ninf_last', 'nan_mid', 'largest_finite'):
            g = golden[f'overflow/{dt}/{label}/g']
            assert oracle.overflow(g, CODE[dt]) == bool(golden[f'overflow/{dt}/{label}/flag']), (dt, label)


def test_golden_casts(oracle, golden):
    x = golden['cast/x']
    assert np.array_equal(oracle.writeback(x, O.F16), golden['cast/f16'])
    assert np.array_equal(oracle.writeback(x, O.BF16), golden['cast/bf16'])


def test_golden_scaler_trajectories(oracle, golden):
    """With hysteresis 1 and no clamp hit the scaler is torch's own scale update rule."""
    for label in ('clean_growth', 'one_overflow', 'burst', 'alternating'):
        sc = O.DynamicGradScalerOracle(initial_scale=1024.0, growth_factor=2, backoff_factor=0.5, growth_interval=3,
                                       hysteresis=1)
        got = []
        for f in golden[f'scaler/{label}/found']:
            sc.update(bool(f))
            got.append(float(sc.scale))
        assert got == list(golden[f'scaler/{label}/scale']), label


# ------------------------------------------------------------------------------------------------
# codecs
# ------------------------------------------------------------------------------------------------


def test_upcast_of_every_16bit_pattern(oracle):
    allbits = np.arange(65536, dtype=np.uint16)
    for code, td in ((O.F16, torch.float16), (O.BF16, torch.bfloat16)):
        got = oracle.lowp_to_f32(allbits, code)
        want = torch.from_numpy(allbits.view(np.int16).copy()).view(td).float().numpy()
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_downcast_random_bit_patterns_and_round_trip(oracle):
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint32).view(np.float32)
    nan = np.isnan(x)
    for code, td in ((O.F16, torch.float16), (O.BF16, torch.bfloat16)):
        got = oracle.writeback(x, code)
        want = bits_of(torch.from_numpy(x.copy()).to(td))
        assert np.array_equal(got[~nan], want[~nan])
        assert np.all(np.isnan(oracle.lowp_to_f32(got[nan], code)))
        # every representable value survives a round trip exactly
        allbits = np.arange(65536, dtype=np.uint16)
        up = oracle.lowp_to_f32(allbits, code)
        keep = ~np.isnan(up)
        assert np.array_equal(oracle.writeback(up, code)[keep], allbits[keep])


def test_downcast_ties_to_even_and_saturation(oracle):
    # halfway between 1.0 and the next fp16 (1 + 2^-11) ties to even = 1.0; just above rounds up
    f = np.array([1.0 + 2.0**-11, 1.0 + 2.0**-11 + 2.0**-20, 1.0 + 3 * 2.0**-11, 65519.9, 65520.0, -65520.0, 2.0**-25,
                  2.0**-25 * 1.0001, 0.0, -0.0], dtype=np.float32)
    got = oracle.writeback(f, O.F16)
    assert list(got) == [0x3C00, 0x3C01, 0x3C02, 0x7BFF, 0x7C00, 0xFC00, 0x0000, 0x0001, 0x0000, 0x8000]


# ------------------------------------------------------------------------------------------------
# Adam / AdamW
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize('adamw,wd,betas', [(False, 0.0, (0.9, 0.999)), (True, 0.01, (0.9, 0.999)),
                                            (False, 0.01, (0.9, 0.999)), (True, 0.1, (0.4, 0.95))])
def test_adam_against_live_torch_cpu(oracle, adamw, wd, betas):
    n = 200_003
    torch.manual_seed(1)
    p0 = torch.randn(n) * 0.02
    tp = torch.nn.Parameter(p0.clone())
    topt = (torch.optim.AdamW if adamw else torch.optim.Adam)([tp], lr=1e-3, betas=betas, eps=1e-8, weight_decay=wd,
                                                              foreach=False)
    p, m, v = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(1, 4):
        g = torch.randn(n) * 1e-2
        tp.grad = g.clone()
        topt.step()
        oracle.adam(g.numpy().copy(), O.F32, p, m, v, lr=1e-3, beta1=betas[0], beta2=betas[1], eps=1e-8, weight_decay=wd,
                    step=step, adamw_mode=adamw)
        st = topt.state[tp]
        want_p = tp.data.numpy()
        assert np.all(np.abs(p.astype(np.float64) - want_p) <= 1e-6 * np.abs(want_p) + 1e-9)
        gmax = float(g.abs().max())
        assert np.all(np.abs(m.astype(np.float64) - st['exp_avg'].numpy()) <= 1e-6 * np.abs(m) + 1e-6 * gmax)
        assert np.all(np.abs(v.astype(np.float64) - st['exp_avg_sq'].numpy()) <= 1e-6 * np.abs(v) + 1e-6 * gmax**2)
        # resynchronise so that each step is an independent single-step comparison
        p[:], m[:], v[:] = want_p, st['exp_avg'].numpy(), st['exp_avg_sq'].numpy()


@pytest.mark.parametrize('seed', seeds(12))
def test_adam_against_live_torch_cpu_random_hypers(oracle, seed):
    """Hyper-parameters drawn at random, the edges included (beta1 of 0 and exactly 0.5, where torch's
    lerp changes formula; beta2 of 0; a large eps; no decay): every step compared on its own."""
    rng = np.random.default_rng(4200 + seed)
    n = 20_011
    adamw = bool(rng.integers(2))
    lr = float(rng.choice([1e-5, 1e-3, 3e-2, 1.0]))
    beta1 = float(rng.choice([0.0, 0.3, 0.5, 0.9, 0.99]))
    beta2 = float(rng.choice([0.0, 0.5, 0.95, 0.999]))
    eps = float(rng.choice([1e-12, 1e-8, 1e-3]))
    wd = float(rng.choice([0.0, 1e-4, 0.1]))
    torch.manual_seed(seed)
    p0 = torch.randn(n) * 0.02
    tp = torch.nn.Parameter(p0.clone())
    topt = (torch.optim.AdamW if adamw else torch.optim.Adam)([tp], lr=lr, betas=(beta1, beta2), eps=eps,
                                                              weight_decay=wd, foreach=False)
    p, m, v = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(1, 5):
        g = torch.randn(n) * float(rng.choice([1e-4, 1e-2, 1.0]))
        tp.grad = g.clone()
        topt.step()
        oracle.adam(g.numpy().copy(), O.F32, p, m, v, lr=lr, beta1=beta1, beta2=beta2, eps=eps, weight_decay=wd,
                    step=step, adamw_mode=adamw)
        st = topt.state[tp]
        want_p, want_m, want_v = tp.data.numpy(), st['exp_avg'].numpy(), st['exp_avg_sq'].numpy()
        gmax = float(g.abs().max())
        what = f'seed {seed} step {step} adamw {adamw} lr {lr} betas {(beta1, beta2)} eps {eps} wd {wd}'
        # p = p - step: the bound is relative to the operands (|p| and the step size lr)
        assert np.all(np.abs(p.astype(np.float64) - want_p) <= 1e-6 * (np.abs(want_p) + lr)), what
        assert np.all(np.abs(m.astype(np.float64) - want_m) <= 1e-6 * (np.abs(want_m) + gmax)), what
        assert np.all(np.abs(v.astype(np.float64) - want_v) <= 1e-6 * (np.abs(want_v) + gmax**2)), what
        p[:], m[:], v[:] = want_p, want_m, want_v


@pytest.mark.parametrize('beta1', [0.0, 0.3, 0.5, 0.9])
def test_adam_signed_zero_moments_match_live_torch(oracle, beta1):
    """Gradients of +0 and -0: the sign of a zero exp_avg depends on how the lerp coefficient of the
    second form is computed (weight - 1, as torch's vectorised kernel does, against -(1 - weight));
    with beta1 = 0 the two differ.  exp_avg and exp_avg_sq must carry torch's bits."""
    n = 4096
    torch.manual_seed(0)
    p0 = torch.randn(n) * 0.02
    g = torch.randn(n) * 1e-2
    g[::3] = 0.0
    g[1::7] = -0.0
    tp = torch.nn.Parameter(p0.clone())
    topt = torch.optim.Adam([tp], lr=1e-3, betas=(beta1, 0.999), foreach=False)
    p, m, v = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in (1, 2, 3):
        gg = g.clone() if step != 2 else -g
        tp.grad = gg.clone()
        topt.step()
        oracle.adam(gg.numpy().copy(), O.F32, p, m, v, lr=1e-3, beta1=beta1, beta2=0.999, eps=1e-8, weight_decay=0.0,
                    step=step, adamw_mode=False)
        st = topt.state[tp]
        assert np.array_equal(st['exp_avg'].numpy().view(np.uint32), m.view(np.uint32)), f'beta1 {beta1} step {step}'
        assert np.array_equal(st['exp_avg_sq'].numpy().view(np.uint32), v.view(np.uint32)), f'beta1 {beta1} step {step}'
        if beta1 == 0.0:
            assert np.array_equal(m.view(np.uint32), gg.numpy().view(np.uint32))    # exp_avg is the gradient, sign of zero included
        p[:] = tp.data.numpy()


def test_adam_fp32_tracks_float64_closed_form(oracle):
    """A wrong sign, a dropped bias correction or a transposed beta shows up at the 1e-2 level
    here; fp32 rounding stays below 1e-5 of the operand sizes."""
    rng = np.random.default_rng(2)
    n = 50_000
    for adamw, wd, step in ((True, 0.1, 1), (True, 0.1, 7), (False, 0.05, 3), (True, 0.0, 1000)):
        p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        m = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        v = (rng.random(n) * 1e-5).astype(np.float32)
        g = (rng.standard_normal(n) * 0.3).astype(np.float32)
        kw = dict(lr=3e-3, beta1=0.8, beta2=0.99, eps=1e-8, weight_decay=wd, step=step, adamw_mode=adamw)
        p64, m64, v64 = oracle.adam_f64(g, O.F32, p, m, v, div_scale=3.0, **kw)
        oracle.adam(g, O.F32, p, m, v, div_scale=3.0, **kw)
        assert np.max(np.abs(p - p64)) <= 1e-5 * 0.02
        assert np.max(np.abs(m - m64)) <= 1e-5 * 0.1
        assert np.max(np.abs(v - v64)) <= 1e-5 * 0.01


def test_first_step_is_sign_descent_and_zero_grad_is_a_fixed_point(oracle):
    n = 1000
    rng = np.random.default_rng(3)
    g = rng.standard_normal(n).astype(np.float32)
    p, m, v = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32)
    oracle.adam(g, O.F32, p, m, v, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, step=1, adamw_mode=True)
    assert np.allclose(p, -1e-3 * np.sign(g), rtol=1e-4, atol=0)    # textbook: p -= lr * g/(|g|+eps)
    assert np.allclose(m, 0.1 * g, rtol=1e-6) and np.allclose(v, 0.001 * g * g, rtol=1e-6)

    p0 = rng.standard_normal(n).astype(np.float32)
    p, m, v = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    oracle.adam(np.zeros(n, np.float32), O.F32, p, m, v, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0,
                step=5, adamw_mode=True)
    assert np.array_equal(p, p0) and not m.any() and not v.any()
    # the allocation step: g == NULL, decoupled decay shrinks p once
    p = p0.copy()
    oracle.adam(None, O.F32, p, m, v, lr=1e-2, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.5, step=1,
                adamw_mode=True)
    assert np.array_equal(p, p0 * np.float32(1 - 1e-2 * 0.5))


def test_unscale_is_a_true_division(oracle):
    n = 4096
    rng = np.random.default_rng(4)
    gbits = rng.integers(0, 0x7C00, size=n, dtype=np.uint16)    # finite positive fp16 values
    for scale in (64.0, 65536.0, 3.0, 5379818.327114731):
        p, m, v = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32)
        oracle.adam(gbits, O.F16, p, m, v, lr=1e-3, beta1=0.0, beta2=0.999, eps=1e-8, weight_decay=0.0, step=1,
                    adamw_mode=True, div_scale=scale)
        # beta1 = 0 makes exp_avg the unscaled gradient itself
        want = oracle.lowp_to_f32(gbits, O.F16) / np.float32(scale)
        assert np.array_equal(m.view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_torch_cpu_step_harness_agrees_with_reference_step(oracle):
    """The two restatements of the whole step (numpy + C oracle, and plain torch CPU ops) agree on a
    clipped AdamW fp16 step, including the skip on overflow."""
    n = 30_000
    torch.manual_seed(5)
    master = torch.randn(n) * 0.02
    m0, v0 = torch.randn(n) * 1e-4, torch.rand(n) * 1e-6
    g = (torch.randn(n) * 5e-2 * 64).to(torch.float16)
    ref = TorchCpuStep(master, torch.float16, lr=1e-3, weight_decay=0.1, exp_avg=m0, exp_avg_sq=v0)
    chunk = O.OracleChunk(lowp=bits_of(g), master=master.numpy().copy(), m=m0.numpy().copy(), v=v0.numpy().copy(),
                          valid_end=n, segments=[O.OracleSegment(0, n, weight_decay=0.1)])
    scaler = O.DynamicGradScalerOracle(initial_scale=64.0, min_scale=1, max_scale=2**24, hysteresis=1)
    found, lowp = ref.step(g, loss_scale=64.0, max_norm=1.0)
    info = O.reference_step([chunk], O.F16, scaler, max_norm=1.0)
    assert found is False and info['found_inf'] is False and info['combined_scale'] > 64.0
    assert np.all(np.abs(chunk.master - ref.master.numpy()) <= 1e-6 * np.abs(chunk.master) + 1e-9)
    assert np.max(np.abs(ordered(chunk.lowp) - ordered(bits_of(lowp)))) <= 1

    g[123] = float('inf')
    before = chunk.master.copy()
    chunk.lowp[:] = bits_of(g)
    found, _ = ref.step(g, loss_scale=64.0, max_norm=1.0)
    info = O.reference_step([chunk], O.F16, scaler, max_norm=1.0)
    assert found is True and info['found_inf'] is True and info['loss_scale'] == 32.0
    assert np.array_equal(chunk.master, before)
    assert np.array_equal(chunk.lowp, oracle.writeback(before, O.F16))


# ------------------------------------------------------------------------------------------------
# flags and norms
# ------------------------------------------------------------------------------------------------


def test_overflow_brute_force_small(oracle):
    rng = np.random.default_rng(6)
    for code, td in ((O.F16, torch.float16), (O.BF16, torch.bfloat16)):
        for _ in range(200):
            bits = rng.integers(0, 65536, size=rng.integers(1, 40), dtype=np.uint16)
            t = torch.from_numpy(bits.view(np.int16).copy()).view(td)
            want = bool(torch.isinf(t).any() | torch.isnan(t).any())
            assert oracle.overflow(bits, code) == want
    assert oracle.overflow(np.zeros(0, np.uint16), O.F16) is False


def test_norm_is_additive_and_matches_the_chunk_test_identity(oracle):
    """test/chunk/test_chunk.py:66-73: the per-chunk l2_norm equals payload.float().norm(2)**2; the
    optimizer adds the per-chunk values (optimizer.py:149-161)."""
    torch.manual_seed(7)
    x = torch.randn(4, 1000)
    parts = [oracle.l2norm_sq_ref(x[i].numpy().copy(), O.F32) for i in range(4)]
    whole = float(x.flatten().float().norm(2)**2)
    assert math.isclose(sum(parts), whole, rel_tol=1e-6)
    xs = x.flatten().numpy().astype(np.float64)
    assert math.isclose(oracle.sumsq(x.flatten().numpy().copy(), O.F32), float(np.dot(xs, xs)), rel_tol=1e-12)
    h = (torch.randn(5000) * 100).to(torch.float16)
    assert math.isclose(oracle.l2norm_sq_ref(bits_of(h), O.F16), float(h.float().norm(2).item()**2), rel_tol=1e-6)


# ------------------------------------------------------------------------------------------------
# host scalars, scaler, layout
# ------------------------------------------------------------------------------------------------


def test_combined_scale_rules():
    assert O.combined_scale(1.0, None, 0.0) == -1                       # nothing to do
    assert O.combined_scale(64.0, None, 0.0) == 64.0                    # loss scale only
    assert O.combined_scale(64.0, 32.0, 1.0) == 64.0                    # unscaled norm 0.5 < 1: no clip
    c = O.combined_scale(64.0, 640.0, 1.0)                              # unscaled norm 10 -> divide by 10 more
    assert math.isclose(c, 64.0 * (10.0 + 1e-6), rel_tol=1e-15)
    # effective gradient g/combined has norm max_norm * n/(n + 1e-6)
    assert math.isclose(640.0 / c, 10.0 / (10.0 + 1e-6), rel_tol=1e-12)
    assert O.combined_scale(1.0, 0.5, 2.0) == -1


def test_global_norm_passes_through_fp32(oracle):
    # the float64 sum 9 + 2**-30 is not an fp32 number: the one-element fp32 buffer of
    # optimizer.py:158-162 rounds it to 9, so the norm is exactly 3 (without the detour it would be
    # 3.0000000001552...)
    assert oracle.global_norm([1.0 + 2.0**-30, 3.0, 5.0]) == 3.0
    assert math.sqrt(1.0 + 2.0**-30 + 3.0 + 5.0) != 3.0
    # and the square root is taken in float64, not in fp32: sqrt(2) keeps all its digits
    assert oracle.global_norm([0.5, 1.5]) == 1.4142135623730951


def test_scaler_hysteresis_and_clamps():
    sc = O.DynamicGradScalerOracle(initial_scale=64.0, min_scale=16.0, max_scale=128.0, growth_interval=2, hysteresis=2)
    seq = [True, True, True, True, False, False, False, False, True]
    want = [64.0, 32.0, 16.0, 16.0, 16.0, 32.0, 32.0, 64.0, 64.0]
    got = []
    for f in seq:
        sc.update(f)
        got.append(float(sc.scale))
    assert got == want
    const = O.ConstantGradScalerOracle(1.0)
    const.update(True)
    assert float(const.scale) == 1.0


# The state machine's corner cases as literals.  Every product is rounded to fp32 (the scale is a
# one-element fp32 tensor): 3 * fp32(1.1) = 3.30000007152557373046875 is an exact tie between two fp32
# neighbours and goes to the even one, 3.3000001907348633 -- float64 arithmetic would give
# 3.3000000000000003, fp32(3.3) is 3.299999952316284.
SCALER_LITERALS = [
    # (constructor arguments, overflow sequence, scale after every update)
    (dict(initial_scale=64.0, hysteresis=0), [True, True, False], [32.0, 16.0, 16.0]),
    (dict(initial_scale=64.0, hysteresis=1), [True, True, False], [32.0, 16.0, 16.0]),
    (dict(initial_scale=64.0, hysteresis=3), [True, True, True, True], [64.0, 64.0, 32.0, 16.0]),
    # back-off landing exactly on min_scale, then held there
    (dict(initial_scale=32.0, hysteresis=1, min_scale=16.0), [True, True, True], [16.0, 16.0, 16.0]),
    # back-off that would pass below min_scale is clamped to it
    (dict(initial_scale=24.0, hysteresis=1, min_scale=16.0), [True, True], [16.0, 16.0]),
    # growth landing exactly on max_scale, then held there
    (dict(initial_scale=64.0, growth_interval=1, max_scale=128.0), [False, False, False], [128.0, 128.0, 128.0]),
    # growth that would pass above max_scale is clamped to it
    (dict(initial_scale=96.0, growth_interval=1, max_scale=128.0), [False, False], [128.0, 128.0]),
    # an overflow resets the growth counter; a growth resets the hysteresis counter
    (dict(initial_scale=64.0, growth_interval=2, hysteresis=2), [False, True, False, False, True, True],
     [64.0, 64.0, 64.0, 128.0, 128.0, 64.0]),
    # factors that are not powers of two, rounded to fp32 at every step
    (dict(initial_scale=3.0, growth_factor=1.1, growth_interval=1), [False] * 4,
     [3.3000001907348633, 3.630000352859497, 3.9930005073547363, 4.392300605773926]),
    (dict(initial_scale=1000.0, backoff_factor=0.3, hysteresis=1), [True] * 4,
     [300.0, 90.0, 27.000001907348633, 8.100001335144043]),
]


@pytest.mark.parametrize('case', range(len(SCALER_LITERALS)))
def test_scaler_corner_cases_as_literals(case):
    kwargs, seq, want = SCALER_LITERALS[case]
    sc = O.DynamicGradScalerOracle(**kwargs)
    got = []
    for f in seq:
        sc.update(f)
        got.append(float(sc.scale))
    assert got == want


def test_the_fp32_tie_of_the_scaler_literal_by_exact_arithmetic():
    from fractions import Fraction
    exact = Fraction(float(np.float32(1.1))) * 3
    lo, hi = Fraction(float.fromhex('0x1.a66666p+1')), Fraction(float.fromhex('0x1.a66668p+1'))
    assert exact - lo == hi - exact                      # a tie ...
    assert float(hi) == 3.3000001907348633               # ... that goes to the neighbour with the even mantissa
    assert int(np.float32(float(hi)).view(np.uint32)) % 2 == 0 and int(np.float32(float(lo)).view(np.uint32)) % 2 == 1


def test_simple_search_known_answer():
    """The reference's own fixture for its chunk plans, test/search/test_simple.py:29-42: the `small`
    model of test/utils/small.py (embedding 20 x 16 tied to the output projection, LayerNorm 16, an MLP
    16 -> 64 -> 16, LayerNorm 16) under simple_search(group_size=1, split_number=5) gets one private
    chunk of 320 for the tied embedding and five public chunks of 1088 with these name lists.  (The
    fixture pins the split-by-count rule and the private/public split; the greedy rule of
    mini_waste.py:78-96 has no fixture in the reference and is pinned by test_greedy_packing_rule.)"""
    named = [('embed.weight', 20 * 16), ('norm1.weight', 16), ('norm1.bias', 16), ('mlp.proj1.weight', 64 * 16),
             ('mlp.proj1.bias', 64), ('mlp.proj2.weight', 16 * 64), ('mlp.proj2.bias', 16), ('norm2.weight', 16),
             ('norm2.bias', 16)]    # named_parameters() order; proj.weight is embed.weight
    names = [n for n, _ in named]
    sizes = [s for _, s in named]
    private_sizes, groups, block = O.simple_pack(sizes, [n == 'embed.weight' for n in names], 1, 5)
    assert private_sizes == [320] and block == 1088
    assert [[names[i] for i in g] for g in groups] == [['norm1.weight', 'norm1.bias'],
                                                       ['mlp.proj1.weight', 'mlp.proj1.bias'],
                                                       ['mlp.proj2.weight', 'mlp.proj2.bias'], ['norm2.weight'],
                                                       ['norm2.bias']]
    # rounding up to the group size (search/simple.py:26-30)
    assert O.simple_pack(sizes, [n == 'embed.weight' for n in names], 256, 5)[::2] == ([512], 1280)
    # fewer tensors than groups: one tensor per chunk
    assert O.simple_pack([5, 7], [False, False], 1, 10) == ([], [[0], [1]], 7)

    # the product's planner gives the same plans
    import elixir_amd as ea
    sr = ea.simple_search(named, 1, 5, torch.float16, private_names=['embed.weight'])
    plans = sr.param_chunk_plans
    assert plans[0].name_list == ['embed.weight'] and plans[0].chunk_size == 320 and plans[0].kwargs['rcache_fused']
    assert [p.name_list for p in plans[1:]] == [[names[i] for i in g] for g in groups]
    assert all(p.chunk_size == 1088 and not p.kwargs.get('rcache_fused') for p in plans[1:])


def test_greedy_packing_rule():
    from elixir_amd import shapes as S
    for fn, csize, n_chunks in ((S.gpt2_shapes, 64 << 20, 2), (S.opt_shapes, 128 << 20, 11), (S.llama_shapes, 256 << 20, 27)):
        sizes = [S.numel(s) for _, s in fn()]
        groups = O.greedy_pack(sizes, csize)
        assert len(groups) == n_chunks
        assert [i for g in groups for i in g] == list(range(len(sizes)))        # order kept, nothing lost
        assert all(sum(sizes[i] for i in g) <= csize for g in groups)
        # a tensor only opens a new chunk when it does not fit the room left in the current one
        for a, b in zip(groups, groups[1:]):
            assert csize - sum(sizes[i] for i in a) < sizes[b[0]]
        # the waste the planner computes for this rule (search/utils.py, calc_waste)
        acc = left = 0
        for s in sizes:
            if s > left:
                acc += left
                left = csize
            left -= s
        assert left + acc == len(groups) * csize - sum(sizes)
    assert O.greedy_pack([3, 3, 3, 5, 1], 6) == [[0, 1], [2], [3, 4]]


def test_valid_end_and_range_rules():
    assert O.valid_end(960, 0, 1024) == 960
    assert O.valid_end(1024, 0, 1024) == 1025          # full shard keeps the sentinel
    assert O.valid_end(0, 0, 1024) == 0
    assert O.valid_end(700, 512, 512) == 188           # second shard of two, partly used
    assert O.valid_end(300, 512, 512) == 0
    assert O.range_pair(100, 300, 0, 1024) == (100, 300)
    assert O.range_pair(400, 700, 512, 512) == (0, 188)
    assert O.range_pair(100, 300, 512, 512)[0] >= O.range_pair(100, 300, 512, 512)[1]    # empty on this shard
    assert O.chunk_offsets([5, 7, 1]) == [(0, 5), (5, 12), (12, 13)]


# ------------------------------------------------------------------------------------------------
# gradient landing
# ------------------------------------------------------------------------------------------------


def _special_payload(n, dtype, seed):
    """Random values across the whole range of the type plus the special ones."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, generator=g) * torch.exp(torch.randn(n, generator=g) * 6.0)
    x[:12] = torch.tensor([0.0, -0.0, float('inf'), float('-inf'), float('nan'), 65504.0, 65520.0, -65536.0, 6e-8,
                           -6.1e-5, 1e-40, 3.3e38])
    return x.to(dtype)


@pytest.mark.parametrize('dtype', ['f16', 'bf16', 'f32'])
def test_landing_same_type_moves_the_bits(oracle, dtype):
    # every 16-bit pattern (signalling NaNs included) comes out as it went in
    if dtype == 'f32':
        src = np.random.default_rng(0).integers(0, 2**32, 100000, dtype=np.uint64).astype(np.uint32).view(np.float32)
        out = oracle.land(src, CODE[dtype], CODE[dtype])
        assert np.array_equal(out.view(np.uint32), src.view(np.uint32))
    else:
        src = np.arange(65536, dtype=np.uint16)
        assert np.array_equal(oracle.land(src, CODE[dtype], CODE[dtype]), src)


@pytest.mark.parametrize('dtype', ['f16', 'bf16'])
def test_landing_from_fp32_is_torchs_cast(oracle, dtype):
    x = _special_payload(200000, torch.float32, 1)
    want = bits_of(x.to(TORCH[dtype]))
    got = oracle.land(x.numpy().copy(), O.F32, CODE[dtype])
    nan = np.isnan(x.numpy())
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(oracle.lowp_to_f32(got[nan], CODE[dtype])))


@pytest.mark.parametrize('dtype', ['f16', 'bf16', 'f32'])
@pytest.mark.parametrize('pg', [2, 4, 8, 64])
def test_landing_scaled_by_a_power_of_two_is_torchs_inplace_division(oracle, dtype, pg):
    # payload /= pg_size (chunk.py:299): for a power of two the division and the multiplication by
    # the reciprocal are the same correctly rounded result, so torch's CPU division pins it
    x = _special_payload(200000, TORCH[dtype], pg)
    want = x.clone()
    want /= pg
    src = bits_of(x)
    got = oracle.land(src, CODE[dtype], CODE[dtype], mul=1.0 / pg)
    wb = bits_of(want)
    if dtype == 'f32':
        nan = np.isnan(wb)
        assert np.array_equal(got.view(np.uint32)[~nan], wb.view(np.uint32)[~nan]) and np.all(np.isnan(got[nan]))
    else:
        nan = np.isnan(oracle.lowp_to_f32(wb, CODE[dtype]))
        assert np.array_equal(got[~nan], wb[~nan])
        assert np.all(np.isnan(oracle.lowp_to_f32(got[nan], CODE[dtype])))


@pytest.mark.parametrize('dtype', ['f16', 'bf16'])
def test_landing_fp32_payload_scaled_then_cast(oracle, dtype):
    # the always-fp32 reduction (chunk.py:291-299,314): fp32 payload / pg, then shard.copy_ casts
    x = _special_payload(100000, torch.float32, 9)
    want = x.clone()
    want /= 4
    wb = bits_of(want.to(TORCH[dtype]))
    got = oracle.land(x.numpy().copy(), O.F32, CODE[dtype], mul=0.25)
    nan = np.isnan(x.numpy())
    assert np.array_equal(got[~nan], wb[~nan])


def test_landing_rounds_twice_not_once(oracle):
    # a value where rounding the product to fp16 first matters is impossible for powers of two, so
    # use mul = 1/3: (fp16(x) * f32(1/3)) -> fp16 must equal the two-step result computed with numpy
    x = np.random.default_rng(4).standard_normal(50000).astype(np.float16)
    third = np.float32(1.0) / np.float32(3.0)
    want = (x.astype(np.float32) * third).astype(np.float16)
    got = oracle.land(x.view(np.uint16), O.F16, O.F16, mul=float(third))
    assert np.array_equal(got, want.view(np.uint16))


def test_golden_landing(oracle, golden):
    """Committed vectors from torch's CPU ops: payload / group size, the copy into the shard, flags."""
    n_checked = 0
    for key in golden.files:
        parts = key.split('/')
        if parts[0] != 'land' or len(parts) != 5:
            continue
        _, sd, label, pg, dd = parts
        x = golden[f'land/{sd}/{label}/x']
        want = golden[key]
        got = oracle.land(x, CODE[sd], CODE[dd], mul=1.0 / int(pg[2:]))
        if dd == 'f32':
            nan = np.isnan(want)
            assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan]), key
            assert np.all(np.isnan(got[nan])), key
        else:
            nan = np.isnan(oracle.lowp_to_f32(want, CODE[dd]))
            assert np.array_equal(got[~nan], want[~nan]), key
            assert np.all(np.isnan(oracle.lowp_to_f32(got[nan], CODE[dd]))), key
        assert oracle.overflow(got, CODE[dd]) == bool(golden[key + '/flag']), key
        if key + '/l2' in golden.files:
            assert math.isclose(oracle.l2norm_sq_ref(got, CODE[dd]), float(golden[key + '/l2']), rel_tol=2e-6), key
        n_checked += 1
    assert n_checked == 20
