"""Shared pieces of the parity tests: seeded chunk sets on the GPU and their oracle twins."""
import os

import numpy as np
import torch

import elixir_amd as ea
from elixir_amd import shapes as S
from oracle import oracle as O


def seeds(n: int) -> range:
    """Seeds of a randomised test: ``n`` in the committed suite, ``n + ELX_EXTRA_SEEDS`` when that
    environment variable is set (a long sweep: ``ELX_EXTRA_SEEDS=5000 python -m pytest tests -m gpu -k random``)."""
    return range(n + int(os.environ.get('ELX_EXTRA_SEEDS', '0')))

CODE = {torch.float32: O.F32, torch.float16: O.F16, torch.bfloat16: O.BF16}


def to_np(t: torch.Tensor) -> np.ndarray:
    """Device tensor -> numpy; 16-bit floats come back as uint16 bit patterns."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def from_bits(bits: np.ndarray, dtype: torch.dtype, device) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(dtype).to(device)


def ordered(bits: np.ndarray) -> np.ndarray:
    """Sign-magnitude 16-bit patterns -> integers ordered like the values (for ulp distances)."""
    b = bits.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)


def ulp_distance(a_bits: np.ndarray, b_bits: np.ndarray) -> int:
    if a_bits.size == 0:
        return 0
    return int(np.max(np.abs(ordered(a_bits) - ordered(b_bits))))


def assert_close_f32(got: np.ndarray, want: np.ndarray, name: str, rtol: float = 1e-6, atol: float = 0.0):
    """|got - want| <= atol + rtol*|want|, NaNs must coincide."""
    assert got.shape == want.shape, name
    nan_g, nan_w = np.isnan(got), np.isnan(want)
    assert np.array_equal(nan_g, nan_w), f'{name}: NaN pattern differs'
    ok = ~nan_w
    err = np.abs(got[ok].astype(np.float64) - want[ok].astype(np.float64))
    bound = atol + rtol * np.abs(want[ok].astype(np.float64))
    bad = err > bound
    assert not bad.any(), (f'{name}: {int(bad.sum())} of {got.size} elements outside rtol={rtol} atol={atol}; '
                           f'worst err {err.max():.3e}')


def build_workload(named_shapes, chunk_size, dtype, *, seed=0, grad_std=1e-3, loss_scale=1.0, lr=1e-3,
                   betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, adamw_mode=True, decay_exempt=True,
                   warm_state=True, device='cuda', host_resident=False, search_result=None, inner_cls=None, groups_of=None,
                   **opt_kwargs):
    """A synthetic chunk set on the GPU with seeded contents, its ElixirOptimizer, and the oracle's
    copy of the same data.  Gradients (already multiplied by ``loss_scale``) sit in the
    low-precision shards, as they do after backward.  ``groups_of``: a function from the list of
    (name, shape, parameter) to the parameter groups of the inner optimizer (default: one group with weight
    decay and one without)."""
    named_shapes = list(named_shapes)
    if search_result is not None:    # chunk plans made by the caller
        sr = search_result
    elif host_resident == 'mixed':    # every other chunk in pinned host memory, the rest on the GPU
        sr = ea.greedy_search([(n, S.numel(s)) for n, s in named_shapes], chunk_size, dtype)
        for plan in sr.param_chunk_plans[::2]:
            plan.kwargs.update(shard_device=torch.device('cpu'), cpu_pin_memory=True)
    elif host_resident:    # shards (and with them the moments) in pinned host memory
        sr = ea.greedy_search([(n, S.numel(s)) for n, s in named_shapes], chunk_size, dtype,
                              shard_device=torch.device('cpu'))
        for plan in sr.param_chunk_plans:
            plan.kwargs['cpu_pin_memory'] = True
    else:
        sr = ea.greedy_search([(n, S.numel(s)) for n, s in named_shapes], chunk_size, dtype)
    module = ea.ElixirModule(dict(named_shapes), sr, dtype=dtype)
    decay, exempt = [], []
    for (name, shape), p in zip(named_shapes, module.parameters()):
        (exempt if (decay_exempt and S.no_decay(name, shape)) else decay).append(p)
    groups = [dict(params=decay, weight_decay=weight_decay)]
    if exempt:
        groups.append(dict(params=exempt, weight_decay=0.0))
    if groups_of is not None:
        groups = groups_of([(name, shape, p) for (name, shape), p in zip(named_shapes, module.parameters())])
    inner = (inner_cls or ea.HybridAdam)(groups, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
                                         adamw_mode=adamw_mode)
    opt = ea.ElixirOptimizer(module, inner, **opt_kwargs)
    if opt.grad_scaler.scale_value != loss_scale:
        opt.grad_scaler._scale = np.float32(loss_scale)

    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    ochunks = []
    for pc in module.param_chunks:
        oc = pc.paired_chunk
        n, used = pc.shard_size, pc.utilized_size
        master = torch.zeros(n, dtype=torch.float32, device=device)
        master[:used] = torch.randn(used, generator=gen, device=device) * 0.02
        oc.shard.copy_(master)
        grads = torch.zeros(n, dtype=torch.float32, device=device)
        grads[:used] = torch.randn(used, generator=gen, device=device) * (grad_std * loss_scale)
        pc.shard.copy_(grads.to(dtype))
        m, v = opt._binding.moments(oc)
        if warm_state:
            m[:used] = torch.randn(used, generator=gen, device=device) * 1e-4
            v[:used] = torch.rand(used, generator=gen, device=device) * 1e-6
        segs = []
        for group in inner.param_groups:
            for fake in group['params']:
                if opt.param_to_optim_chunk[fake] is oc:
                    b, e = opt.param_to_range[fake]
                    segs.append(O.OracleSegment(b, e, lr=group['lr'], betas=tuple(group['betas']), eps=group['eps'],
                                                weight_decay=group['weight_decay'],
                                                bias_correction=group['bias_correction'], step=0))
        segs.sort(key=lambda s: s.begin)
        ochunks.append(O.OracleChunk(lowp=to_np(pc.shard), master=to_np(oc.shard), m=to_np(m), v=to_np(v),
                                     valid_end=pc.n_valid, segments=segs))
    return module, opt, ochunks


def refresh_oracle_grads(module, ochunks):
    """Copy the (new) gradients that sit in the GPU shards into the oracle's chunks."""
    for pc, oc in zip(module.param_chunks, ochunks):
        oc.lowp[:] = to_np(pc.shard)


def compare_state(module, opt, ochunks, dtype, *, exact=False, rtol=1e-6, atol_p=0.0, atol_m=0.0, atol_v=0.0, tag=''):
    """GPU chunk contents against the oracle's after a step.  Returns the worst ulp distance of the
    low-precision writeback."""
    worst_ulp = 0
    for i, (pc, oc) in enumerate(zip(module.param_chunks, ochunks)):
        fc = pc.paired_chunk
        m, v = opt._binding.moments(fc)
        got = dict(master=to_np(fc.shard), m=to_np(m), v=to_np(v))
        want = dict(master=oc.master, m=oc.m, v=oc.v)
        for name, atol in (('master', atol_p), ('m', atol_m), ('v', atol_v)):
            if exact:
                assert np.array_equal(got[name].view(np.uint32), want[name].view(np.uint32)), \
                    f'{tag} chunk {i} {name}: bits differ'
            else:
                assert_close_f32(got[name], want[name], f'{tag} chunk {i} {name}', rtol=rtol, atol=atol)
        lowp = to_np(pc.shard)
        if dtype == torch.float32:
            assert np.array_equal(lowp.view(np.uint32), oc.lowp.view(np.uint32)), f'{tag} chunk {i} fp32 writeback'
        else:
            d = ulp_distance(lowp, oc.lowp)
            worst_ulp = max(worst_ulp, d)
            assert d <= 1, f'{tag} chunk {i}: low-precision writeback off by {d} ulp'
    return worst_ulp
