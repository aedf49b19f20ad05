"""Host-resident shards: the deferred low-precision refresh fused into the source copy of the gather
(elixir/chunk/core/chunk.py:264-281, 403-421, 475-499).  After an update of a host-resident
optimizer chunk the parameter chunk is only marked out of sync; the next ``replicate`` produces the
low-precision slice of the block straight from the fp32 shard (the cast kernel reads pinned host
memory in place), and ``scatter`` brings the host shard back in sync.

Bar: the block equals the oracle's cast of the fp32 shard bit for bit (= torch's ``.to()``)."""
import numpy as np
import pytest
import torch

import elixir_amd as ea
from oracle import oracle as O

from helpers import CODE, to_np

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _pair(dtype, sizes, chunk_size, pinned):
    p = ea.Chunk(None, chunk_size, dtype, None, shard_device='cpu', temp_device='cpu', cpu_pin_memory=pinned)
    o = ea.Chunk(None, chunk_size, torch.float32, None, shard_device='cpu', temp_device='cpu', cpu_pin_memory=pinned)
    g = torch.Generator().manual_seed(sum(sizes))
    for n in sizes:
        t = torch.randn(n, generator=g) * 0.05
        p.append_tensor(t.to(dtype))
        o.append_tensor(t.clone())
    p.close_chunk()
    o.close_chunk()
    p.init_pair(o)
    assert p.shard.is_pinned() is pinned and o.shard.is_pinned() is pinned
    return p, o


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('pinned', [True, False])
def test_deferred_refresh_rides_the_gather_source_copy(oracle, dtype, pinned):
    sizes = [4097, 3, 15000, 1, 8191, 70001]
    p, o = _pair(dtype, sizes, 1 << 17, pinned)
    old = p.shard.clone()
    # an update of the host-resident master (what a step or a state load leaves behind)
    g = torch.Generator().manual_seed(1)
    o.shard[:sum(sizes)] = torch.randn(sum(sizes), generator=g) * 0.3
    o.shard[:6] = torch.tensor([0.0, -0.0, 65504.0, 65520.0, 1e-8, -3.0e38])
    p.optim_update()
    assert p.optim_sync_flag is False and torch.equal(p.shard, old)       # deferred: nothing moved yet

    block = torch.full((p.chunk_size,), 9.0, dtype=dtype, device=DEV)
    p.replicate(block)
    want = oracle.writeback(o.shard.numpy().copy(), CODE[dtype])
    assert np.array_equal(to_np(block), want)
    assert torch.equal(block.cpu(), o.shard.to(dtype))
    assert torch.equal(p.shard, old) and p.optim_sync_flag is False       # the host shard is refreshed on release

    p.scatter(block)
    assert p.optim_sync_flag is True
    assert torch.equal(p.shard, o.shard.to(dtype))

    # in sync again: the next gather is a plain transfer of the low-precision shard
    o.shard.add_(1.0)                                                     # must NOT show up
    block2 = torch.zeros(p.chunk_size, dtype=dtype, device=DEV)
    p.replicate(block2)
    assert torch.equal(block2, block)


def test_device_resident_chunks_gather_by_copy(oracle):
    named = [('w', (300, 40)), ('b', (40,))]
    sr = ea.greedy_search([(n, int(np.prod(s))) for n, s in named], 16384, torch.float16)
    module = ea.ElixirModule(dict(named), sr, dtype=torch.float16)
    pc = module.param_chunks[0]
    pc.paired_chunk.shard.normal_(0, 0.1)
    pc.optim_update()
    assert pc.optim_sync_flag is True
    block = torch.zeros(pc.chunk_size, dtype=torch.float16, device=DEV)
    pc.replicate(block)
    assert torch.equal(block, pc.paired_chunk.shard.half())
    pc.scatter(block)


def test_load_state_dict_into_host_resident_chunks():
    """module.py:294-344 with an offload placement: values go into the fp32 host shards, the refresh
    is deferred, and the parameters the forward pass sees come from the fused gather copy."""
    torch.manual_seed(0)
    net = torch.nn.Sequential(torch.nn.Linear(24, 48), torch.nn.LayerNorm(48), torch.nn.Linear(48, 10))
    named = [(n, p.numel()) for n, p in net.named_parameters()]
    sr = ea.greedy_search(named, 2048, torch.float16, shard_device=torch.device('cpu'))
    for plan in sr.param_chunk_plans:
        plan.kwargs['cpu_pin_memory'] = True
    module = ea.ElixirModule(net, sr, dtype=torch.float16)
    assert all(pc.shard_device.type == 'cpu' and pc.shard.is_pinned() for pc in module.param_chunks)
    new = {n: torch.randn_like(p, dtype=torch.float32) * 0.2 for n, p in net.named_parameters()}
    module.load_state_dict(new)
    assert all(pc.optim_sync_flag for pc in module.param_chunks)          # released after the gather
    for n, p in net.named_parameters():
        assert p.is_cuda and torch.equal(p.data.cpu(), new[n].half()), n
    sd = module.state_dict()
    for n in new:
        assert torch.equal(sd[n], new[n])
    for pc in module.param_chunks:
        assert torch.equal(pc.shard, pc.paired_chunk.shard.half())


# ------------------------------------------------------------------------------------------------
# the step over host-resident shards: the same launches, reading and writing pinned host memory
# ------------------------------------------------------------------------------------------------


def _tiny_named():
    return [('wte.weight', (500, 48)), ('h.ln.weight', (48,)), ('h.ln.bias', (48,)), ('h.fc.weight', (48, 192)),
            ('h.fc.bias', (192,)), ('h.proj.weight', (192, 48)), ('odd', (4097,)), ('lnf.weight', (48,))]


@pytest.mark.parametrize('dtype,loss_scale,max_norm', [(torch.float16, 128.0, 0.0), (torch.bfloat16, 1.0, 1.0)])
def test_step_over_pinned_host_shards_matches_oracle(oracle, dtype, loss_scale, max_norm):
    import math
    from helpers import build_workload, compare_state, refresh_oracle_grads
    kw = dict(initial_scale=loss_scale, hysteresis=1) if dtype == torch.float16 else {}
    module, opt, ochunks = build_workload(_tiny_named(), 1 << 15, dtype, seed=31, loss_scale=loss_scale,
                                          grad_std=2e-2 if max_norm else 1e-3, weight_decay=0.1, max_norm=max_norm,
                                          host_resident=True, **kw)
    assert len(module.param_chunks) >= 2
    for pc in module.param_chunks:
        assert pc.shard.is_pinned() and pc.paired_chunk.shard.is_pinned()
        assert all(t.is_pinned() for t in opt._binding.moments(pc.paired_chunk))
    scaler = (O.DynamicGradScalerOracle(initial_scale=loss_scale, min_scale=1, max_scale=2**24, hysteresis=1)
              if dtype == torch.float16 else O.ConstantGradScalerOracle(1.0))
    g = torch.Generator().manual_seed(5)
    for step in range(2):
        if step:
            for pc in module.param_chunks:
                grads = torch.randn(pc.shard_size, generator=g) * (1e-3 * loss_scale)
                grads[pc.utilized_size:] = 0
                pc.shard.copy_(grads.to(dtype))
                pc.invalidate_stats()
            refresh_oracle_grads(module, ochunks)
        opt.mark_gradients_scaled()
        opt.step()
        torch.cuda.synchronize()
        info = O.reference_step(ochunks, CODE[dtype], scaler, max_norm=max_norm, adamw_mode=True)
        assert opt.last_step_info['found_inf'] is False and info['found_inf'] is False
        if max_norm:
            assert math.isclose(opt.last_step_info['combined_scale'], info['combined_scale'], rel_tol=1e-6)
            compare_state(module, opt, ochunks, dtype, rtol=1e-6, atol_p=1e-9, atol_m=1e-11, atol_v=1e-14)
        else:
            assert opt.last_step_info['combined_scale'] == info['combined_scale']
            assert compare_state(module, opt, ochunks, dtype, exact=True) == 0
        assert all(pc.optim_sync_flag for pc in module.param_chunks)

    # an overflow: skipped, master and moments untouched, the refresh of the host shard deferred
    module.param_chunks[0].shard[3] = float('inf')
    module.param_chunks[0].invalidate_stats()
    before = [pc.paired_chunk.shard.clone() for pc in module.param_chunks]
    opt.mark_gradients_scaled()
    opt.step()
    torch.cuda.synchronize()
    assert opt.last_step_info['found_inf'] is True
    for pc, p0 in zip(module.param_chunks, before):
        assert torch.equal(pc.paired_chunk.shard, p0)
        # the refresh of a host shard is either deferred to the next gather (chunk.py:416-419) or, when
        # the step was decided on the device, already done in place by the launch that found the skip flag
        if pc.optim_sync_flag:
            assert torch.equal(pc.shard, p0.to(dtype))
        block = torch.empty(pc.chunk_size, dtype=dtype, device=DEV)
        pc.replicate(block)
        pc.scatter(block)
        assert torch.equal(pc.shard, p0.to(dtype)) and pc.optim_sync_flag is True


def test_pageable_host_shards_are_refused():
    named = [('w', (64, 64))]
    sr = ea.greedy_search([('w', 4096)], 8192, torch.float16, shard_device=torch.device('cpu'))
    module = ea.ElixirModule(dict(named), sr, dtype=torch.float16)
    inner = ea.HybridAdam(list(module.parameters()), lr=1e-3)
    opt = ea.ElixirOptimizer(module, inner, initial_scale=2.0)
    opt.mark_gradients_scaled()
    # refused BEFORE anything is launched: a kernel over pageable host memory would fault the device (the
    # stats launch of a step goes out ahead of the host's other preparations, so the check must come first)
    from elixir_amd import _abi
    launched = []
    launchers = ('grad_partials_mt', 'grad_stats_mt', 'finish_decide', 'adam_step_mt', 'adam_step_gated_mt', 'writeback_mt',
                 'put_hypers')
    originals = {name: getattr(_abi, name) for name in launchers}
    try:
        for name in launchers:
            setattr(_abi, name, lambda *a, _n=name, **k: launched.append(_n))
        for gated in (True, False):
            opt.gated_step = gated
            with pytest.raises(RuntimeError, match='pinned'):
                opt.step()
    finally:
        for name, fn in originals.items():
            setattr(_abi, name, fn)
    assert launched == []
    torch.cuda.synchronize()


def test_mixed_placement_steps_in_one_launch(oracle):
    """Every other chunk pair in pinned host memory, the others in device memory: one stats launch and
    one update launch cover both, and the result is the oracle's bit for bit."""
    from helpers import build_workload, compare_state
    dtype = torch.float16
    module, opt, ochunks = build_workload(_tiny_named(), 1 << 15, dtype, seed=33, loss_scale=64.0, weight_decay=0.1,
                                          host_resident='mixed', initial_scale=64.0, hysteresis=1)
    where = [pc.shard_device.type for pc in module.param_chunks]
    assert 'cpu' in where and 'cuda' in where
    opt.mark_gradients_scaled()
    opt.step()
    torch.cuda.synchronize()
    scaler = O.DynamicGradScalerOracle(initial_scale=64.0, min_scale=1, max_scale=2**24, hysteresis=1)
    info = O.reference_step(ochunks, CODE[dtype], scaler, max_norm=0.0, adamw_mode=True)
    assert opt.last_step_info['found_inf'] is False and opt.last_step_info['combined_scale'] == info['combined_scale']
    assert compare_state(module, opt, ochunks, dtype, exact=True) == 0
