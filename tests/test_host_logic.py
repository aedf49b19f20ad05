"""Host side of the optimizer step without a GPU: loss scaler, combined scale, hyper-parameter
records, chunk layout, chunk pairing, fake-parameter ranges, and the refusal to run without the
HIP path."""
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
import torch.nn as nn

import elixir_amd as ea
from elixir_amd import _abi
from elixir_amd import shapes as S
from elixir_amd.chunk import l2_norm_from_sumsq, stats_launch_blocks
from elixir_amd.hybrid_adam import make_hyper_record
from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------------------------------------
# scalers and host scalars
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize('hysteresis', [1, 2, 3])
@pytest.mark.parametrize('factors', [(2, 0.5), (1.7, 0.3)])
def test_dynamic_scaler_follows_the_oracle(hysteresis, factors):
    growth, backoff = factors
    rng = np.random.default_rng(hysteresis)
    kw = dict(initial_scale=2**10, growth_factor=growth, backoff_factor=backoff, growth_interval=4, min_scale=1,
              max_scale=2**14, hysteresis=hysteresis)
    a, b = ea.DynamicGradScaler(**kw), O.DynamicGradScalerOracle(**kw)
    for _ in range(400):
        found = bool(rng.random() < 0.2)
        a.update(found)
        b.update(found)
        assert a.scale_value == float(b.scale)
        assert a.scale.dtype == torch.float32 and a.scale.item() == float(b.scale)


def test_dynamic_scaler_corner_cases_as_literals():
    """The same literal trajectories the oracle is pinned with (hysteresis 0 / 1 / 3, clamps hit
    exactly and passed, counter resets, factors that are not powers of two rounded to fp32)."""
    from test_oracle import SCALER_LITERALS
    for kwargs, seq, want in SCALER_LITERALS:
        sc = ea.DynamicGradScaler(**kwargs)
        got = []
        for f in seq:
            sc.update(f)
            got.append(sc.scale_value)
        assert got == want, kwargs


def test_default_scaler_settings_skip_without_backoff_on_first_overflow():
    """With the wrapper's default hysteresis of 2 the first overflow only arms the back-off."""
    sc = ea.DynamicGradScaler(initial_scale=32768, min_scale=1, growth_factor=2, backoff_factor=0.5,
                              growth_interval=1000, hysteresis=2, max_scale=2**24)
    sc.update(True)
    assert sc.scale_value == 32768.0
    sc.update(True)
    assert sc.scale_value == 16384.0
    for _ in range(1000):
        sc.update(False)
    assert sc.scale_value == 32768.0
    sd = sc.state_dict()
    sc2 = ea.DynamicGradScaler(initial_scale=1.0)
    sc2.load_state_dict(sd)
    assert sc2.scale_value == 32768.0 and float(sc.inv_scale) == 1 / 32768.0
    const = ea.ConstantGradScaler(1.0)
    const.update(True)
    assert const.scale_value == 1.0


def test_combined_scale_matches_the_oracle():
    rng = np.random.default_rng(0)
    for _ in range(2000):
        loss_scale = float(2.0**rng.integers(0, 20))
        norm = float(10.0**rng.uniform(-6, 6)) * loss_scale
        max_norm = float(rng.choice([0.0, 0.5, 1.0, 2.0]))
        got = ea.calc_combined_scale(loss_scale, norm, max_norm, max_norm > 0)
        assert got == O.combined_scale(loss_scale, norm if max_norm > 0 else None, max_norm)
    assert ea.calc_combined_scale(1.0, None, 0.0, False) == -1


def test_l2_norm_takes_the_fp32_detour():
    for sumsq in (0.0, 1.0, 3.0, 123456.789, 1e-12, 6.5e9):
        assert l2_norm_from_sumsq(sumsq) == float(np.float32(math.sqrt(sumsq)))**2
    x = (np.random.default_rng(1).standard_normal(5000) * 30).astype(np.float32)
    assert l2_norm_from_sumsq(O.sumsq(x, O.F32)) == O.l2norm_sq_ref(x, O.F32)


def test_hyper_record_scalars():
    """float64 host scalars narrowed to fp32, as torch narrows Python scalars in tensor ops."""
    lr, b1, b2, eps, wd, step = 3e-4, 0.9, 0.95, 1e-8, 0.1, 7
    r = make_hyper_record(lr, b1, b2, eps, wd, step, True, True)[0]
    bc1, bc2 = 1 - b1**step, 1 - b2**step
    assert r['decay_mul'] == np.float32(1 - lr * wd) and r['l2_wd'] == 0 and r['flags'] == 0
    assert r['lerp_w'] == np.float32(1 - b1) and r['beta2'] == np.float32(b2) and r['omb2'] == np.float32(1 - b2)
    assert r['bc2_sqrt'] == np.float32(math.sqrt(bc2)) and r['neg_step'] == np.float32(-(lr / bc1))
    assert r['eps'] == np.float32(eps)
    r = make_hyper_record(lr, b1, b2, eps, wd, step, True, False)[0]                # L2 mode
    assert r['decay_mul'] == 1.0 and r['l2_wd'] == np.float32(wd) and r['flags'] == _abi.ELX_HYPER_L2
    r = make_hyper_record(lr, b1, b2, eps, 0.0, step, False, True)[0]               # no decay, no bias correction
    assert r['decay_mul'] == 1.0 and r['bc2_sqrt'] == 1.0 and r['neg_step'] == np.float32(-lr) and r['flags'] == 0
    r = make_hyper_record(lr, 0.4, b2, eps, 0.0, 1, True, True)[0]                  # 1-beta1 >= 0.5
    assert r['flags'] == _abi.ELX_HYPER_LERP_FROM_G
    assert r['lerp_w'] == np.float32(np.float32(1 - 0.4) - np.float32(1.0))


def test_stats_launch_blocks():
    assert stats_launch_blocks(1) == 1 and stats_launch_blocks(16384) == 1 and stats_launch_blocks(16385) == 2
    assert stats_launch_blocks(1 << 28) == 1024


# ------------------------------------------------------------------------------------------------
# chunk layout (CPU tensors)
# ------------------------------------------------------------------------------------------------


def test_chunk_append_close_and_valid_end():
    """test/chunk/test_chunk.py: tensors are packed back to back and keep their values."""
    a, b, c, d = torch.randn(2, 64), torch.randn(2, 2, 128), torch.randn(128), torch.randn(4, 32)
    copies = [t.clone() for t in (a, b, c, d)]
    chunk = ea.Chunk(None, 1024, torch.float, None, shard_device='cpu', temp_device='cpu')
    assert chunk.chunk_size == 1024 and chunk.chunk_dtype == torch.float and chunk.shard_size == 1024
    for t in (a, b, c, d):
        chunk.append_tensor(t)
    for t, cp in zip((a, b, c, d), copies):
        assert torch.equal(t, cp)                      # still readable while the chunk is open
    assert [(i.offset, i.end) for i in chunk.tensors_info.values()] == O.chunk_offsets([128, 512, 128, 128])
    with pytest.raises(ea.ChunkFullError):
        chunk.append_tensor(torch.randn(200))
    chunk.close_chunk()
    assert chunk.is_replica is False and chunk.is_init is False
    assert chunk.utilized_size == 896 and chunk.valid_end == 896 == O.valid_end(896, 0, 1024) and chunk.n_valid == 896
    flat = torch.cat([cp.flatten() for cp in copies])
    assert torch.equal(chunk.shard[:896], flat) and torch.count_nonzero(chunk.shard[896:]) == 0
    assert chunk.tensor_state_cnter[ea.TensorState.HOLD] == 4

    full = ea.Chunk(None, 256, torch.float16, None, shard_device='cpu', temp_device='cpu')
    full.append_tensor(torch.randn(256).half())
    full.close_chunk()
    assert full.valid_end == 257 and full.n_valid == 256              # sentinel of a completely used shard
    with pytest.raises(AssertionError):
        full.append_tensor(torch.randn(1).half())                     # closed
    other = ea.Chunk(None, 256, torch.float, None, shard_device='cpu', temp_device='cpu')
    with pytest.raises(AssertionError):
        other.append_tensor(torch.randn(4).half())                    # dtype mismatch


def test_chunk_pairing_and_meta_tensors():
    p = ea.Chunk(None, 100, torch.float16, None, shard_device='cpu')
    o = ea.Chunk(None, 100, torch.float, None, shard_device='cpu')
    t16 = nn.Parameter(torch.empty(3, 7, dtype=torch.float16, device='meta'))
    t32 = torch.empty(3, 7, dtype=torch.float, device='meta')
    p.append_tensor(t16)
    o.append_tensor(t32)
    p.close_chunk()
    o.close_chunk()
    p.init_pair(o)
    assert p.paired_chunk is o and o.paired_chunk is p
    p.init_pair(o)                                                    # idempotent
    assert p.tensors_info[t16].end == 21 and torch.count_nonzero(p.shard) == 0
    third = ea.Chunk(None, 100, torch.float, None, shard_device='cpu')
    with pytest.raises(AssertionError):
        p.init_pair(third)
    with pytest.raises(RuntimeError):                                 # flags come from the HIP kernels only
        p.update_extra_reduce_info()
    # a host-resident shard defers the refresh exactly like the reference (chunk.py:416-419)
    p.optim_update()
    assert p.optim_sync_flag is False


class TinyNet(nn.Module):

    def __init__(self):
        super().__init__()
        self.embed = nn.Embedding(20, 16)
        self.norm = nn.LayerNorm(16)
        self.fc = nn.Linear(16, 40)
        self.out = nn.Linear(40, 20, bias=False)

    def forward(self, x):
        return self.out(torch.relu(self.fc(self.norm(self.embed(x))))).sum()


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_module_builds_paired_chunks(dtype):
    torch.manual_seed(0)
    net = TinyNet()
    originals = {n: p.detach().clone() for n, p in net.named_parameters()}
    named = [(n, p.numel()) for n, p in net.named_parameters()]
    sr = ea.greedy_search(named, 1024, dtype, shard_device=torch.device('cpu'))
    assert [len(pl.name_list) for pl in sr.param_chunk_plans] == [len(g) for g in O.greedy_pack([s for _, s in named], 1024)]
    module = ea.ElixirModule(net, sr, dtype=dtype)
    assert module.use_amp == (dtype == torch.float16)
    for pc in module.param_chunks:
        oc = pc.paired_chunk
        assert oc.chunk_dtype == torch.float32 and pc.chunk_dtype == dtype and oc.paired_chunk is pc
        assert pc.chunk_size == oc.chunk_size == 1024 and pc.valid_end == oc.valid_end
        # identical offsets in both chunks (module.py:120-127)
        assert [(i.offset, i.end) for i in pc.tensors_info.values()] == [(i.offset, i.end) for i in oc.tensors_info.values()]
        assert torch.equal(pc.shard, oc.shard.to(dtype))
    for name, param in net.named_parameters():
        pc = module.fetcher.get_one_chunk(param)
        info = pc.tensors_info[param]
        assert torch.equal(pc.paired_chunk.shard[info.offset:info.end], originals[name].flatten())    # fp32 master
        assert param.dtype == dtype and torch.equal(param.data.flatten(), originals[name].flatten().to(dtype))
    sd = module.state_dict()
    for name, t in originals.items():
        assert torch.equal(sd[name], t) and sd[name].dtype == torch.float32
    assert module.state_dict(from_param=True)['fc.weight'].dtype == dtype


def test_module_accepts_the_forward_pass_settings_of_the_reference_callers():
    """example/common/elx.py:37 builds ElixirModule(model, sr, group, prefetch=True, dtype=torch.float16,
    use_fused_kernels=True): both are speed settings of the forward pass, accepted and without effect here."""
    net = TinyNet()
    named = [(n, p.numel()) for n, p in net.named_parameters()]
    sr = ea.greedy_search(named, 1024, torch.float16, shard_device=torch.device('cpu'))
    module = ea.ElixirModule(net, sr, None, prefetch=True, dtype=torch.float16, use_fused_kernels=True)
    assert module.use_amp and module.prefetch_flag and module.use_fused_kernels
    opt = ea.ElixirOptimizer(module, ea.HybridAdam(net.parameters(), lr=1e-3), initial_scale=64, hysteresis=1)
    assert opt.loss_scale == 64.0


def test_optimizer_ranges_groups_and_refusal_to_run_on_cpu():
    torch.manual_seed(0)
    net = TinyNet()
    named = [(n, p.numel()) for n, p in net.named_parameters()]
    module = ea.ElixirModule(net, ea.greedy_search(named, 1024, torch.float16, shard_device=torch.device('cpu')),
                             dtype=torch.float16)
    decay = [p for n, p in net.named_parameters() if p.dim() > 1]
    exempt = [p for n, p in net.named_parameters() if p.dim() == 1]
    inner = ea.HybridAdam([dict(params=decay, weight_decay=0.1), dict(params=exempt, weight_decay=0.0, lr=5e-4)], lr=1e-3)
    opt = ea.ElixirOptimizer(module, inner, initial_scale=64, hysteresis=1, max_norm=1.0)
    assert isinstance(opt.grad_scaler, ea.DynamicGradScaler) and opt.loss_scale == 64.0
    assert all(c.l2_norm_flag for c in opt.param_chunk_set)
    # every real parameter became one zero-size fake parameter with its (begin, end) in the shard
    assert [len(g['params']) for g in opt.param_groups] == [len(decay), len(exempt)]
    assert [g['weight_decay'] for g in opt.param_groups] == [0.1, 0.0] and opt.param_groups[1]['lr'] == 5e-4
    for group, real in zip(opt.param_groups, (decay, exempt)):
        for fake, p in zip(group['params'], real):
            assert fake.numel() == 0
            pc = module.fetcher.get_one_chunk(p)
            info = pc.tensors_info[p]
            assert opt.param_to_range[fake] == O.range_pair(info.offset, info.end, 0, pc.shard_size)
            assert opt.param_to_optim_chunk[fake] is pc.paired_chunk
    # fp32 / bf16 modules get the constant scaler
    m32 = ea.ElixirModule(TinyNet(), ea.greedy_search(named, 1024, torch.float32, shard_device=torch.device('cpu')))
    o32 = ea.ElixirOptimizer(m32, ea.HybridAdam(m32.parameters()))
    assert isinstance(o32.grad_scaler, ea.ConstantGradScaler) and o32.loss_scale == 1.0
    with pytest.raises(AssertionError):
        ea.ElixirOptimizer(m32, ea.HybridAdam(m32.parameters()), max_norm=1.0, norm_type=1.0)
    # no GPU, no step: the product has no CPU path
    opt.mark_gradients_scaled()
    with pytest.raises(RuntimeError, match='HIP|GPU'):
        opt.step()
    p = nn.Parameter(torch.zeros(4))
    p.grad = torch.ones(4)
    with pytest.raises(RuntimeError, match='GPU'):
        ea.HybridAdam([p]).step()
    with pytest.raises(NotImplementedError):
        ea.HybridAdam([p], nvme_offload_fraction=0.5)


def test_land_gradients_moves_grads_into_the_shards_on_cpu():
    torch.manual_seed(0)
    net = TinyNet()
    named = [(n, p.numel()) for n, p in net.named_parameters()]
    module = ea.ElixirModule(net, ea.greedy_search(named, 1024, torch.float32, shard_device=torch.device('cpu')))
    loss = module(torch.randint(0, 20, (4, 8)))
    loss.backward()
    grads = {n: p.grad.detach().clone() for n, p in net.named_parameters()}
    module.land_gradients(sync=False)
    for name, param in net.named_parameters():
        pc = module.fetcher.get_one_chunk(param)
        info = pc.tensors_info[param]
        assert torch.equal(pc.shard[info.offset:info.end], grads[name].flatten())
        assert torch.count_nonzero(pc.shard[pc.utilized_size:]) == 0


def test_workload_shapes():
    for fn, tensors, total in ((S.gpt2_shapes, 148, 124_439_808), (S.opt_shapes, 388, 1_315_758_080),
                               (S.llama_shapes, 291, 6_738_415_616)):
        sh = fn()
        assert len(sh) == tensors and sum(S.numel(s) for _, s in sh) == total
        assert len({n for n, _ in sh}) == tensors


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--gpus', '2'], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True)
    assert proc.returncode != 0 and 'ONE GPU' in proc.stderr


# ------------------------------------------------------------------------------------------------
# launch plan
# ------------------------------------------------------------------------------------------------


def test_launch_plan_blocks_segments_and_padding():
    from elixir_amd.launch_plan import FlatBuffer, build_plan
    tile = _abi.tile_elems()
    base = 0x40000000
    # a 64 Ki-element buffer with 40,000 valid elements in three tensors; the rest is padding
    buf = FlatBuffer(grad=base, lowp_out=base, master=base + (1 << 24), m=base + (2 << 24), v=base + (3 << 24),
                     n_alloc=65536, n_valid=40000, segs=[(0, 5000, 0), (5000, 5003, 1), (5003, 40000, 0)])
    plan = build_plan([buf], 2, 2, 2, _abi.ELX_F16, _abi.ELX_F16, fold_padding_below=0)
    B = plan.block_elems
    assert B % tile == 0 and B >= 16 * tile
    n_rows = -(-40000 // B)
    assert len(plan.rows) == n_rows and plan.info.max_tiles == B // tile
    covered = 0
    for i, row in enumerate(plan.rows):
        b = i * B
        assert row['master'] == buf.master + 4 * b and row['grad'] == buf.grad + 2 * b == row['lowp_out']
        assert row['m'] == buf.m + 4 * b and row['v'] == buf.v + 4 * b
        assert row['n_alloc'] == min(B, 65536 - b) and row['n_valid'] == max(0, min(row['n_alloc'], 40000 - b))
        segs = plan.segs[row['seg_begin']:row['seg_end']]
        # the row's segments are the buffer's segments clipped to the block and re-based
        want = [(max(sb, b) - b, min(se, b + B) - b, h) for sb, se, h in buf.segs if se > b and sb < b + B]
        assert [(int(s['begin']), int(s['end']), int(s['hyper'])) for s in segs] == want
        covered += sum(int(s['end'] - s['begin']) for s in segs)
    assert covered == 40000
    # padding beyond the last update block goes to the refresh launch
    up_end = min(65536, n_rows * B)
    if up_end < 65536:
        assert len(plan.refresh_rows) == 1 and plan.refresh_rows[0]['n_alloc'] == 65536 - up_end
        assert plan.refresh_rows[0]['lowp_out'] == base + 2 * up_end and plan.refresh_rows[0]['master'] == buf.master + 4 * up_end
    else:
        assert plan.refresh_rows is None
    # no low-precision copy, no refresh rows; zero valid elements, no update rows
    solo = FlatBuffer(grad=base, lowp_out=0, master=base + (1 << 24), m=base + (2 << 24), v=base + (3 << 24),
                      n_alloc=65536, n_valid=40000, segs=[(0, 40000, 0)])
    assert build_plan([solo], 4, 4, 1, _abi.ELX_F32, _abi.ELX_NONE).refresh_rows is None
    empty = FlatBuffer(grad=base, lowp_out=base, master=base + (1 << 24), m=base + (2 << 24), v=base + (3 << 24),
                       n_alloc=65536, n_valid=0, segs=[])
    plan = build_plan([empty], 2, 2, 1, _abi.ELX_F16, _abi.ELX_F16, fold_padding_below=0)
    assert len(plan.rows) == 0 and plan.refresh_rows[0]['n_alloc'] == 65536
    # a little padding rides the update launch instead: every block of the buffer is a row (those behind the
    # valid head with no valid element and no segment), and there is no refresh launch
    for b in (buf, empty):
        folded = build_plan([b], 2, 2, 2, _abi.ELX_F16, _abi.ELX_F16)
        assert folded.refresh_rows is None and len(folded.rows) == -(-65536 // folded.block_elems)
        assert int(folded.rows['n_alloc'].sum()) == 65536 and int(folded.rows['n_valid'].sum()) == b.n_valid
        tail = folded.rows[folded.rows['n_valid'] == 0]
        assert all(r['seg_begin'] == r['seg_end'] for r in tail)
    # ... but not when there is a lot of it
    big = FlatBuffer(grad=base, lowp_out=base, master=base + (1 << 32), m=base + (2 << 32), v=base + (3 << 32),
                     n_alloc=1 << 26, n_valid=1 << 20, segs=[(0, 1 << 20, 0)])
    plan = build_plan([big], 2, 2, 1, _abi.ELX_F16, _abi.ELX_F16)
    assert plan.refresh_rows is not None and int(plan.rows['n_alloc'].sum()) + int(plan.refresh_rows['n_alloc'].sum()) == 1 << 26


def test_launch_plan_chooses_the_cache_policy_of_the_update_launch_by_size():
    """Low-precision shards of up to 2 GiB in all, in device memory: the update launch is told to write them
    with the stores the memory-side cache takes in (ELX_FLAG_KEEP_CACHED).  Everything the launch touches at
    most 256 MiB: ELX_FLAG_KEEP_STATE_CACHED on top.  Larger sets, host-resident ones and large launches
    without a low-precision copy stream."""
    from elixir_amd.launch_plan import KEEP_LOWP_CACHED_BELOW, KEEP_STATE_CACHED_BELOW, FlatBuffer, build_plan
    base = 0x40000000
    assert KEEP_LOWP_CACHED_BELOW == 2 << 30 and KEEP_STATE_CACHED_BELOW == 256 << 20
    lowp_flag, state_flags = _abi.ELX_FLAG_KEEP_CACHED, _abi.ELX_FLAG_KEEP_CACHED | _abi.ELX_FLAG_KEEP_STATE_CACHED

    def plan_of(n_buffers, n_alloc, lowp=True, **kw):
        bufs = [FlatBuffer(grad=base + (i << 34), lowp_out=(base + (i << 34)) if lowp else 0, master=base + (i << 34) + (1 << 32),
                           m=base + (i << 34) + (2 << 32), v=base + (i << 34) + (3 << 32), n_alloc=n_alloc, n_valid=n_alloc,
                           segs=[(0, n_alloc, 0)]) for i in range(n_buffers)]
        esize = 2 if lowp else 4
        return build_plan(bufs, esize, esize, 1, _abi.ELX_F16 if lowp else _abi.ELX_F32,
                          _abi.ELX_F16 if lowp else _abi.ELX_NONE, **kw)

    small = plan_of(2, 64 << 20)                     # 256 MiB of fp16 shards, 1.75 GiB of state
    assert small.info.cache_policy == 1 and small.info.flags == lowp_flag
    assert plan_of(8, 128 << 20).info.cache_policy == 1              # exactly 2 GiB of shards
    large = plan_of(9, 128 << 20)                                    # 2.25 GiB
    assert large.info.cache_policy == 0 and large.info.flags == 0
    assert plan_of(2, 64 << 20, device_resident=False).info.cache_policy == 0
    # the whole state: 14 B per element with the gradients in the low-precision shard, 16 B for a flat fp32
    # parameter with fp32 gradients
    tiny = plan_of(1, (256 << 20) // 14 // 1024 * 1024)
    assert tiny.info.cache_policy == 2 and tiny.info.flags == state_flags
    assert plan_of(1, (256 << 20) // 14 // 1024 * 1024 + 1024).info.cache_policy == 1
    flat = plan_of(1, 1 << 24, lowp=False)           # configuration 1: 4 x 64 MiB
    assert flat.info.cache_policy == 2 and flat.info.flags == state_flags and flat.info.keep_state_cached
    assert plan_of(1, (1 << 24) + 1024, lowp=False).info.cache_policy == 0
    assert plan_of(1, 1 << 24, lowp=False, device_resident=False).info.cache_policy == 0
    # what elx_check_tables reports carries no choice
    info = _abi.check_tables(small.rows, small.segs, 1, _abi.ELX_F16, _abi.ELX_F16)
    assert info.cache_policy == 0 and not info.keep_lowp_cached and info.with_keep_lowp_cached(True).flags == lowp_flag
    assert info.with_cache_policy(2).flags == state_flags and info.with_cache_policy(2)[:3] == tuple(info)


def test_greedy_packing_carries_tensors_without_elements():
    """mini_waste.py:78-96 with sizes of zero in the list: such a tensor never opens a chunk of its own
    behind the first and never overflows one; at the head of the list it opens the first chunk."""
    from elixir_amd.module import greedy_groups
    assert greedy_groups([0, 5, 0, 60, 10, 0], 64) == [[0, 1, 2], [3], [4, 5]]
    assert greedy_groups([64, 0, 0, 1], 64) == [[0, 1, 2], [3]]
    assert greedy_groups([0], 64) == [[0]] and greedy_groups([], 64) == []
    with pytest.raises(AssertionError, match='does not fit'):
        greedy_groups([65], 64)


def test_launch_plan_keeps_rows_bounded_for_the_large_workloads():
    from elixir_amd.launch_plan import FlatBuffer, build_plan
    from elixir_amd.module import greedy_groups
    sizes = [S.numel(s) for _, s in S.llama_shapes()]
    bufs = []
    for k, grp in enumerate(greedy_groups(sizes, 256 << 20)):
        off, segs = 0, []
        for i in grp:
            segs.append((off, off + sizes[i], 0))
            off += sizes[i]
        base = (k + 1) << 34
        bufs.append(FlatBuffer(base, base, base + (1 << 32), base + (2 << 32), base + (3 << 32), 256 << 20, off, segs))
    plan = build_plan(bufs, 2, 2, 1, _abi.ELX_F16, _abi.ELX_F16)
    assert len(plan.rows) < 65536 and plan.info.max_tiles == plan.block_elems // _abi.tile_elems()
    assert int(plan.rows['n_valid'].sum()) == sum(sizes)
    padding = 27 * (256 << 20) - int(plan.rows['n_alloc'].sum())
    assert padding == int(plan.refresh_rows['n_alloc'].sum()) and padding > 0
    # few workgroups of the 2-D grid find no work
    assert plan.info.max_tiles * len(plan.rows) - plan.info.total_tiles < 0.01 * plan.info.total_tiles


def test_land_rows_tile_every_piece_exactly():
    from elixir_amd.chunk import land_rows, _land_block_elems
    block = 4096
    pieces = [(0, 1 << 30, 1 << 40, 10000), (0, 0, (1 << 40) + 20000, 5000), (1, 1 << 31, 1 << 41, 4096),
              (2, 1 << 32, 1 << 42, 1), (2, 0, (1 << 42) + 2, 8193)]
    rows, offsets = land_rows(pieces, 3, block, ssize=4, dsize=2)
    assert offsets.tolist() == [0, 3 + 2, 3 + 2 + 1, 3 + 2 + 1 + 1 + 3]
    k = 0
    for slot, src, dst, count in pieces:
        left = count
        done = 0
        while left > 0:
            r = rows[k]
            n = min(block, left)
            assert r['n_alloc'] == n and r['n_valid'] == (n if src else 0)
            assert r['grad'] == (src + 4 * done if src else 0) and r['lowp_out'] == dst + 2 * done
            assert offsets[slot] <= k < offsets[slot + 1]
            done += n
            left -= n
            k += 1
    assert k == len(rows)


def test_land_block_is_sized_to_the_tensors():
    """The grid of a per-tensor landing is (tiles of the longest row, rows): the block is chosen so that
    few workgroups find no work.  Long tensors keep the 2048-tile block; a set whose tensors leave part of such a block without work gets
    a shorter one; a set too large for 32 Ki rows a longer one.  Checked on the tensor lists of the three
    model families, chunk by chunk (one launch per chunk, as backward issues them) and all at once."""
    from elixir_amd import shapes as S
    from elixir_amd.chunk import LAND_IDLE_ALLOWED, LAND_MAX_ROWS, _land_block_elems
    from elixir_amd.module import greedy_groups
    tile = 2048

    def idle_share(counts, block):
        counts = np.asarray(counts, dtype=np.int64)
        rows = int((-(-counts // block)).sum())
        work = int((-(-counts // tile)).sum())
        width = min(block // tile, int((-(-counts // tile)).max()))
        return rows, (rows * width - work) / work

    assert _land_block_elems([1000], tile) == 2048 * tile                  # one short row: nothing idles
    assert _land_block_elems([7_247_757_312], tile) == 2048 * tile         # one long tensor
    b = _land_block_elems([1 << 40], tile)
    assert b & (b - 1) == 0 and (1 << 40) // b <= LAND_MAX_ROWS < (1 << 40) // (b // 2)
    for shapes, csize, expect_small in ((S.gpt2_shapes(), 64 << 20, True), (S.opt_shapes(), 128 << 20, True),
                                        (S.llama_shapes(), 256 << 20, True)):
        sizes = [S.numel(shape) for _, shape in shapes]
        groups = greedy_groups(sizes, csize)
        per_chunk = [[sizes[i] for i in g] + [csize - sum(sizes[i] for i in g)] for g in groups]    # tensors + padding
        for counts in per_chunk + [[c for cs in per_chunk for c in cs]]:
            counts = [c for c in counts if c > 0]
            block = _land_block_elems(counts, tile)
            assert block % tile == 0 and (block // tile) & (block // tile - 1) == 0 and 8 * tile <= block <= 2048 * tile
            rows, idle = idle_share(counts, block)
            assert rows <= LAND_MAX_ROWS and idle <= LAND_IDLE_ALLOWED + 1e-9, (len(counts), block // tile, rows, idle)
            _, idle_at_2048 = idle_share(counts, 2048 * tile)
            if idle_at_2048 <= LAND_IDLE_ALLOWED:
                assert block == 2048 * tile
        whole = [c for cs in per_chunk for c in cs if c > 0]
        assert (_land_block_elems(whole, tile) < 2048 * tile) == expect_small


def test_pinned_arena_slots_survive_any_landing_order():
    """An optimizer pins its chunks' record slots in chunk order; landings in any order and grouping then
    keep them, a landing over chunks whose slots do not follow each other is cut into runs, and chunks
    nobody pinned still get consecutive slots per landing.  (CPU arena: nothing is launched.)"""
    from elixir_amd.chunk import StatsArena

    def chunk():
        c = ea.Chunk(None, 64, torch.float16, None, shard_device='cpu', temp_device='cpu')
        c.append_tensor(torch.zeros(8).half())
        c.close_chunk()
        return c

    arena = StatsArena(torch.device('cpu'))
    loose = chunk()
    arena.assign([loose])
    cs = [chunk() for _ in range(5)]
    arena.pin(cs)
    first = cs[0]._stats_slot
    assert [c._stats_slot for c in cs] == [first + i for i in range(5)] and all(c._stats_pinned for c in cs)
    arena.pin(cs)                                                    # again: nothing moves
    assert [c._stats_slot for c in cs] == [first + i for i in range(5)]
    for c in reversed(cs):                                           # last chunk first, one landing each
        assert arena.runs([c]) == [[c]]
    assert [c._stats_slot for c in cs] == [first + i for i in range(5)]
    assert arena.runs(cs) == [cs]                                    # all at once: one run
    assert arena.runs([cs[0], cs[2], cs[3]]) == [[cs[0]], [cs[2], cs[3]]]    # a gap cuts the landing in two
    extra = [chunk(), chunk()]
    runs = arena.runs([cs[4]] + extra + [loose])                     # pinned, then chunks without a pinned slot
    assert runs == [[cs[4]], extra + [loose]]
    assert extra[1]._stats_slot == extra[0]._stats_slot + 1 and loose._stats_slot == extra[1]._stats_slot + 1
    assert [c._stats_slot for c in cs] == [first + i for i in range(5)]
    arena.assign(cs[1:3])                                            # already side by side: kept, still pinned
    assert cs[1]._stats_pinned and [c._stats_slot for c in cs] == [first + i for i in range(5)]
    arena.assign([cs[3], cs[1]])                                     # an explicit assign out of order moves and unpins
    assert not cs[1]._stats_pinned and not cs[3]._stats_pinned and cs[1]._stats_slot == cs[3]._stats_slot + 1
    arena.pin(cs)                                                    # the optimizer is built again: a fresh run
    assert all(c._stats_pinned for c in cs) and [c._stats_slot - cs[0]._stats_slot for c in cs] == list(range(5))


# ------------------------------------------------------------------------------------------------
# checkpoint of the optimizer state (no GPU: host-resident shards can be saved and loaded, not stepped)
# ------------------------------------------------------------------------------------------------


def _cpu_optimizer(seed):
    torch.manual_seed(seed)
    net = TinyNet()
    named = [(n, p.numel()) for n, p in net.named_parameters()]
    module = ea.ElixirModule(net, ea.greedy_search(named, 1024, torch.float16, shard_device=torch.device('cpu')),
                             dtype=torch.float16)
    decay = [p for p in net.parameters() if p.dim() > 1]
    exempt = [p for p in net.parameters() if p.dim() == 1]
    inner = ea.HybridAdam([dict(params=decay, weight_decay=0.1), dict(params=exempt, weight_decay=0.0)], lr=1e-3)
    return module, ea.ElixirOptimizer(module, inner, initial_scale=1024.0, hysteresis=2, growth_interval=7)


def test_optimizer_state_dict_round_trip_keeps_flat_storage():
    module, opt = _cpu_optimizer(0)
    sd0 = opt.state_dict()
    n_params = sum(len(g['params']) for g in opt.param_groups)
    assert set(sd0) == {'state', 'param_groups', 'grad_scaler'} and len(sd0['state']) == n_params
    assert all(st['step'] == 0 and st['exp_avg'].device.type == 'cpu' for st in sd0['state'].values())

    # invent a state: moments, step counts, changed hyper-parameters, a scaler in mid-flight
    gen = torch.Generator().manual_seed(1)
    for i, st in sd0['state'].items():
        st['exp_avg'] = torch.randn(st['exp_avg'].shape, generator=gen)
        st['exp_avg_sq'] = torch.rand(st['exp_avg_sq'].shape, generator=gen)
        st['step'] = 5 + i
    sd0['param_groups'][0]['lr'] = 3e-4
    sd0['param_groups'][1]['betas'] = (0.8, 0.95)
    sd0['grad_scaler'].update(scale=torch.tensor([256.0]), growth_step=3, hysteresis_step=1)

    flat_before = {c: (opt._binding.moments(c)[0].data_ptr(), opt._binding.moments(c)[1].data_ptr())
                   for c in opt._binding.chunks}
    opt.load_state_dict(sd0)
    assert opt.loss_scale == 256.0 and opt.grad_scaler._growth_step == 3 and opt.grad_scaler._hysteresis_step == 1
    assert opt.param_groups[0]['lr'] == 3e-4 and opt.param_groups[1]['betas'] == (0.8, 0.95)
    sd1 = opt.state_dict()
    for i, st in sd0['state'].items():
        assert sd1['state'][i]['step'] == st['step']
        assert torch.equal(sd1['state'][i]['exp_avg'], st['exp_avg'])
        assert torch.equal(sd1['state'][i]['exp_avg_sq'], st['exp_avg_sq'])
    # the values went INTO the flat per-chunk buffers: same storage, and the per-tensor views see them
    for c, (pm, pv) in flat_before.items():
        m, v = opt._binding.moments(c)
        assert (m.data_ptr(), v.data_ptr()) == (pm, pv)
    k = 0
    for group in opt.param_groups:
        for fake in group['params']:
            chunk, (b, e) = opt.param_to_optim_chunk[fake], opt.param_to_range[fake]
            assert torch.equal(opt._binding.moments(chunk)[0][b:e], sd0['state'][k]['exp_avg'])
            k += 1

    other_module, other = _cpu_optimizer(0)
    bad = opt.state_dict()
    bad['param_groups'][0]['params'] = bad['param_groups'][0]['params'][:-1]
    with pytest.raises(ValueError):
        other.load_state_dict(bad)


def test_wrapper_is_a_torch_optimizer_and_schedulers_reach_the_hyper_table():
    """The reference's wrapper is an Optimizer (optimizer.py:27) and its own callers hand it to a
    learning-rate scheduler (example/fine-tune/elixir_mini.py:90).  torch's schedulers accept this one,
    and the learning rate they set is the one the next step's hyper records are made from."""
    module, opt = _cpu_optimizer(3)
    assert isinstance(opt, torch.optim.Optimizer)
    assert opt.param_groups is opt.optim.param_groups and opt.state is opt.optim.state
    assert opt.defaults is opt.optim.defaults and 'HybridAdam' in repr(opt)
    sched = torch.optim.lr_scheduler.LambdaLR(opt, lr_lambda=lambda epoch: 0.5**epoch)
    assert [g['initial_lr'] for g in opt.param_groups] == [1e-3, 1e-3]

    def neg_steps():
        return sorted(set(float(x) for x in opt.optim.hyper_table_of_next_step()['neg_step']))

    bc1 = 1.0 - 0.9**1    # the first step of every tensor
    assert neg_steps() == [float(np.float32(-(1e-3 / bc1)))]
    opt._opt_called = True    # what the scheduler's wrapper around step() records; no GPU, no step here
    sched.step()
    assert [g['lr'] for g in opt.param_groups] == [5e-4, 5e-4]
    assert neg_steps() == [float(np.float32(-(5e-4 / bc1)))]
    # a warm-up schedule on one group only: two different records
    opt.param_groups[1]['lr'] = 1e-4
    assert neg_steps() == sorted([float(np.float32(-(5e-4 / bc1))), float(np.float32(-(1e-4 / bc1)))])
    # decoupled decay follows the learning rate as well (torch/optim/adam.py:414-419)
    table = opt.optim.hyper_table_of_next_step()
    assert sorted(float(x) for x in table['decay_mul']) == sorted([float(np.float32(1 - 5e-4 * 0.1)), 1.0])
    # other schedulers construct too
    torch.optim.lr_scheduler.StepLR(opt, step_size=2)
    torch.optim.lr_scheduler.CosineAnnealingLR(opt, T_max=10)


def test_hybrid_adam_dispatches_step_hooks_itself():
    """HybridAdam.step is not wrapped by torch (the wrapper's profiler scope costs the device tens of
    microseconds per step); hooks registered on the optimizer are still run, in torch's order."""
    p = nn.Parameter(torch.zeros(4))
    p.grad = torch.ones(4)
    opt = ea.HybridAdam([p])
    assert getattr(type(opt).step, 'hooked', False) and not hasattr(type(opt).step, '__wrapped__')
    seen = []
    opt.register_step_pre_hook(lambda o, args, kwargs: seen.append(('pre', args, dict(kwargs))))
    opt.register_step_post_hook(lambda o, args, kwargs: seen.append(('post', args, dict(kwargs))))
    with pytest.raises(RuntimeError, match='GPU'):    # no device here: the launch is refused, after the pre-hook ran
        opt.step(div_scale=4.0)
    assert seen == [('pre', (None, 4.0), dict(gated=False, defer_commit=False))]


def test_wrapper_runs_its_step_hooks_and_refuses_to_be_copied(monkeypatch):
    """Hooks registered on the wrapper -- which is an Optimizer that never ran Optimizer.__init__ -- fire
    around its step, a pre-hook may replace the arguments; torch's process-wide hooks are left to the inner
    optimizer's own step (where the reference's wrapper has them fire too).  State-dict hooks go to the
    inner optimizer, whose state it is.  Copying or pickling the wrapper is refused with the reason."""
    import copy
    import pickle
    from torch.optim.optimizer import register_optimizer_step_post_hook, register_optimizer_step_pre_hook
    module, opt = _cpu_optimizer(5)
    seen = []
    monkeypatch.setattr(opt, '_step', lambda *a, **k: seen.append(('step', a, k)) or 'ret')
    handles = [register_optimizer_step_pre_hook(lambda o, a, k: seen.append(('global pre', type(o).__name__))),
               register_optimizer_step_post_hook(lambda o, a, k: seen.append(('global post', type(o).__name__))),
               opt.register_step_pre_hook(lambda o, a, k: (seen.append('own pre'), ((), dict(marker=1)))[1]),
               opt.register_step_post_hook(lambda o, a, k: seen.append(('own post', k)))]
    try:
        assert opt.step() == 'ret'
        assert seen == ['own pre', ('step', (), dict(marker=1)), ('own post', dict(marker=1))]
        # the process-wide ones fire in the inner optimizer's step, with the inner optimizer
        seen.clear()
        monkeypatch.setattr(opt.optim, 'launch_step', lambda *a, **k: seen.append('inner launch'))
        opt.optim.step(gated=True, defer_commit=True)
        assert seen == [('global pre', 'HybridAdam'), 'inner launch', ('global post', 'HybridAdam')]
    finally:
        for h in handles:
            h.remove()
    seen.clear()
    opt.step()                                   # no hook left: straight through
    assert seen == [('step', (), {})]
    # a torch that names its process-wide hook tables differently: no such hooks, no AttributeError
    import torch.optim.optimizer as TO
    from elixir_amd.hybrid_adam import _global_step_hooks
    monkeypatch.delattr(TO, '_global_optimizer_pre_hooks')
    monkeypatch.delattr(TO, '_global_optimizer_post_hooks')
    assert _global_step_hooks() == ({}, {})
    monkeypatch.undo()
    called = []
    opt.register_state_dict_post_hook(lambda o, sd: called.append(type(o).__name__))
    opt.state_dict()
    assert called == ['HybridAdam']
    for attempt in (lambda: copy.deepcopy(opt), lambda: pickle.dumps(opt)):
        with pytest.raises(TypeError, match='cannot be copied or pickled'):
            attempt()


def test_the_chunk_members_the_optimizer_touches_are_the_documented_ones():
    """A chunk object has to offer the members the reference's wrapper reads of its own Chunk plus a dozen
    that this build adds (where the flags wait between landing and step).  Stand-ins that carry exactly
    those -- anything else raises AttributeError -- go through the wrapper's host logic: construction
    with the ranges of optimizer.py:238-265, the flags, the global norm, the combined scale, the
    decision where the flags come from, the state dict."""
    from elixir_amd.optimizer import CHUNK_MEMBERS_ADDED, CHUNK_MEMBERS_OF_THE_REFERENCE
    allowed = set(CHUNK_MEMBERS_OF_THE_REFERENCE) | set(CHUNK_MEMBERS_ADDED)

    class StandIn:
        """Exactly the documented members, taken from a real chunk; sorted and hashed like one."""

        def __init__(self, real):
            object.__setattr__(self, '_real', real)

        def __getattr__(self, name):
            if name not in allowed:
                raise AttributeError(f'{name} is not among the documented chunk members')
            value = getattr(object.__getattribute__(self, '_real'), name)
            return value

        def __setattr__(self, name, value):
            if name not in allowed:
                raise AttributeError(f'{name} is not among the documented chunk members')
            setattr(object.__getattribute__(self, '_real'), name, value)

        def __hash__(self):
            return self.chunk_id

        def __eq__(self, other):
            return isinstance(other, StandIn) and other.chunk_id == self.chunk_id

        def __lt__(self, other):
            return self.chunk_id < other.chunk_id

    module, _ = _cpu_optimizer(9)
    real_chunks = module.param_chunks
    stand = {c: StandIn(c) for c in real_chunks}
    stand_optim = {c.paired_chunk: StandIn(c.paired_chunk) for c in real_chunks}

    class Shim:    # what the wrapper reads of the module (optimizer.py:58-66,77,253)
        use_amp = module.use_amp
        optim_chunk_group = module.optim_chunk_group

        class param_chunk_group:
            fused_chunks = set()
            float_chunks = set(stand.values())

        class fetcher:
            @staticmethod
            def get_one_chunk(param):
                return stand[module.fetcher.get_one_chunk(param)]

    for c, s in stand.items():    # the pairing, between stand-ins
        c.paired_chunk = stand_optim[c.paired_chunk]
        c.paired_chunk._real.paired_chunk = s
    params = [p for p in module.parameters()]
    opt = ea.ElixirOptimizer(Shim, ea.HybridAdam(params, lr=1e-3), initial_scale=8.0, max_norm=2.0)
    assert len(opt.param_to_range) == len(params) and all(b < e for b, e in opt.param_to_range.values())
    chunks = opt._param_chunk_list
    assert chunks == sorted(stand.values()) and all(c.l2_norm_flag for c in chunks)
    assert opt._stats_source() == ('launch', None)
    for i, c in enumerate(chunks):
        c._apply_stats(False, 4.0 * (i + 1))
    assert opt._check_overflow() is False
    assert opt._calc_global_norm() == pytest.approx(math.sqrt(sum(4.0 * (i + 1) for i in range(len(chunks)))), rel=1e-6)
    opt.optim_state = ea.OptimState.SCALED
    assert opt._get_combined_scale() > 0
    chunks[-1]._apply_stats(True, 1.0)
    assert opt._check_overflow() is True
    opt._clear_optim_states()
    assert opt._stats_source() == ('launch', None) and opt._check_overflow() is False
    assert len(opt.state_dict()['state']) == len(params)


def test_every_optimizer_of_the_references_scaled_list_is_here():
    """optimizer.py:19 lists the optimizers that may be handed a ``div_scale``: FusedAdam, CPUAdam and
    HybridAdam.  All three exist with ColossalAI's argument order, count as scaled optimizers inside the
    wrapper, and keep their step out of torch's profiling wrapper."""
    import inspect
    from elixir_amd.optimizer import _AVAIL_OPTIM_LIST
    assert _AVAIL_OPTIM_LIST == {ea.FusedAdam, ea.CPUAdam, ea.HybridAdam}
    assert list(inspect.signature(ea.FusedAdam.__init__).parameters)[1:] == [
        'params', 'lr', 'bias_correction', 'betas', 'eps', 'adamw_mode', 'weight_decay', 'amsgrad', 'set_grad_none']
    assert list(inspect.signature(ea.FusedAdam.step).parameters)[1:7] == [
        'closure', 'grads', 'output_params', 'scale', 'grad_norms', 'div_scale']
    assert list(inspect.signature(ea.CPUAdam.__init__).parameters)[1:10] == [
        'model_params', 'lr', 'bias_correction', 'betas', 'eps', 'weight_decay', 'adamw_mode', 'nvme_offload_fraction',
        'nvme_offload_dir']
    assert list(inspect.signature(ea.CPUAdam.step).parameters)[1:3] == ['closure', 'div_scale']
    p = nn.Parameter(torch.zeros(4))
    p.grad = torch.ones(4)
    # positional use as in ColossalAI: the sixth argument of FusedAdam is adamw_mode, of CPUAdam weight_decay
    fused = ea.FusedAdam([p], 1e-3, True, (0.9, 0.999), 1e-8, False, 0.1)
    assert fused.adamw_mode is False and fused.param_groups[0]['weight_decay'] == 0.1
    cpu = ea.CPUAdam([p], 1e-3, True, (0.9, 0.999), 1e-8, 0.1, False)
    assert cpu.adamw_mode is False and cpu.param_groups[0]['weight_decay'] == 0.1
    with pytest.raises(RuntimeError, match='AMSGrad'):
        ea.FusedAdam([p], amsgrad=True)
    with pytest.raises(RuntimeError, match='no arguments'):
        fused.step(grads=[p.grad])
    for opt in (fused, cpu):
        assert getattr(type(opt).step, 'hooked', False) and not hasattr(type(opt).step, '__wrapped__')
        with pytest.raises(RuntimeError, match='GPU'):    # no device here, and no other way to step
            opt.step(div_scale=2.0)
    fused.zero_grad()
    assert p.grad is None
    p.grad = torch.ones(4)
    ea.FusedAdam([p], set_grad_none=False).zero_grad()
    assert p.grad is not None and float(p.grad.sum()) == 0.0
    for cls in (ea.FusedAdam, ea.CPUAdam):
        module, _ = _cpu_optimizer(3)
        wrapped = ea.ElixirOptimizer(module, cls(module.parameters(), lr=1e-3), initial_scale=64)
        assert wrapped.scaled_optimizer and wrapped._binding is not None


def test_chunk_cpu_copy_and_load_tensors():
    a, b = torch.randn(3, 5), torch.randn(7)
    chunk = ea.Chunk(None, 32, torch.float, None, shard_device='cpu', temp_device='cpu')
    chunk.append_tensor(a)
    chunk.append_tensor(b)
    chunk.close_chunk()
    ca, cb = chunk.get_cpu_copy()
    assert ca.shape == (3, 5) and cb.shape == (7,)
    assert torch.equal(ca.flatten(), chunk.shard[:15]) and torch.equal(cb, chunk.shard[15:22])
    new_b = torch.arange(7.0)
    chunk.load_tensors([None, new_b])
    assert torch.equal(chunk.shard[:15], ca.flatten()) and torch.equal(chunk.shard[15:22], new_b)
    assert torch.count_nonzero(chunk.shard[22:]) == 0


def test_launch_plan_properties_random():
    """Whatever the buffers and segments: update rows + refresh rows tile every buffer exactly once,
    every segment element appears in exactly one row segment with its hyper index, and the tables
    pass the library's own validation."""
    from hypothesis import given, settings, strategies as st
    from elixir_amd.launch_plan import FlatBuffer, build_plan
    import elixir_amd.launch_plan as LP

    @st.composite
    def buffers(draw):
        out = []
        for k in range(draw(st.integers(1, 4))):
            n_alloc = draw(st.integers(1, 300_000))
            n_valid = draw(st.integers(0, n_alloc))
            cuts = sorted(set(draw(st.lists(st.integers(0, n_valid), max_size=8)) + [0, n_valid]))
            segs = []
            for a, b in zip(cuts, cuts[1:]):
                if b > a and draw(st.booleans()):
                    lo = draw(st.integers(a, b - 1))
                    segs.append((lo, b, draw(st.integers(0, 2))))
            base = (k + 1) << 36
            lowp = draw(st.booleans())
            out.append(FlatBuffer(grad=base, lowp_out=base if lowp else 0, master=base + (1 << 32), m=base + (2 << 32),
                                  v=base + (3 << 32), n_alloc=n_alloc, n_valid=n_valid, segs=segs))
        if any(b.lowp_out for b in out):    # one launch has one low-precision type: all or none
            for b in out:
                b.lowp_out = b.grad
        return out

    @settings(max_examples=60, deadline=None, derandomize=True, database=None)
    @given(buffers(), st.sampled_from([16, 64, 2048]))
    def check(bufs, block_tiles):
        LP.BLOCK_TILES = block_tiles
        try:
            lowp = _abi.ELX_F16 if bufs[0].lowp_out else _abi.ELX_NONE
            plan = build_plan(bufs, 2, 2, 3, _abi.ELX_F16, lowp)
        finally:
            LP.BLOCK_TILES = 2048
        B = plan.block_elems
        for buf in bufs:
            rows = [r for r in plan.rows if buf.master <= r['master'] < buf.master + 4 * buf.n_alloc]
            rows.sort(key=lambda r: r['master'])
            pos = 0
            seen = {}
            for r in rows:
                b = (int(r['master']) - buf.master) // 4
                assert b == pos and b % B == 0 and 0 < r['n_alloc'] <= B
                assert r['n_valid'] == max(0, min(int(r['n_alloc']), buf.n_valid - b))
                prev = 0
                for sg in plan.segs[r['seg_begin']:r['seg_end']]:
                    assert prev <= sg['begin'] < sg['end'] <= r['n_valid']
                    prev = int(sg['end'])
                    for e in (int(sg['begin']), int(sg['end']) - 1):
                        seen[b + e] = int(sg['hyper'])
                pos += int(r['n_alloc'])
            up_end = pos
            assert up_end >= buf.n_valid and (up_end == buf.n_alloc or up_end % B == 0)
            if plan.refresh_rows is not None and buf.lowp_out:
                # the padding run behind the update rows is tiled by refresh rows of at most one block
                tail = sorted((int(r['master']), int(r['n_alloc'])) for r in plan.refresh_rows
                              if buf.master + 4 * up_end <= r['master'] < buf.master + 4 * buf.n_alloc)
                at = buf.master + 4 * up_end
                for addr, cnt in tail:
                    assert addr == at and 0 < cnt <= B
                    at += 4 * cnt
                assert at == buf.master + 4 * buf.n_alloc
            else:
                assert up_end == buf.n_alloc or not buf.lowp_out
            for sb, se, h in buf.segs:    # the ends of every segment are covered with the right hyper index
                assert seen.get(sb) == h and seen.get(se - 1) == h
        covered = sum(int(s['end'] - s['begin']) for s in plan.segs)
        assert covered == sum(se - sb for buf in bufs for sb, se, _ in buf.segs)

    check()


def test_stats_arena_hands_out_runs_and_takes_them_back(monkeypatch):
    """Slots of the record arena: consecutive runs in list order, kept when a list lands again, given
    back when a chunk moves to another run or is garbage-collected, and a clear error when no run is
    free.  (The arena's buffer sits on the CPU here; nothing is launched.)"""
    import gc
    from elixir_amd.chunk import StatsArena
    assert StatsArena.CAPACITY == 65535                      # as many chunks as one launch takes rows
    monkeypatch.setattr(StatsArena, 'CAPACITY', 4096)        # a small one, so that the churn below outnumbers it

    def chunk():
        c = ea.Chunk(None, 64, torch.float16, None, shard_device='cpu', temp_device='cpu')
        c.append_tensor(torch.zeros(8).half())
        c.close_chunk()
        return c

    arena = StatsArena(torch.device('cpu'))
    a, b, c = chunk(), chunk(), chunk()
    arena.assign([a, b])
    assert (a._stats_slot, b._stats_slot) == (0, 1)
    arena.assign([a, b])                                     # the same list again: nothing moves
    assert (a._stats_slot, b._stats_slot) == (0, 1) and arena.used.sum() == 2
    arena.assign([b, c])                                     # b moves next to c; its old slot is free again
    assert (b._stats_slot, c._stats_slot) == (2, 3) and list(np.flatnonzero(arena.used)) == [0, 2, 3]
    arena.assign([a])
    assert a._stats_slot == 0
    arena.assign([a, b, c])                                  # a fresh run of three; 0, 2, 3 come back
    assert [x._stats_slot for x in (a, b, c)] == [4, 5, 6] and list(np.flatnonzero(arena.used)) == [4, 5, 6]
    d = chunk()
    arena.assign([d])
    assert d._stats_slot == 0                                # first fit reuses what was released
    del d
    gc.collect()
    assert list(np.flatnonzero(arena.used)) == [4, 5, 6]     # a dead chunk gives its slot back
    # churn: far more chunks over time than the arena has slots
    for _ in range(3 * StatsArena.CAPACITY // 4):
        xs = [chunk() for _ in range(4)]
        arena.assign(xs)
        del xs
    gc.collect()
    assert arena.used.sum() == 3
    with pytest.raises(RuntimeError, match='free stats slots'):
        arena.new_slots(StatsArena.CAPACITY - 2)
    first = arena.new_slots(StatsArena.CAPACITY - 7)         # the longest free run is behind slot 6
    assert first == 7
